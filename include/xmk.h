/*
 * xmk.h — C ABI of the MI355X (gfx950) kernels behind the XLA custom calls
 *         "__cublas$gemm", "__cublas$lt$matmul", "__cudnn$fmhaSoftmax",
 *         "__cudnn$fmhaScaleBiasSoftmax" and the two weight-quantised targets
 *         this library adds ("__xmk$int4_gemm", "__cublas$lt$matmul$f8").
 *
 * Plain pointers and sizes only.  Every `stream` argument is a hipStream_t
 * passed as void* (NULL = the null stream).  Every entry point enqueues work
 * on that stream and returns; none synchronises the device, none allocates
 * device memory, none frees or retains a caller's buffer.
 *
 * Return value: 0 on success, otherwise an absl::StatusCode-compatible code
 * (see xmk_status).  The message of the last failure on the calling thread is
 * returned by xmk_last_error().
 *
 * Reference interfaces replaced (paths relative to the reference tree):
 *   xla/service/gpu/sycl_custom_call.cc:154-226      FFI handlers (GEMM)
 *   xla/service/gpu/sycl_onednn.cc:38-54             RunGemmCustomCall
 *   xla/service/gpu/onednn_matmul_utils.h:35-73      epilogue enum + RunGemm
 *   xla/service/gpu/matrix_descriptor.h:30-46        MatrixDescriptor
 *   xla/service/gpu/xetla/gemm/gemm.h:57-108         XetlaGemmKernel builder
 *   xla/service/gpu/xetla/sdp/sdp_forward.h:22-36    fmha_forward_kernel_*
 *   xla/service/gpu/xetla_gpu_fused_mha_runner.h:36-41  RunXetlaGpuFMHA
 */
#ifndef XMK_H_
#define XMK_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes: the subset of absl::StatusCode the reference path returns
 * (onednn_matmul_utils.cc:322,334,613; xetla_gpu_fused_mha_runner.cc:60,145,217). */
typedef enum xmk_status {
  XMK_OK = 0,
  XMK_INVALID_ARGUMENT = 3,
  XMK_UNIMPLEMENTED = 12,
  XMK_INTERNAL = 13
} xmk_status;

/* Element types, numbered as xla::PrimitiveType (the values the reference's
 * attribute dictionary carries in "{lhs,rhs,output}_layout_dtype",
 * onednn_matmul_utils.cc:592-610). */
typedef enum xmk_dtype {
  XMK_S8 = 2,
  XMK_S32 = 4,
  XMK_F16 = 10,
  XMK_F32 = 11,
  XMK_BF16 = 16,
  XMK_F8E4M3FN = 20
} xmk_dtype;

/* Epilogues, numbered as SYCLGemm::GemmBackendEpilogue
 * (onednn_matmul_utils.h:35-45). */
typedef enum xmk_epilogue {
  XMK_EPI_DEFAULT = 0,
  XMK_EPI_RELU = 1,
  XMK_EPI_GELU = 2,
  XMK_EPI_BIAS = 3,
  XMK_EPI_BIAS_RELU = 4,
  XMK_EPI_BIAS_GELU = 5,
  XMK_EPI_GELU_AUX = 6,      /* rejected: XMK_UNIMPLEMENTED, as in the reference */
  XMK_EPI_BIAS_GELU_AUX = 7  /* rejected: XMK_UNIMPLEMENTED, as in the reference */
} xmk_epilogue;

/* Mirrors xla::gpu::MatrixDescriptor (matrix_descriptor.h:30-46) with the
 * device pointer flattened.  The buffer holds a row-major
 * [num_rows, num_cols] matrix whose rows are leading_dim_stride elements
 * apart; transpose != 0 means the operand of the product is the transpose of
 * that stored matrix (what GetMatrixDesc, onednn_matmul_utils.cc:206-218,
 * produces for a column-major layout). */
typedef struct xmk_matrix {
  void* data;
  int32_t transpose;
  int64_t num_rows;
  int64_t num_cols;
  int64_t batch_stride;       /* elements between consecutive batch members */
  int64_t leading_dim_stride; /* elements between consecutive stored rows */
} xmk_matrix;

/* One GEMM custom call, after the attribute dictionary has been decoded
 * (RunGemm, onednn_matmul_utils.cc:533-621):
 *     out = act(alpha * lhs·rhs + beta * c + bias)
 * computed with fp32 accumulation and one rounding to dtype_out.
 * c may alias out.data.  bias is a length-n vector of dtype_in or NULL.
 * Dtype triples accepted (onednn_matmul_utils.cc:605-610):
 *   (BF16,BF16,BF16) (F16,F16,F16) (BF16,BF16,F32) (F16,F16,F32) (F32,F32,F32). */
typedef struct xmk_gemm_desc {
  xmk_matrix lhs;
  xmk_matrix rhs;
  xmk_matrix out;
  const void* c;     /* matrix addend, laid out like out; NULL iff beta == 0 */
  const void* bias;  /* vector addend; required iff the epilogue adds a bias */
  int32_t dtype_in;  /* xmk_dtype of lhs, rhs, bias */
  int32_t dtype_out; /* xmk_dtype of out and c */
  int64_t batch_size;
  float alpha;
  float beta;
  int32_t epilogue;  /* xmk_epilogue */
} xmk_gemm_desc;

/* Library version and the message of the calling thread's last failure. */
const char* xmk_version(void);
const char* xmk_last_error(void);

/* Replaces RunGemm (onednn_matmul_utils.h:58-73) and everything under it
 * (DoGemm :493-511, RunXetlaGemm :245-324, XetlaGemmKernel::run gemm.cc:315-325,
 * hgemm_* hgemm_impl.h:101-459).  The MFMA kernel takes the cases the
 * reference's XeTLA path takes (gemm.h:82-102: batch 1, alpha 1, A row-major,
 * 16-bit in == out type); every other accepted combination runs a generic
 * tiled kernel, where the reference falls back to oneDNN. */
int xmk_gemm(const xmk_gemm_desc* desc, void* stream);

/* xmk_gemm with caller-provided scratch (the reference's handlers receive a scratch allocator for
 * this purpose, sycl_custom_call.cc:155).  When the output has too few tiles to fill the device and K
 * is long (small-M decode shapes such as the 1_4096_4096 and 4_4096_16384 entries of the reference's
 * table, xetla/gemm/gemm.cc:32-37, which it runs with SLM_KS k-slicing), K is split over work-groups:
 * fp32 partial sums go to the workspace and a second kernel adds them in slice order and applies the
 * epilogue.  xmk_gemm_workspace_bytes returns the bytes that makes possible for this descriptor
 * (0: the call would not split).  With a NULL or too small workspace the call is xmk_gemm. */
size_t xmk_gemm_workspace_bytes(const xmk_gemm_desc* desc);
int xmk_gemm_ws(const xmk_gemm_desc* desc, void* workspace, size_t workspace_bytes, void* stream);

/* Three GEMMs that share the left operand: out_i = act(lhs · rhs_i + bias_i), i = q, k, v.
 * Replaces XetlaQKVGemmKernel (xetla/gemm/gemm.h:112-170) and hgemm_qkv / hgemm_qkv_bias
 * (xetla/gemm/hgemm_impl.h:461-608), which the reference launches as one kernel over a
 * 3 x tiles grid.  desc describes the first product: rhs.data is rhs_q and rhs.batch_stride
 * the distance in elements to rhs_k and from there to rhs_v (k*n when the three weights are
 * stacked, as the reference assumes, hgemm_impl.h:523-527); out.data is out_q, and out_k,
 * out_v are laid out like it; bias, when the epilogue adds one, holds the three vectors
 * stacked [3, n].  batch_size 1, beta 0, 16-bit dtype_in == dtype_out. */
int xmk_gemm_qkv(const xmk_gemm_desc* desc, void* out_k, void* out_v, void* stream);

/* Name of the tile policy xmk_gemm would pick for (m, n, k): the counterpart
 * of selectXetlaGemmConfig (xetla/gemm/gemm.cc:286-308).  Returns a static
 * string: "mfma_<BM>x<BN>x<BK>_..." for a matrix-core tile,
 * "stream_rows_8x512_w8" for the streaming kernels that a few rows against
 * a wide matrix take, in either storage order of B (packed, aligned
 * operands assumed). */
const char* xmk_gemm_policy_name(int64_t m, int64_t n, int64_t k, int32_t rhs_transpose,
                                 int32_t dtype_in, int32_t dtype_out);

/* Fused multi-head-attention forward.  Replaces fmha_forward_kernel_fp16 /
 * _bf16 (xetla/sdp/sdp_forward.h:22-36; same argument meaning and order apart
 * from the queue becoming a trailing stream, the dtype becoming an argument,
 * dropout being dropped because the reference rejects it
 * (xetla_gpu_fused_mha_runner.cc:59-61), and `causal` being a run-time flag
 * where the reference hard-codes false, sdp_forward.cc:41).
 *   query [B,N,F,H], key [B,N,T,H], value [B,N,T,H], out [B,N,F,H], all
 *   H-contiguous and packed; bias [B,N,F,T] of the same dtype or NULL
 *   (added after scaling, fmha_forward.h:266-281); lse fp32 [B*N,F] or NULL
 *   (written as m + log l, fmha_forward.h:433-450).
 *   causal != 0 masks key x > query y, top-left aligned (fmha_utils.h:45-96).
 * dtype is XMK_F16 or XMK_BF16; 1 <= H <= 256. */
int xmk_fmha_fwd(const void* query, const void* key, const void* value, const void* bias,
                 void* out, float* lse, int32_t dtype, uint32_t num_batches,
                 uint32_t num_heads, uint32_t head_size, uint32_t num_queries,
                 uint32_t num_keys, float head_scale, int32_t causal, void* stream);

/* Bytes of device workspace xmk_fmha_bwd needs for the given shape. */
size_t xmk_fmha_bwd_workspace_bytes(uint32_t num_batches, uint32_t num_heads, uint32_t head_size,
                                    uint32_t num_queries, uint32_t num_keys);

/* Fused multi-head-attention backward.  Replaces fmha_backward_kernel_fp16 / _bf16
 * (xetla/sdp/sdp_backward.h:22-36; same tensors, with the reference's two scratch arguments
 * dp_sum and grad_query_accum folded into one workspace, the dtype and `causal` as arguments).
 *   query, key, value, bias, out as in xmk_fmha_fwd; grad_out [B,N,F,H]; lse fp32 [B*N,F] as
 *   written by xmk_fmha_fwd; grad_query [B,N,F,H], grad_key and grad_value [B,N,T,H] of dtype.
 * No gradient is produced for the bias (the reference passes d_bias but never writes it,
 * xetla_gpu_fused_mha_runner.cc:383-385).  workspace: 256-byte aligned device memory of at least
 * xmk_fmha_bwd_workspace_bytes() bytes. */
int xmk_fmha_bwd(const void* query, const void* key, const void* value, const void* bias,
                 const void* out, const void* grad_out, const float* lse, void* grad_query,
                 void* grad_key, void* grad_value, int32_t dtype, uint32_t num_batches,
                 uint32_t num_heads, uint32_t head_size, uint32_t num_queries, uint32_t num_keys,
                 float head_scale, int32_t causal, void* workspace, size_t workspace_bytes,
                 void* stream);

/* Bytes of device workspace xmk_fmha_decode needs for the given shape. */
size_t xmk_fmha_decode_workspace_bytes(uint32_t num_batches, uint32_t num_heads,
                                       uint32_t head_size, uint32_t num_keys);

/* Bytes of workspace that serve xmk_fmha_decode for EVERY num_keys in 1..cache_capacity (the split
 * count is not monotonic in num_keys): what a caller that allocates once for a KV cache asks for. */
size_t xmk_fmha_decode_cache_workspace_bytes(uint32_t num_batches, uint32_t num_heads,
                                             uint32_t head_size, uint32_t cache_capacity);

/* Attention for one query row per (batch, head) (num_queries == 1), with the
 * keys split over work-groups and merged by a second pass.  Same tensors as
 * xmk_fmha_fwd with F = 1; key/value may sit in a cache whose rows per head
 * are kv_head_stride elements apart (>= T*H).  The reference has no such
 * kernel: it would run fmha_forward with a 64-row tile (fmha_forward.h:633-640). */
int xmk_fmha_decode(const void* query, const void* key, const void* value, void* out,
                    int32_t dtype, uint32_t num_batches, uint32_t num_heads,
                    uint32_t head_size, uint32_t num_keys, int64_t kv_head_stride,
                    float head_scale, void* workspace, size_t workspace_bytes, void* stream);

/* xmk_fmha_decode for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): no workspace argument; the partial results of the
 * key splits go to an array that is part of the library image on each GPU (4 MiB per GPU, held from
 * the first call there until the process ends).  No counterpart in the reference.  Calls neither
 * hipMalloc / hipFree nor any allocating routine; results equal xmk_fmha_decode's bit for bit.  Shapes
 * whose xmk_fmha_decode_workspace_bytes() exceeds xmk_fmha_decode_static_max_bytes() are rejected with
 * XMK_INVALID_ARGUMENT.  All calls on one GPU share that GPU's array: calls that overlap in time on
 * one GPU (different streams, or threads) race; calls ordered on one stream are safe.  The device
 * the stream belongs to must be the calling thread's current device.
 * The first call on a device looks up the array's device address (hipGetSymbolAddress), which makes
 * the runtime load the library's code object there if it has not yet: not something to do under
 * stream capture.  xmk_fmha_decode_static_init() does that lookup for the calling thread's current
 * device and nothing else; call it (or make one ordinary call) on each device before capturing. */
size_t xmk_fmha_decode_static_max_bytes(void);
int xmk_fmha_decode_static_init(void);
int xmk_fmha_decode_static(const void* query, const void* key, const void* value, void* out,
                           int32_t dtype, uint32_t num_batches, uint32_t num_heads,
                           uint32_t head_size, uint32_t num_keys, int64_t kv_head_stride,
                           float head_scale, void* stream);

/* Int4 weight-only GEMM (not in the reference snapshot; the contract is this
 * header's):
 *   qweight int32 [K/8, N]: nibble j (bits 4j..4j+3) of qweight[r, n] is the
 *     unsigned 4-bit weight of input channel k = 8r + j, output channel n;
 *   scales, zeros fp16 [K/group, N];
 *   w[k, n] = (float(q) - float(zeros[k/group, n])) * float(scales[k/group, n])
 *     with a separate fp32 subtract and fp32 multiply;
 *   W[k, n] = fp16(w[k, n]), rounded to nearest even, is what xmk_int4_dequant writes;
 *   out[m, n] = fp16( sum_k float(act[m, k]) * w[k, n] + float(bias[n]) ),
 *     fp32 accumulation, no intermediate rounding of w to fp16; bias fp16 [N] or NULL.
 * act fp16 [M, K] packed, out fp16 [M, N] packed.  K % group == 0, N % 8 == 0;
 * group is 32, 64, 128 or 256 for xmk_int4_gemm and any multiple of 8 for
 * xmk_int4_dequant. */
int xmk_int4_gemm(const void* act, const void* qweight, const void* scales, const void* zeros,
                  const void* bias, void* out, int64_t m, int64_t k, int64_t n,
                  int64_t group, void* stream);

/* xmk_int4_gemm for many rows (prompt processing) with caller-provided scratch: when
 * xmk_int4_gemm_workspace_bytes(m, k, n) is not 0 and the workspace (16-byte aligned) holds that many
 * bytes, W = xmk_int4_dequant(...) is written to it once and out = fp16(act . W + bias) runs on the dense
 * fp16 GEMM, so w IS rounded to fp16 on this path (a relative 2^-11 per weight, inside the tolerance of
 * the direct kernel).  Otherwise the call is xmk_int4_gemm.  Not in the reference snapshot. */
size_t xmk_int4_gemm_workspace_bytes(int64_t m, int64_t k, int64_t n);
int xmk_int4_gemm_ws(const void* act, const void* qweight, const void* scales, const void* zeros,
                     const void* bias, void* out, int64_t m, int64_t k, int64_t n, int64_t group,
                     void* workspace, size_t workspace_bytes, void* stream);

/* The dequantised weight matrix itself, fp16 [K, N]: the bit-exact check
 * surface for the formula above. */
int xmk_int4_dequant(const void* qweight, const void* scales, const void* zeros, void* w_out,
                     int64_t k, int64_t n, int64_t group, void* stream);

/* FP8 GEMM (not in the reference snapshot; follows XLA's
 * "__cublas$lt$matmul$f8" convention):
 *   out[m, n] = bf16( a_scale * b_scale * sum_k float(a[m,k]) * float(b) ), fp32 accumulate.
 * a e4m3fn [M, K] row-major; b e4m3fn, [K, N] row-major when
 * rhs_transpose == 0 or [N, K] row-major when rhs_transpose != 0;
 * a_scale, b_scale device pointers to one fp32 each; out bf16 [M, N]. */
int xmk_fp8_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale,
                 void* out, int64_t m, int64_t n, int64_t k, int32_t rhs_transpose,
                 void* stream);

/* The same product with the rest of the "__cublas$lt$matmul$f8" operand list applied on the device:
 * out = bf16(d_scale * (a_scale * b_scale * A B + bias)).  d_scale (device fp32 scalar) and bias
 * (bf16 [N]) may each be NULL.  The reference's handlers use every operand they are handed
 * (xla/service/gpu/sycl_custom_call.cc:168-205); this is the entry point the f8 handler calls. */
int xmk_fp8_gemm_ex(const void* a, const void* b, const float* a_scale, const float* b_scale,
                    const float* d_scale, const void* bias, void* out, int64_t m, int64_t n,
                    int64_t k, int32_t rhs_transpose, void* stream);

/* ------------------------------------------------------------------------
 * GPT-J-shaped decode step on int4 weights: one new token per sequence through
 * n_layer blocks, reading the KV cache of the earlier positions.  The model the
 * reference runs for this workload is FlaxGPTJForCausalLM under jax.jit
 * (example/gptj/jax_gptj.py:57-68,94-97), with dense weights; the block structure
 * restated here is GPT-J's: h = ln_1(x); x' = x + out_proj(attn(rotary(q), rotary(k), v))
 * + fc_out(gelu_new(fc_in(h))); q/k/v/out_proj without bias, fc_in/fc_out/lm_head with
 * bias; rotary on the first rotary_dim dims of each head, interleaved pairs, base 10000;
 * scores scaled by 1/sqrt(head_dim); final ln_f then lm_head. */
typedef struct xmk_int4_linear {
  const void* qweight; /* int32 [k/8, n] */
  const void* scales;  /* fp16 [k/group, n] */
  const void* zeros;   /* fp16 [k/group, n] */
  const void* bias;    /* fp16 [n] or NULL */
  int64_t k, n;
} xmk_int4_linear;

typedef struct xmk_gptj_layer {
  const void* ln_gamma; /* fp16 [d_model] */
  const void* ln_beta;  /* fp16 [d_model] */
  xmk_int4_linear qkv;      /* d_model -> 3 d_model, output columns [q | k | v], no bias */
  xmk_int4_linear out_proj; /* d_model -> d_model, no bias */
  xmk_int4_linear fc_in;    /* d_model -> d_ff, bias */
  xmk_int4_linear fc_out;   /* d_ff -> d_model, bias */
  void* k_cache; /* fp16 [batch, n_head, cache_capacity, head_dim]; row `position` is written */
  void* v_cache; /* same */
} xmk_gptj_layer;

typedef struct xmk_gptj_config {
  int32_t n_layer, n_head, head_dim, rotary_dim, d_model, d_ff, vocab, group;
  int32_t batch, cache_capacity;
  float ln_eps;
} xmk_gptj_config;

size_t xmk_gptj_decode_workspace_bytes(const xmk_gptj_config* cfg);

/* hidden_in fp16 [batch, d_model] (the new token's embedding); position = index of the new
 * token (the caches hold positions 0..position-1); logits fp16 [batch, vocab].
 * Enqueues every kernel of the step on `stream` in order; a caller may capture the call in a
 * HIP graph. */
int xmk_gptj_decode_step(const xmk_gptj_config* cfg, const xmk_gptj_layer* layers,
                         const void* lnf_gamma, const void* lnf_beta,
                         const xmk_int4_linear* lm_head, const void* hidden_in, int32_t position,
                         void* logits, void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* XMK_H_ */
