// Multi-head attention backward: entry point, D = rowsum(dO o O), and the second implementation beside
// the fused kernels (fmha_bwd_fused.hip), selected with XMK_FMHA_BWD_COMPOSED=1 -- a composition of the batched
// MFMA GEMM and two elementwise passes over the score matrix, for a chunk of (batch, head) units at a time:
//     D   = rowsum(dO o O)                          (dp_sum, fmha_backward.h:48)
//     S   = Q K^T                    fp32           (GEMM)
//     P   = exp(scale S + bias - LSE), masked       (elementwise, rounded to the operand type)
//     dV  = P^T dO                                  (GEMM)
//     dP  = dO V^T                   fp32           (GEMM, overwrites S)
//     dS  = scale P o (dP - D)                      (elementwise, overwrites P)
//     dQ  = dS K,   dK = dS^T Q                     (GEMMs)
// The score-sized intermediates live in caller-provided workspace (the reference's backward
// also takes its scratch, dp_sum and grad_query_accum, from the caller:
// xetla_gpu_fused_mha_runner.cc:331-339); the chunk size bounds them.  No gradient is produced
// for the bias, as in the reference (xetla_gpu_fused_mha_runner.cc:383-385).
#include <cstdlib>

#include "common.h"
#include "fmha_bwd_fused.h"

namespace {

constexpr size_t kChunkBytes = (size_t)1 << 30;  // score-sized intermediates per chunk, at most

// D[row] = sum_h O[row][h] dO[row][h].  H % 8 == 0: a lane reads 8 elements (16 bytes) of each tensor;
// LPR lanes (a power of two >= H / 8) share a row and a wave covers 64 / LPR rows.
// With lse2 != NULL it also writes lse2[row] = lse[row] * log2(e), the form the fused kernels use in their
// exponentials (one multiplication per row here instead of one per score there).
template <typename T, int LPR>
__global__ __launch_bounds__(256) void dp_sum_kernel(const T* __restrict__ o, const T* __restrict__ d_o,
                                                     float* __restrict__ dsum, int64_t rows, int H,
                                                     const float* __restrict__ lse, float* __restrict__ lse2) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  constexpr int RPW = 64 / LPR;
  const int lane = threadIdx.x & 63;
  const int64_t row = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * RPW + lane / LPR;
  const int c = (lane % LPR) * 8;
  float s = 0.f;
  if (row < rows && c < H) {
    const u32x4 a = *reinterpret_cast<const u32x4*>(o + row * H + c);
    const u32x4 b = *reinterpret_cast<const u32x4*>(d_o + row * H + c);
    const T* ae = reinterpret_cast<const T*>(&a);
    const T* be = reinterpret_cast<const T*>(&b);
#pragma unroll
    for (int j = 0; j < 8; ++j) s += (float)ae[j] * (float)be[j];
  }
#pragma unroll
  for (int off = LPR / 2; off >= 1; off >>= 1) s += __shfl_xor(s, off);
  if (row < rows && lane % LPR == 0) {
    dsum[row] = s;
    if (lse2) lse2[row] = lse[row] * 1.4426950408889634f;
  }
}

// P[u, f, t] = exp(scale * S + bias - lse[f]); masked entries (causal: t > f) are zero.
// s32 / p: [units_in_chunk, F, ldT]; bias: [units, F, T] of the whole problem or null.
template <typename T>
__global__ __launch_bounds__(256) void probs_kernel(const float* __restrict__ s32, const T* __restrict__ bias,
                                                    const float* __restrict__ lse, T* __restrict__ p, int F, int Tk,
                                                    int ldT, int64_t unit0, float scale, int causal) {
  const int64_t row = blockIdx.x;  // (unit in chunk) * F + f
  const int f = (int)(row % F);
  const int64_t grow = unit0 * F + row;
  const float l = lse[grow];
  const float* sr = s32 + row * ldT;
  const T* br = bias ? bias + grow * Tk : nullptr;
  T* pr = p + row * ldT;
  for (int t = threadIdx.x; t < ldT; t += 256) {
    float v = 0.f;
    if (t < Tk && !(causal && t > f)) {
      float x = sr[t] * scale;
      if (br) x += (float)br[t];
      v = __expf(x - l);
    }
    pr[t] = (T)v;  // padding columns (t >= Tk) are written as zero: they enter the GEMMs' k loops
  }
}

// dS = scale * P * (dP - D[f]), in place over P.
template <typename T>
__global__ __launch_bounds__(256) void dscore_kernel(const float* __restrict__ dp32, const float* __restrict__ dsum,
                                                     T* __restrict__ p, int F, int Tk, int ldT, int64_t unit0,
                                                     float scale) {
  const int64_t row = blockIdx.x;
  const float d = dsum[unit0 * F + row];
  const float* dr = dp32 + row * ldT;
  T* pr = p + row * ldT;
  for (int t = threadIdx.x; t < Tk; t += 256) pr[t] = (T)(scale * (float)pr[t] * (dr[t] - d));
}

struct Plan {
  int64_t ldT;          // padded row length of the score-sized buffers (elements)
  int64_t chunk;        // units per chunk
  size_t off_s, off_p;  // byte offsets of the fp32 and the 16-bit score buffers; dsum is at 0
  size_t total;
};

Plan make_plan(uint64_t units, uint64_t F, uint64_t T) {
  Plan p;
  p.ldT = (int64_t)((T + 7) / 8 * 8);
  const size_t per_unit = (size_t)F * p.ldT * 6;  // fp32 + 16-bit
  p.chunk = (int64_t)(kChunkBytes / (per_unit ? per_unit : 1));
  if (p.chunk < 1) p.chunk = 1;
  if ((uint64_t)p.chunk > units) p.chunk = (int64_t)units;
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  p.off_s = up((size_t)units * F * sizeof(float));
  p.off_p = p.off_s + up((size_t)p.chunk * F * p.ldT * sizeof(float));
  p.total = p.off_p + up((size_t)p.chunk * F * p.ldT * 2);
  return p;
}

xmk_matrix mat(const void* data, int transpose, int64_t rows, int64_t cols, int64_t batch_stride, int64_t ld) {
  xmk_matrix m;
  m.data = const_cast<void*>(data);
  m.transpose = transpose;
  m.num_rows = rows;
  m.num_cols = cols;
  m.batch_stride = batch_stride;
  m.leading_dim_stride = ld;
  return m;
}

int gemm(const xmk_matrix& lhs, const xmk_matrix& rhs, const xmk_matrix& out, int dtype_in, int dtype_out,
         int64_t batch, void* stream) {
  xmk_gemm_desc d;
  d.lhs = lhs; d.rhs = rhs; d.out = out;
  d.c = nullptr; d.bias = nullptr;
  d.dtype_in = dtype_in; d.dtype_out = dtype_out;
  d.batch_size = batch;
  d.alpha = 1.0f; d.beta = 0.0f;
  d.epilogue = XMK_EPI_DEFAULT;
  return xmk_gemm(&d, stream);
}

// Whether the fused kernels take the call (they need only the rowsum(dO o O) part of the workspace).
// A bias is assumed when `bias` is unknown (the workspace query): its size only tightens the test.
bool fused_path(uint64_t units, uint32_t H, uint32_t F, uint32_t T, bool maybe_bias) {
  static const bool composed = getenv("XMK_FMHA_BWD_COMPOSED") != nullptr;
  if (composed) return false;
  fmha_bwd_fused::Args a{};
  a.H = (int)H; a.F = (int)F; a.T = (int)T;
  a.bias = maybe_bias ? &a : nullptr;  // any non-null value: only its presence is looked at
  return fmha_bwd_fused::eligible(a, units);
}

size_t dsum_bytes(uint64_t units, uint64_t F) { return ((size_t)units * F * sizeof(float) + 255) & ~(size_t)255; }
// Scratch of the fused path: rowsum(dO o O), then LSE * log2(e), one float per query row each.
size_t fused_bytes(uint64_t units, uint64_t F) { return 2 * dsum_bytes(units, F); }

template <typename T>
int run(const void* q, const void* k, const void* v, const void* bias, const void* o, const void* d_o,
        const float* lse, void* dq, void* dk, void* dv, int dtype, int64_t units, int64_t H, int64_t F, int64_t Tk,
        float scale, int causal, char* ws, const Plan& pl, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  float* dsum = reinterpret_cast<float*>(ws);
  float* s32 = reinterpret_cast<float*>(ws + pl.off_s);
  T* p = reinterpret_cast<T*>(ws + pl.off_p);
  const T* Q = (const T*)q; const T* K = (const T*)k; const T* V = (const T*)v; const T* dO = (const T*)d_o;
  T* dQ = (T*)dq; T* dK = (T*)dk; T* dV = (T*)dv;
  const int64_t rows = units * F;
  const bool fused = fused_path((uint64_t)units, (uint32_t)H, (uint32_t)F, (uint32_t)Tk, bias != nullptr);
  float* lse2 = reinterpret_cast<float*>(ws + dsum_bytes((uint64_t)units, (uint64_t)F));  // fused path only
  // The gradients come from the fused kernels, which keep the scores on chip and form the two per-row
  // statistics (D, LSE log2(e)) themselves; XMK_FMHA_BWD_COMPOSED=1 forces the GEMM composition below.
  if (fused) {
    const fmha_bwd_fused::Args a{q, k, v, d_o, o, bias, lse, lse2, dsum, dq, dk, dv, (int)H, (int)F, (int)Tk, scale, causal != 0};
    fmha_bwd_fused::launch(a, (uint64_t)units, dtype == XMK_BF16, st);
    return xmk::check_launch("fmha_bwd");
  }
  if (H <= 64)
    hipLaunchKernelGGL((dp_sum_kernel<T, 8>), dim3((unsigned)xmk::ceil_div(rows, 32)), dim3(256), 0, st, (const T*)o, dO,
                       dsum, rows, (int)H, (const float*)nullptr, (float*)nullptr);
  else if (H <= 128)
    hipLaunchKernelGGL((dp_sum_kernel<T, 16>), dim3((unsigned)xmk::ceil_div(rows, 16)), dim3(256), 0, st, (const T*)o, dO,
                       dsum, rows, (int)H, (const float*)nullptr, (float*)nullptr);
  else
    hipLaunchKernelGGL((dp_sum_kernel<T, 32>), dim3((unsigned)xmk::ceil_div(rows, 8)), dim3(256), 0, st, (const T*)o, dO,
                       dsum, rows, (int)H, (const float*)nullptr, (float*)nullptr);
  const int64_t ldT = pl.ldT, sst = F * ldT;  // score buffers: row length, unit stride
  int rc;
  for (int64_t u0 = 0; u0 < units; u0 += pl.chunk) {
    const int64_t uc = units - u0 < pl.chunk ? units - u0 : pl.chunk;
    const T* Qc = Q + u0 * F * H; const T* Kc = K + u0 * Tk * H; const T* Vc = V + u0 * Tk * H;
    const T* dOc = dO + u0 * F * H;
    // S = Q K^T
    if ((rc = gemm(mat(Qc, 0, F, H, F * H, H), mat(Kc, 1, Tk, H, Tk * H, H), mat(s32, 0, F, Tk, sst, ldT), dtype,
                   XMK_F32, uc, stream)) != XMK_OK) return rc;
    hipLaunchKernelGGL(probs_kernel<T>, dim3((unsigned)(uc * F)), dim3(256), 0, st, (const float*)s32,
                       (const T*)bias, lse, p, (int)F, (int)Tk, (int)ldT, u0, scale, causal);
    // dV = P^T dO
    if ((rc = gemm(mat(p, 1, F, Tk, sst, ldT), mat(dOc, 0, F, H, F * H, H), mat(dV + u0 * Tk * H, 0, Tk, H, Tk * H, H),
                   dtype, dtype, uc, stream)) != XMK_OK) return rc;
    // dP = dO V^T (over S)
    if ((rc = gemm(mat(dOc, 0, F, H, F * H, H), mat(Vc, 1, Tk, H, Tk * H, H), mat(s32, 0, F, Tk, sst, ldT), dtype,
                   XMK_F32, uc, stream)) != XMK_OK) return rc;
    hipLaunchKernelGGL(dscore_kernel<T>, dim3((unsigned)(uc * F)), dim3(256), 0, st, (const float*)s32,
                       (const float*)dsum, p, (int)F, (int)Tk, (int)ldT, u0, scale);
    // dQ = dS K, dK = dS^T Q
    if ((rc = gemm(mat(p, 0, F, Tk, sst, ldT), mat(Kc, 0, Tk, H, Tk * H, H), mat(dQ + u0 * F * H, 0, F, H, F * H, H),
                   dtype, dtype, uc, stream)) != XMK_OK) return rc;
    if ((rc = gemm(mat(p, 1, F, Tk, sst, ldT), mat(Qc, 0, F, H, F * H, H), mat(dK + u0 * Tk * H, 0, Tk, H, Tk * H, H),
                   dtype, dtype, uc, stream)) != XMK_OK) return rc;
  }
  return xmk::check_launch("fmha_bwd");
}

int check_dims(uint32_t B, uint32_t N, uint32_t H, uint32_t F, uint32_t T) {
  if (B == 0 || N == 0 || H == 0 || F == 0 || T == 0)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_bwd: empty dimension");
  if (H > 256) return xmk::fail(XMK_UNIMPLEMENTED, "fmha_bwd: head_size %u > 256", H);
  if (H % 8 != 0) return xmk::fail(XMK_UNIMPLEMENTED, "fmha_bwd: head_size %u is not a multiple of 8", H);
  if ((uint64_t)B * N > 65535u * 64u || (uint64_t)F * T > ((uint64_t)1 << 40))
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_bwd: shape too large");
  return XMK_OK;
}

}  // namespace

extern "C" size_t xmk_fmha_bwd_workspace_bytes(uint32_t num_batches, uint32_t num_heads, uint32_t head_size,
                                               uint32_t num_queries, uint32_t num_keys) {
  if (check_dims(num_batches, num_heads, head_size, num_queries, num_keys) != XMK_OK) return 0;
  const uint64_t units = (uint64_t)num_batches * num_heads;
  // The fused kernels keep the scores on chip; only the GEMM composition needs the score-sized buffers.
  if (fused_path(units, head_size, num_queries, num_keys, true)) return fused_bytes(units, num_queries);
  return make_plan(units, num_queries, num_keys).total;
}

extern "C" int xmk_fmha_bwd(const void* query, const void* key, const void* value, const void* bias,
                            const void* out, const void* grad_out, const float* lse, void* grad_query,
                            void* grad_key, void* grad_value, int32_t dtype, uint32_t num_batches,
                            uint32_t num_heads, uint32_t head_size, uint32_t num_queries, uint32_t num_keys,
                            float head_scale, int32_t causal, void* workspace, size_t workspace_bytes,
                            void* stream) {
  if (!query || !key || !value || !out || !grad_out || !lse || !grad_query || !grad_key || !grad_value || !workspace)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_bwd: null pointer");
  if (dtype != XMK_F16 && dtype != XMK_BF16)
    return xmk::fail(XMK_INTERNAL, "Invalid MHA datatype");  // xetla_gpu_fused_mha_runner.cc:352
  int rc = check_dims(num_batches, num_heads, head_size, num_queries, num_keys);
  if (rc != XMK_OK) return rc;
  if (!(head_scale > 0.0f) || head_scale > 3.0e38f)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_bwd: head_scale must be positive and finite");
  const uint64_t units = (uint64_t)num_batches * num_heads;
  const Plan pl = make_plan(units, num_queries, num_keys);
  const size_t need = fused_path(units, head_size, num_queries, num_keys, bias != nullptr) ? fused_bytes(units, num_queries)
                                                                                          : pl.total;
  if (workspace_bytes < need)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_bwd: workspace of %zu bytes, %zu needed", workspace_bytes, need);
  if (pl.chunk > 65535) return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_bwd: shape too large");
  if (!xmk::aligned(workspace, 256) || !xmk::aligned(query, 16) || !xmk::aligned(key, 16) ||
      !xmk::aligned(value, 16) || !xmk::aligned(out, 16) || !xmk::aligned(grad_out, 16) ||
      !xmk::aligned(grad_query, 16) || !xmk::aligned(grad_key, 16) || !xmk::aligned(grad_value, 16))
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_bwd: tensors must be 16-byte and the workspace 256-byte aligned");
  xmk::trace("fmha_bwd B=%u N=%u F=%u T=%u H=%u causal=%d bias=%d chunk=%lld", num_batches, num_heads, num_queries,
             num_keys, head_size, causal, bias != nullptr, (long long)pl.chunk);
  if (dtype == XMK_BF16)
    return run<__bf16>(query, key, value, bias, out, grad_out, lse, grad_query, grad_key, grad_value, dtype,
                       (int64_t)units, head_size, num_queries, num_keys, head_scale, causal != 0, (char*)workspace, pl,
                       stream);
  return run<_Float16>(query, key, value, bias, out, grad_out, lse, grad_query, grad_key, grad_value, dtype,
                       (int64_t)units, head_size, num_queries, num_keys, head_scale, causal != 0, (char*)workspace, pl,
                       stream);
}
