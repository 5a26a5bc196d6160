// bf16 / fp16 GEMM with fp32 accumulation and a fused epilogue:
//     out = act(alpha * op(lhs) op(rhs) + beta * c + bias)
//
// MFMA kernel (gemm_mfma_kernel): one work-group owns a BM x BN tile of the output and walks K in
// steps of BK (32 for the 256x256 tile, 64 for the smaller ones).  Operand tiles go from global memory
// straight into LDS (buffer_load ... lds, 16 bytes per lane, no staging registers and no ds_write): a
// wave's load fills 1 KiB of contiguous LDS, and the per-lane *global* address is chosen so that the
// data lands swizzled.  A ring of three or four LDS stages; the loads of later K steps are issued
// between the MFMAs of step t and are waited for with a counted s_waitcnt at the one barrier per step.
//   "KC" operand (reduction index contiguous in memory: A[M,K] row-major, B stored [N,K]):
//       LDS [row][64 k], the 16-byte chunks of a row XOR-swizzled by the row number, read
//       with one ds_read_b128 per fragment.
//   "MC" operand (free index contiguous: B[K,N] row-major, A stored [K,M]):
//       LDS [k][cols], chunks XOR-swizzled by k, read with the LDS transpose loads
//       (ds_read_b64_tr_b16), which hand each lane four consecutive k of one column.
// The products are issued with the operands swapped (D^T = B^T A^T) so that a lane ends up
// holding four consecutive output columns of one row.
//
// 16-bit operands whose strides or sizes the direct loads cannot take run the same kernel with a
// gathering loader, fp32 operands the fp32 MFMA kernel (gemm_f32.hip), int8 operands the int8 MFMA
// kernel (gemm_s8.hip); what is left (outputs that are not 16-byte aligned) runs
// gemm_generic_kernel, a plain LDS-tiled kernel.  This is where
// the reference falls back to oneDNN (onednn_matmul_utils.cc:394-491).
#include "gemm_f32.h"
#include "gemm_kernel.h"
#include "gemm_rows.h"
#include "gemm_s8.h"

namespace {

using namespace gemm_impl;

// ------------------------------------------------------------------ generic kernel
// Any accepted dtype triple, any strides/transposes: 16x16 threads, 64x64 tile,
// operands converted to fp32 (or int32) while staging.
enum : int { G_BF16 = 0, G_F16 = 1, G_F32 = 2, G_S8 = 3, G_S32 = 4 };

__device__ __forceinline__ float load_as_f32(const void* p, int kind, int64_t i) {
  switch (kind) {
    case G_BF16: return (float)reinterpret_cast<const __bf16*>(p)[i];
    case G_F16: return (float)reinterpret_cast<const _Float16*>(p)[i];
    case G_S8: return (float)reinterpret_cast<const int8_t*>(p)[i];
    case G_S32: return (float)reinterpret_cast<const int32_t*>(p)[i];
    default: return reinterpret_cast<const float*>(p)[i];
  }
}

struct GenericParams {
  const void* a;
  const void* b;
  void* out;
  const void* c;
  const void* bias;
  int M, N, K;
  int64_t lda, ldb, ldc, sa, sb, sc;
  int ta, tb;  // operand is the transpose of the stored matrix
  int kin, kout;
  float alpha, beta;
  int act;
  void* out_alt[2];  // see GemmParams
  int64_t sbias;
};

__global__ __launch_bounds__(256) void gemm_generic_kernel(GenericParams p) {
  __shared__ float As[16][65];
  __shared__ float Bs[16][65];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int64_t bz = blockIdx.z;
  if (p.out_alt[0] && bz > 0) p.out = p.out_alt[bz - 1];
  const bool integer = p.kin == G_S8;
  float acc[4][4] = {};
  int iacc[4][4] = {};
  for (int k0 = 0; k0 < p.K; k0 += 16) {
    for (int e = threadIdx.x; e < 16 * 64; e += 256) {
      const int kk = e / 64, r = e % 64;
      const int k = k0 + kk;
      float av = 0.f, bv = 0.f;
      if (k < p.K && m0 + r < p.M) {
        const int64_t i = bz * p.sa + (p.ta ? (int64_t)k * p.lda + (m0 + r) : (int64_t)(m0 + r) * p.lda + k);
        av = load_as_f32(p.a, p.kin, i);
      }
      if (k < p.K && n0 + r < p.N) {
        const int64_t i = bz * p.sb + (p.tb ? (int64_t)(n0 + r) * p.ldb + k : (int64_t)k * p.ldb + (n0 + r));
        bv = load_as_f32(p.b, p.kin, i);
      }
      As[kk][r] = av;
      Bs[kk][r] = bv;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { a[i] = As[kk][ty * 4 + i]; b[i] = Bs[kk][tx * 4 + i]; }
      if (integer) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) iacc[i][j] += (int)a[i] * (int)b[j];
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= p.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= p.N) continue;
      const int64_t off = bz * p.sc + (int64_t)m * p.ldc + n;
      if (integer) {
        reinterpret_cast<int32_t*>(p.out)[off] = iacc[i][j];
        continue;
      }
      float v = p.alpha * acc[i][j];
      if (p.beta != 0.f && p.c) v += p.beta * load_as_f32(p.c, p.kout, off);
      if (p.bias) v += load_as_f32(p.bias, p.kin, bz * p.sbias + n);
      v = apply_act(v, p.act);
      switch (p.kout) {
        case G_BF16: reinterpret_cast<__bf16*>(p.out)[off] = (__bf16)v; break;
        case G_F16: reinterpret_cast<_Float16*>(p.out)[off] = (_Float16)v; break;
        default: reinterpret_cast<float*>(p.out)[off] = v; break;
      }
    }
  }
}

// Second pass of a K-split GEMM: out = act(alpha * sum_z partial[z] + beta * c + bias), one rounding.
// partial: fp32 [ks][M][N] packed; out / c: [M][ldc] of kind kout; bias of kind kin.
struct ReduceParams {
  const float* partial;
  void* out;
  const void* c;
  const void* bias;
  int M, N, ks;
  int64_t ldc;
  int kin, kout;
  float alpha, beta;
  int act;
};
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(ReduceParams p) {
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;  // four consecutive columns; N % 4 == 0
  const int64_t total = (int64_t)p.M * p.N;
  if (idx >= total) return;
  const int m = (int)(idx / p.N), n = (int)(idx % p.N);
  floatx4 s = {0.f, 0.f, 0.f, 0.f};
  for (int z = 0; z < p.ks; ++z) s += *reinterpret_cast<const floatx4*>(p.partial + (int64_t)z * total + idx);
  const int64_t off = (int64_t)m * p.ldc + n;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float v = p.alpha * s[j];
    if (p.beta != 0.f && p.c) v += p.beta * load_as_f32(p.c, p.kout, off + j);
    if (p.bias) v += load_as_f32(p.bias, p.kin, n + j);
    v = apply_act(v, p.act);
    switch (p.kout) {
      case G_BF16: reinterpret_cast<__bf16*>(p.out)[off + j] = (__bf16)v; break;
      case G_F16: reinterpret_cast<_Float16*>(p.out)[off + j] = (_Float16)v; break;
      default: reinterpret_cast<float*>(p.out)[off + j] = v; break;
    }
  }
}

// ------------------------------------------------------------------ host side

int generic_kind(int dtype) {
  switch (dtype) {
    case XMK_BF16: return G_BF16;
    case XMK_F16: return G_F16;
    case XMK_F32: return G_F32;
    case XMK_S8: return G_S8;
    case XMK_S32: return G_S32;
    default: return -1;
  }
}

int elem_size(int dtype) {
  switch (dtype) {
    case XMK_BF16: case XMK_F16: return 2;
    case XMK_F32: case XMK_S32: return 4;
    case XMK_S8: return 1;
    default: return 0;
  }
}

}  // namespace

extern "C" const char* xmk_gemm_policy_name(int64_t m, int64_t n, int64_t k, int32_t rhs_transpose,
                                            int32_t dtype_in, int32_t dtype_out) {
  const bool sixteen = dtype_in == XMK_BF16 || dtype_in == XMK_F16;
  if (dtype_in == XMK_F32 && dtype_out == XMK_F32) return "mfma_f32_128x128x16";
  if (dtype_in == XMK_S8 && dtype_out == XMK_S32) return "mfma_s8_128x128x64";
  if (!sixteen || !(dtype_out == dtype_in || dtype_out == XMK_F32)) return "generic_64x64";
  // (packed, aligned operands assumed, as everywhere in this query)
  int rows_kind = kRowsNone;
  if (m >= 1 && m <= kRowsMaxM && k % 8 == 0) {
    if (!rhs_transpose && n % 8 == 0) rows_kind = kRowsMC;
    if (rhs_transpose && k <= kColsMaxK) rows_kind = kRowsKC;
  }
  return kPolicies[select_policy(m, n, k, 1, rows_kind, !rhs_transpose)].name;
}

namespace {
// out1 / out2: further outputs of the shared-lhs three-GEMM form, or null for a plain GEMM.
// policy: tile policy to use instead of select_policy's choice (the K-split planner's), or -1.
int run_gemm(const xmk_gemm_desc* d, void* out1, void* out2, void* stream, int policy = -1);

// The conditions of the direct (non-gathering) 16-bit kernels on the stored operands.
bool direct_ok(const xmk_matrix& lhs, const xmk_matrix& rhs) {
  return xmk::aligned(lhs.data, 16) && xmk::aligned(rhs.data, 16) && lhs.leading_dim_stride % 8 == 0 &&
         rhs.leading_dim_stride % 8 == 0 && lhs.batch_stride % 8 == 0 && rhs.batch_stride % 8 == 0 &&
         lhs.num_cols % 8 == 0 && rhs.num_cols % 8 == 0;
}

// Which streaming kernel for a few rows (gemm_rows.hip) can run this descriptor's product, if any.
int rows_kind_desc(const xmk_gemm_desc* d, int64_t m, int64_t n, int64_t k) {
  if (d->out.transpose || d->lhs.transpose || !direct_ok(d->lhs, d->rhs) || !xmk::aligned(d->out.data, 16))
    return kRowsNone;
  if (d->dtype_in != XMK_BF16 && d->dtype_in != XMK_F16) return kRowsNone;
  GemmParams p{};
  p.M = (int)m; p.N = (int)n; p.K = (int)k;
  p.lda = d->lhs.leading_dim_stride; p.ldb = d->rhs.leading_dim_stride;
  return gemm_rows_applicable(p, false, d->rhs.transpose == 0);
}

// K slices worth using for a plain 16-bit GEMM of this shape when scratch is available: few
// output tiles (the device has 256 CUs) and a long reduction.  1: do not split.
// *policy: the tile policy of the slices (-1: whatever select_policy picks for a slice).
int plan_splitk(const xmk_gemm_desc* d, int64_t m, int64_t n, int64_t k, int* policy) {
  *policy = -1;
  if (d->batch_size != 1 || n % 4 != 0) return 1;
  if (d->dtype_in != XMK_BF16 && d->dtype_in != XMK_F16) return 1;
  auto divides = [&](int ks) { return ks >= 1 && ks <= 16 && k % (ks * 8) == 0; };
  // XMK_GEMM_SPLITK=<slices> overrides the choice (read at every call; the autotuner's handle).
  const char* forced_env = getenv("XMK_GEMM_SPLITK");
  const int forced = forced_env ? atoi(forced_env) : 0;
  if (forced >= 1) return divides(forced) ? forced : 1;
  const int rows_kind = (forced_policy() < 0 || forced_policy() == kRowsPolicy) ? rows_kind_desc(d, m, n, k) : kRowsNone;
  const bool rows_ok = rows_kind != kRowsNone;
  // (the table was measured with B stored [K, N])
  if (const TunedShape* t = tuned_shape(m, n, k); forced_policy() < 0 && !d->rhs.transpose && t && t->ksplit >= 1 && divides(t->ksplit) &&
                                                  (t->policy != kRowsPolicy || rows_ok)) {
    if (t->ksplit > 1) *policy = t->policy;
    return t->ksplit;
  }
  if (rows_streams_by_default(rows_kind, m, n)) return 1;  // streamed in one launch
  if (rows_ok && forced_policy() == kRowsPolicy) {
    // The streaming kernel forced on a narrower matrix (tests, the autotuner): slices until its narrowest
    // column blocks are about one work-group per CU, each slice keeping 512 rows (a batch of 64 per wave).
    const int64_t blocks = xmk::ceil_div(n, (int64_t)(rows_kind == kRowsMC ? kRowsMinBN : kColsBN));
    int ks = 1;
    if (blocks < kRowsEnoughBlocks)
      while (ks < 16 && blocks * ks < 256 && k % (ks * 2 * 8) == 0 && k / (ks * 2) >= 512) ks *= 2;
    if (ks > 1) *policy = kRowsPolicy;
    return ks;
  }
  const Policy& pol = kPolicies[select_policy(m, n, k, 1, kRowsNone, !d->rhs.transpose)];
  const int64_t tiles = xmk::ceil_div(m, pol.bm) * xmk::ceil_div(n, pol.bn);
  int ks = 1;
  while (ks < 8 && tiles * ks * 2 <= 256 && k % (ks * 2 * 8) == 0 && k / (ks * 2) >= 512) ks *= 2;
  return ks;
}

void gemm_dims(const xmk_gemm_desc* d, int64_t* m, int64_t* n, int64_t* k) {
  const bool t = d->out.transpose != 0;  // C^T = B^T A^T swaps the roles
  const xmk_matrix& lhs = t ? d->rhs : d->lhs;
  const xmk_matrix& rhs = t ? d->lhs : d->rhs;
  const bool lt = t ? !lhs.transpose : lhs.transpose, rt = t ? !rhs.transpose : rhs.transpose;
  *m = lt ? lhs.num_cols : lhs.num_rows;
  *k = lt ? lhs.num_rows : lhs.num_cols;
  *n = rt ? rhs.num_rows : rhs.num_cols;
}
}  // namespace

extern "C" int xmk_gemm(const xmk_gemm_desc* d, void* stream) { return run_gemm(d, nullptr, nullptr, stream); }

extern "C" size_t xmk_gemm_workspace_bytes(const xmk_gemm_desc* d) {
  if (!d || d->out.transpose) return 0;
  int64_t m, n, k;
  gemm_dims(d, &m, &n, &k);
  if (m <= 0 || n <= 0 || k <= 0) return 0;
  int pol;
  const int ks = plan_splitk(d, m, n, k, &pol);
  return ks > 1 ? (size_t)ks * m * n * sizeof(float) : 0;
}

extern "C" int xmk_gemm_ws(const xmk_gemm_desc* d, void* workspace, size_t workspace_bytes, void* stream) {
  if (!d) return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: null descriptor");
  const size_t need = xmk_gemm_workspace_bytes(d);
  if (need == 0 || !workspace || workspace_bytes < need || !xmk::aligned(workspace, 16) || d->lhs.transpose)
    return run_gemm(d, nullptr, nullptr, stream);
  int64_t m, n, k;
  gemm_dims(d, &m, &n, &k);
  int slice_policy;
  const int ks = plan_splitk(d, m, n, k, &slice_policy);
  // Pass 1: the K slices as a batched GEMM into fp32 partial sums (no epilogue); a slice is a
  // column range of lhs and a row (or column) range of rhs, so only the batch strides change.
  xmk_gemm_desc p = *d;
  const int64_t kz = k / ks;
  p.lhs.num_cols = kz;
  p.lhs.batch_stride = kz;
  if (p.rhs.transpose) { p.rhs.num_cols = kz; p.rhs.batch_stride = kz; }
  else { p.rhs.num_rows = kz; p.rhs.batch_stride = kz * p.rhs.leading_dim_stride; }
  p.out.data = workspace; p.out.leading_dim_stride = n; p.out.batch_stride = m * n;
  p.c = nullptr; p.bias = nullptr;
  p.dtype_out = XMK_F32;
  p.batch_size = ks; p.alpha = 1.0f; p.beta = 0.0f; p.epilogue = XMK_EPI_DEFAULT;
  // what the full call would have rejected must still be rejected: validate it first
  int act = ACT_NONE;
  bool wants_bias = false;
  switch (d->epilogue) {
    case XMK_EPI_DEFAULT: break;
    case XMK_EPI_RELU: act = ACT_RELU; break;
    case XMK_EPI_GELU: act = ACT_GELU; break;
    case XMK_EPI_BIAS: wants_bias = true; break;
    case XMK_EPI_BIAS_RELU: wants_bias = true; act = ACT_RELU; break;
    case XMK_EPI_BIAS_GELU: wants_bias = true; act = ACT_GELU; break;
    default: return run_gemm(d, nullptr, nullptr, stream);  // reports the error
  }
  // (the sliced copy would hide a reduction size that differs between the operands, or a leading
  // dimension shorter than the full row)
  const int64_t k_rhs = d->rhs.transpose ? d->rhs.num_cols : d->rhs.num_rows;
  if (k_rhs != k || d->lhs.leading_dim_stride < d->lhs.num_cols || d->rhs.leading_dim_stride < d->rhs.num_cols)
    return run_gemm(d, nullptr, nullptr, stream);  // reports the error
  if ((wants_bias && !d->bias) || (d->beta != 0.0f && !d->c) || !d->out.data ||
      d->out.num_rows != m || d->out.num_cols != n || d->out.leading_dim_stride < n ||
      (d->dtype_out != d->dtype_in && d->dtype_out != XMK_F32))
    return run_gemm(d, nullptr, nullptr, stream);  // reports the error
  xmk::trace("gemm m=%lld n=%lld k=%lld -> split K %d ways", (long long)m, (long long)n, (long long)k, ks);
  int rc = run_gemm(&p, nullptr, nullptr, stream, slice_policy);
  if (rc != XMK_OK) return rc;
  ReduceParams r;
  r.partial = (const float*)workspace; r.out = d->out.data; r.c = d->beta != 0.0f ? d->c : nullptr;
  r.bias = wants_bias ? d->bias : nullptr;
  r.M = (int)m; r.N = (int)n; r.ks = ks; r.ldc = d->out.leading_dim_stride;
  r.kin = generic_kind(d->dtype_in); r.kout = generic_kind(d->dtype_out);
  r.alpha = d->alpha; r.beta = d->beta; r.act = act;
  hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)xmk::ceil_div(m * n / 4, 256)), dim3(256), 0,
                     (hipStream_t)stream, r);
  return xmk::check_launch("gemm");
}

extern "C" int xmk_gemm_qkv(const xmk_gemm_desc* d, void* out_k, void* out_v, void* stream) {
  if (!d) return xmk::fail(XMK_INVALID_ARGUMENT, "gemm_qkv: null descriptor");
  if (!out_k || !out_v) return xmk::fail(XMK_INVALID_ARGUMENT, "gemm_qkv: null output");
  if (d->batch_size != 1 || d->beta != 0.0f || d->out.transpose)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gemm_qkv: needs batch_size 1, beta 0 and a row-major output");
  if (d->dtype_in != d->dtype_out || (d->dtype_in != XMK_BF16 && d->dtype_in != XMK_F16))
    return xmk::fail(XMK_UNIMPLEMENTED, "gemm_qkv: 16-bit input and output of one type only");  // gemm.h:112-170
  return run_gemm(d, out_k, out_v, stream);
}

namespace {
int run_gemm(const xmk_gemm_desc* d, void* out1, void* out2, void* stream, int policy) {
  if (!d) return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: null descriptor");
  if (!d->lhs.data || !d->rhs.data || !d->out.data)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: null operand");
  // Accepted dtype triples: onednn_matmul_utils.cc:605-610.
  const int din = d->dtype_in, dout = d->dtype_out;
  const bool ok_types = (din == XMK_BF16 && (dout == XMK_BF16 || dout == XMK_F32)) ||
                        (din == XMK_F16 && (dout == XMK_F16 || dout == XMK_F32)) ||
                        (din == XMK_F32 && dout == XMK_F32) || (din == XMK_S8 && dout == XMK_S32);
  if (!ok_types)
    return xmk::fail(XMK_INTERNAL, "Unexpected GEMM lhs type %d, rhs type %d and output type %d", din,
                     din, dout);
  int act = ACT_NONE;
  bool wants_bias = false;
  switch (d->epilogue) {
    case XMK_EPI_DEFAULT: break;
    case XMK_EPI_RELU: act = ACT_RELU; break;
    case XMK_EPI_GELU: act = ACT_GELU; break;
    case XMK_EPI_BIAS: wants_bias = true; break;
    case XMK_EPI_BIAS_RELU: wants_bias = true; act = ACT_RELU; break;
    case XMK_EPI_BIAS_GELU: wants_bias = true; act = ACT_GELU; break;
    case XMK_EPI_GELU_AUX:
    case XMK_EPI_BIAS_GELU_AUX:
      // onednn_matmul_utils.cc:321-322,452-453
      return xmk::fail(XMK_UNIMPLEMENTED, "Unsupported Activation mode");
    default: return xmk::fail(XMK_INTERNAL, "Unknown Epilogue.");
  }
  if (wants_bias && !d->bias)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: epilogue adds a vector bias but bias is null");
  if (d->beta != 0.0f && !d->c)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: beta != 0 but c is null");
  if (d->batch_size < 1) return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: batch_size < 1");

  // Column-major output: C^T = B^T A^T (MakeBlasGemmCompatible, onednn_matmul_utils.cc:513-530).
  xmk_matrix lhs = d->lhs, rhs = d->rhs, out = d->out;
  if (out.transpose) {
    xmk_matrix t = lhs;
    lhs = rhs;
    rhs = t;
    lhs.transpose = !lhs.transpose;
    rhs.transpose = !rhs.transpose;
    out.transpose = 0;
  }
  const int64_t m = lhs.transpose ? lhs.num_cols : lhs.num_rows;
  const int64_t k = lhs.transpose ? lhs.num_rows : lhs.num_cols;
  const int64_t k2 = rhs.transpose ? rhs.num_cols : rhs.num_rows;
  const int64_t n = rhs.transpose ? rhs.num_rows : rhs.num_cols;
  if (m <= 0 || n <= 0 || k <= 0) return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: empty dimension");
  if (k != k2)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: reduction sizes differ (lhs %lld, rhs %lld)",
                     (long long)k, (long long)k2);
  if (out.num_rows != m || out.num_cols != n)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: output is %lldx%lld, product is %lldx%lld",
                     (long long)out.num_rows, (long long)out.num_cols, (long long)m, (long long)n);
  if (lhs.leading_dim_stride < lhs.num_cols || rhs.leading_dim_stride < rhs.num_cols ||
      out.leading_dim_stride < n)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: leading_dim_stride smaller than the row length");
  if (m > INT32_MAX / 2 || n > INT32_MAX / 2 || k > INT32_MAX / 2 || d->batch_size > 65535)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: dimension too large");
  if (!d->bias && wants_bias) return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: bias missing");
  // The tile loaders form byte offsets of up to 256 rows of an operand in 32 bits.
  constexpr int64_t kMaxLd = int64_t{1} << 22;
  if (lhs.leading_dim_stride >= kMaxLd || rhs.leading_dim_stride >= kMaxLd || out.leading_dim_stride >= kMaxLd)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gemm: leading_dim_stride of 2^22 elements or more");

  hipStream_t st = (hipStream_t)stream;
  const bool qkv = out1 != nullptr;
  const bool sixteen = din == XMK_BF16 || din == XMK_F16;
  const bool fast = sixteen && direct_ok(lhs, rhs) && xmk::aligned(out.data, 16) && xmk::aligned(out1, 16) &&
                    xmk::aligned(out2, 16);
  // 16-bit operands that miss those conditions still run on the matrix cores, with operands gathered
  // element by element; the output pointers must allow the epilogue's vector stores.
  const bool gather = !fast && sixteen && xmk::aligned(out.data, 16) && xmk::aligned(out1, 16) &&
                      xmk::aligned(out2, 16) && xmk::aligned(d->c, 16);
  if (fast || gather) {
    GemmParams p;
    p.a = lhs.data; p.b = rhs.data; p.out = out.data; p.c = d->beta != 0.0f ? d->c : nullptr;
    p.bias = wants_bias ? d->bias : nullptr;
    p.M = (int)m; p.N = (int)n; p.K = (int)k;
    p.lda = lhs.leading_dim_stride; p.ldb = rhs.leading_dim_stride; p.ldc = out.leading_dim_stride;
    p.sa = lhs.batch_stride; p.sb = rhs.batch_stride; p.sc = out.batch_stride;
    p.alpha = d->alpha; p.beta = d->beta; p.act = act;
    p.out_alt[0] = out1; p.out_alt[1] = out2; p.sbias = 0;
    if (qkv) { p.sa = 0; p.sc = 0; p.sbias = n; }
    // Widest load of the gathering kernel per operand: the pointer, the leading dimension, the batch
    // stride and the stored row length must all be multiples of it.
    auto widest = [](const xmk_matrix& x) {
      int v = 8;
      while (v > 1 && (!xmk::aligned(x.data, 2 * v) || x.leading_dim_stride % v || x.batch_stride % v || x.num_cols % v))
        v /= 2;
      return v;
    };
    p.vec_a = widest(lhs);
    p.vec_b = widest(rhs);
    const bool a_mc = lhs.transpose != 0;   // stored [K, M]
    const bool b_mc = rhs.transpose == 0;   // stored [K, N]
    const int batch = qkv ? 3 : (int)d->batch_size;
    const int rows_kind = fast ? gemm_rows_applicable(p, a_mc, b_mc) : kRowsNone;
    // the forced policy first, then the K-split planner's, then the table and the rules
    const int pol = (forced_policy() < 0 && policy >= 0 && policy < kNumPolicies &&
                     (policy != kRowsPolicy || rows_kind != kRowsNone))
                        ? policy : select_policy(m, n, k, batch, rows_kind, b_mc);
    xmk::trace("gemm m=%lld n=%lld k=%lld batch=%lld lhs_t=%d rhs_t=%d epilogue=%d beta=%g -> %s",
               (long long)m, (long long)n, (long long)k, (long long)d->batch_size, lhs.transpose,
               rhs.transpose, d->epilogue, d->beta, gather ? kGatherPolicy.name : kPolicies[pol].name);
    if (gather) {
      if (din == XMK_BF16) {
        if (dout == XMK_F32) launch_layout_gather<__bf16, true>(a_mc, b_mc, p, batch, st);
        else launch_layout_gather<__bf16, false>(a_mc, b_mc, p, batch, st);
      } else {
        if (dout == XMK_F32) launch_layout_gather<_Float16, true>(a_mc, b_mc, p, batch, st);
        else launch_layout_gather<_Float16, false>(a_mc, b_mc, p, batch, st);
      }
      return xmk::check_launch("gemm");
    }
    if (pol == kRowsPolicy) {
      launch_gemm_rows(p, b_mc, din == XMK_BF16, dout == XMK_F32, batch, st);
      return xmk::check_launch("gemm");
    }
    if (din == XMK_BF16) {
      if (dout == XMK_F32) launch_layout<__bf16, true>(a_mc, b_mc, pol, p, batch, st);
      else launch_layout<__bf16, false>(a_mc, b_mc, pol, p, batch, st);
    } else {
      if (dout == XMK_F32) launch_layout<_Float16, true>(a_mc, b_mc, pol, p, batch, st);
      else launch_layout<_Float16, false>(a_mc, b_mc, pol, p, batch, st);
    }
    return xmk::check_launch("gemm");
  }

  if (din == XMK_F32 && dout == XMK_F32 && xmk::aligned(out.data, 16) && xmk::aligned(out1, 16) &&
      xmk::aligned(out2, 16) && xmk::aligned(d->c, 16) && xmk::aligned(lhs.data, 4) && xmk::aligned(rhs.data, 4)) {
    GemmParams p;
    p.a = lhs.data; p.b = rhs.data; p.out = out.data; p.c = d->beta != 0.0f ? d->c : nullptr;
    p.bias = wants_bias ? d->bias : nullptr;
    p.M = (int)m; p.N = (int)n; p.K = (int)k;
    p.lda = lhs.leading_dim_stride; p.ldb = rhs.leading_dim_stride; p.ldc = out.leading_dim_stride;
    p.sa = lhs.batch_stride; p.sb = rhs.batch_stride; p.sc = out.batch_stride;
    p.alpha = d->alpha; p.beta = d->beta; p.act = act;
    p.out_alt[0] = out1; p.out_alt[1] = out2; p.sbias = 0;
    if (qkv) { p.sa = 0; p.sc = 0; p.sbias = n; }
    auto vec4 = [](const xmk_matrix& x) {
      return (xmk::aligned(x.data, 16) && x.leading_dim_stride % 4 == 0 && x.batch_stride % 4 == 0 && x.num_cols % 4 == 0) ? 4 : 1;
    };
    p.vec_a = vec4(lhs);
    p.vec_b = vec4(rhs);
    xmk::trace("gemm m=%lld n=%lld k=%lld batch=%lld lhs_t=%d rhs_t=%d -> mfma_f32_128x128x16", (long long)m,
               (long long)n, (long long)k, (long long)d->batch_size, lhs.transpose, rhs.transpose);
    launch_gemm_f32(p, lhs.transpose != 0, rhs.transpose == 0, qkv ? 3 : (int)d->batch_size, st);
    return xmk::check_launch("gemm");
  }
  if (din == XMK_S8 && (d->alpha != 1.0f || d->beta != 0.0f || d->epilogue != XMK_EPI_DEFAULT))
    return xmk::fail(XMK_UNIMPLEMENTED, "gemm: s8 x s8 -> s32 supports alpha=1, beta=0, no epilogue");
  if (din == XMK_S8 && dout == XMK_S32 && xmk::aligned(out.data, 16) && xmk::aligned(out1, 16) && xmk::aligned(out2, 16)) {
    GemmParams p{};
    p.a = lhs.data; p.b = rhs.data; p.out = out.data;
    p.M = (int)m; p.N = (int)n; p.K = (int)k;
    p.lda = lhs.leading_dim_stride; p.ldb = rhs.leading_dim_stride; p.ldc = out.leading_dim_stride;
    p.sa = lhs.batch_stride; p.sb = rhs.batch_stride; p.sc = out.batch_stride;
    p.out_alt[0] = out1; p.out_alt[1] = out2;
    if (qkv) { p.sa = 0; p.sc = 0; }
    auto vec16 = [](const xmk_matrix& x) {
      return (xmk::aligned(x.data, 16) && x.leading_dim_stride % 16 == 0 && x.batch_stride % 16 == 0 && x.num_cols % 16 == 0) ? 16 : 1;
    };
    p.vec_a = vec16(lhs);
    p.vec_b = vec16(rhs);
    xmk::trace("gemm m=%lld n=%lld k=%lld batch=%lld lhs_t=%d rhs_t=%d -> mfma_s8_128x128x64", (long long)m,
               (long long)n, (long long)k, (long long)d->batch_size, lhs.transpose, rhs.transpose);
    launch_gemm_s8(p, lhs.transpose != 0, rhs.transpose == 0, qkv ? 3 : (int)d->batch_size, st);
    return xmk::check_launch("gemm");
  }
  GenericParams g;
  g.a = lhs.data; g.b = rhs.data; g.out = out.data; g.c = d->beta != 0.0f ? d->c : nullptr;
  g.bias = wants_bias ? d->bias : nullptr;
  g.M = (int)m; g.N = (int)n; g.K = (int)k;
  g.lda = lhs.leading_dim_stride; g.ldb = rhs.leading_dim_stride; g.ldc = out.leading_dim_stride;
  g.sa = lhs.batch_stride; g.sb = rhs.batch_stride; g.sc = out.batch_stride;
  g.ta = lhs.transpose; g.tb = rhs.transpose;
  g.kin = generic_kind(din); g.kout = generic_kind(dout);
  g.alpha = d->alpha; g.beta = d->beta; g.act = act;
  g.out_alt[0] = out1; g.out_alt[1] = out2; g.sbias = 0;
  if (qkv) { g.sa = 0; g.sc = 0; g.sbias = n; }
  xmk::trace("gemm m=%lld n=%lld k=%lld -> generic_64x64", (long long)m, (long long)n, (long long)k);
  hipLaunchKernelGGL(gemm_generic_kernel,
                     dim3((unsigned)xmk::ceil_div(n, 64), (unsigned)xmk::ceil_div(m, 64),
                          (unsigned)(qkv ? 3 : d->batch_size)),
                     dim3(256), 0, st, g);
  return xmk::check_launch("gemm");
}
}  // namespace
