// Int4 weight-only GEMM for small M (decode): HBM-bound streaming of the packed
// weights through MFMA, plus the stand-alone dequantisation kernel.
//
// Weight word qweight[r, n] holds the 8 nibbles of input channels k = 8r..8r+7 for
// output channel n.  That is exactly the B-operand fragment of one lane of
// v_mfma_f32_16x16x32_f16 (lane -> column l%16, k-slots 8*(l/16)..+7), so a lane
// loads words, expands each to 8 fp16 integers in registers and feeds the matrix
// core; nothing is staged through LDS.  Zero points and scales are applied once
// per quantisation group on the fp32 accumulator:
//     out[m,n] = sum_g s[g,n] * ( sum_{k in g} a[m,k] q[k,n]  -  z[g,n] * sum_{k in g} a[m,k] )
// where the second sum comes from one extra MFMA against a B operand of ones.
#include "common.h"
#include "int4_gemm.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

union Frag {
  half8 h;
  uint32_t u[4];
  half2v p[4];
};

// One packed word -> 8 exact fp16 integers, in k-slot order (0,4,1,5,2,6,3,7).
// 0x6400 | q is 1024 + q; 0x5400 | (q << 4) is 64 + q; the packed subtract is exact.
__device__ __forceinline__ half8 unpack_word(uint32_t w) {
  const uint32_t w8 = w >> 8;
  Frag f;
  f.u[0] = (w & 0x000f000fu) | 0x64006400u;
  f.u[1] = (w & 0x00f000f0u) | 0x54005400u;
  f.u[2] = (w8 & 0x000f000fu) | 0x64006400u;
  f.u[3] = (w8 & 0x00f000f0u) | 0x54005400u;
  const half2v k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
  const half2v k64 = {(_Float16)64.0f, (_Float16)64.0f};
  f.p[0] -= k1024;
  f.p[1] -= k64;
  f.p[2] -= k1024;
  f.p[3] -= k64;
  return f.h;
}

// 8 consecutive activations -> the same k-slot order (0,4,1,5,2,6,3,7).
__device__ __forceinline__ half8 permute_act(u32x4 d) {
  Frag f;
  f.u[0] = __builtin_amdgcn_perm(d[2], d[0], 0x05040100u);  // (h0, h4)
  f.u[1] = __builtin_amdgcn_perm(d[2], d[0], 0x07060302u);  // (h1, h5)
  f.u[2] = __builtin_amdgcn_perm(d[3], d[1], 0x05040100u);  // (h2, h6)
  f.u[3] = __builtin_amdgcn_perm(d[3], d[1], 0x07060302u);  // (h3, h7)
  return f.h;
}

template <int W>
struct Words {
  uint32_t w[W];
};

template <int W>
__device__ __forceinline__ Words<W> load_words(const uint32_t* p) {
  Words<W> r;
  if constexpr (W == 4) {
    u32x4 v = *reinterpret_cast<const u32x4*>(p);
    r.w[0] = v[0]; r.w[1] = v[1]; r.w[2] = v[2]; r.w[3] = v[3];
  } else if constexpr (W == 2) {
    uint2 v = *reinterpret_cast<const uint2*>(p);
    r.w[0] = v.x; r.w[1] = v.y;
  } else {
    r.w[0] = *p;
  }
  return r;
}

// W    : words (output channels) per lane; a block covers 16*W output channels
// MT   : 16-row activation tiles (1 or 2)
// SPG  : 32-channel k-steps per quantisation group (group = 32*SPG)
// NW   : waves per block; wave w takes groups w, w+NW, ... and the partial
//        sums meet in LDS in a fixed order (deterministic result)
template <int W, int MT, int SPG, int NW>
__global__ __launch_bounds__(NW * 64) void int4_gemm_kernel(
    const _Float16* __restrict__ act, const uint32_t* __restrict__ qw,
    const _Float16* __restrict__ scales, const _Float16* __restrict__ zeros,
    const _Float16* __restrict__ bias, _Float16* __restrict__ out, int m_base, int M, int K,
    int N, xmk::Int4Epilogue ep) {
  constexpr int NCOL = 16 * W;
  __shared__ float red[NW][MT * 16][NCOL];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int col16 = lane & 15;
  const int kg = lane >> 4;
  const int n0 = blockIdx.x * NCOL + col16 * W;
  const bool col_ok = n0 < N;
  const int nsafe = col_ok ? n0 : 0;
  const int ngroups = K / (32 * SPG);

  const _Float16* arow[MT];
  bool row_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m_base + mt * 16 + col16;
    row_ok[mt] = m < M;
    arow[mt] = act + (size_t)(row_ok[mt] ? m : 0) * K + 8 * kg;
  }

  floatx4 acc[MT][W];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int c = 0; c < W; ++c) acc[mt][c] = floatx4{0.f, 0.f, 0.f, 0.f};

  Frag ones;
#pragma unroll
  for (int i = 0; i < 4; ++i) ones.u[i] = 0x3c003c00u;

  Words<W> cur[SPG], nxt[SPG];
  int g = wave;
  if (g < ngroups) {
#pragma unroll
    for (int s = 0; s < SPG; ++s)
      cur[s] = load_words<W>(qw + (size_t)(g * 4 * SPG + s * 4 + kg) * N + nsafe);
  }
  for (; g < ngroups; g += NW) {
    const int gn = g + NW;
    if (gn < ngroups) {
#pragma unroll
      for (int s = 0; s < SPG; ++s)
        nxt[s] = load_words<W>(qw + (size_t)(gn * 4 * SPG + s * 4 + kg) * N + nsafe);
    }
    _Float16 sc[W], zp[W];
#pragma unroll
    for (int c = 0; c < W; ++c) {
      sc[c] = scales[(size_t)g * N + nsafe + c];
      zp[c] = zeros[(size_t)g * N + nsafe + c];
    }
    floatx4 d[MT][W], asum[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      asum[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < W; ++c) d[mt][c] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int s = 0; s < SPG; ++s) {
      const int k0 = (g * SPG + s) * 32;
      half8 a[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (row_ok[mt]) raw = *reinterpret_cast<const u32x4*>(arow[mt] + k0);
        a[mt] = permute_act(raw);
      }
#pragma unroll
      for (int c = 0; c < W; ++c) {
        const half8 b = unpack_word(cur[s].w[c]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          d[mt][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[mt], b, d[mt][c], 0, 0, 0);
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        asum[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[mt], ones.h, asum[mt], 0, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < W; ++c) {
      const float s = (float)sc[c], z = (float)zp[c];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[mt][c][i] += s * (d[mt][c][i] - z * asum[mt][i]);
    }
#pragma unroll
    for (int s = 0; s < SPG; ++s) cur[s] = nxt[s];
  }

  // Lane holds rows 4*kg+i of columns col16*W+c.
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int c = 0; c < W; ++c) red[wave][mt * 16 + 4 * kg + i][col16 * W + c] = acc[mt][c][i];
  __syncthreads();

  const int rows = min(MT * 16, M - m_base);
  for (int e = threadIdx.x; e < rows * NCOL; e += NW * 64) {
    const int row = e / NCOL, col = e % NCOL;
    const int n = blockIdx.x * NCOL + col;
    if (n >= N) continue;
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) s += red[w][row][col];
    if (bias) s += (float)bias[n];
    if (ep.gelu) {  // gelu_new: 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) = x / (1 + e^{-2u})
      const float u = 0.7978845608028654f * (s + 0.044715f * s * s * s);
      s = s / (1.0f + __expf(-2.0f * u));
    }
    const size_t o = (size_t)(m_base + row) * N + n;
    if (ep.add0) s += (float)reinterpret_cast<const _Float16*>(ep.add0)[o];
    if (ep.add1) s += (float)reinterpret_cast<const _Float16*>(ep.add1)[o];
    out[o] = (_Float16)s;
  }
}

// W[k,n] = fp16_rne((float(q) - float(z)) * float(s)): two separately rounded
// fp32 operations (no fused multiply-add), then one rounding to fp16.
__global__ __launch_bounds__(256) void int4_dequant_kernel(
    const uint32_t* __restrict__ qw, const _Float16* __restrict__ scales,
    const _Float16* __restrict__ zeros, _Float16* __restrict__ w_out, int K, int N, int group) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one (word row, 4 columns)
  const int n4 = N / 4;
  const int64_t total = (int64_t)(K / 8) * n4;
  if (idx >= total) return;
  const int r = (int)(idx / n4);
  const int n = (int)(idx % n4) * 4;
  const u32x4 words = *reinterpret_cast<const u32x4*>(qw + (size_t)r * N + n);
  const int g = (r * 8) / group;
  float s[4], z[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    s[c] = (float)scales[(size_t)g * N + n + c];
    z[c] = (float)zeros[(size_t)g * N + n + c];
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    union { _Float16 h[4]; uint2 v; } o;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const float q = (float)((words[c] >> (4 * j)) & 0xfu);
      o.h[c] = (_Float16)__fmul_rn(__fsub_rn(q, z[c]), s[c]);
    }
    *reinterpret_cast<uint2*>(w_out + (size_t)(r * 8 + j) * N + n) = o.v;
  }
}

template <int W, int MT, int SPG, int NW>
void launch(const void* act, const void* qw, const void* scales, const void* zeros,
            const void* bias, void* out, int m_base, int M, int K, int N,
            const xmk::Int4Epilogue& ep, hipStream_t st) {
  const int blocks = (int)xmk::ceil_div(N, 16 * W);
  hipLaunchKernelGGL((int4_gemm_kernel<W, MT, SPG, NW>), dim3(blocks), dim3(NW * 64), 0, st,
                     (const _Float16*)act, (const uint32_t*)qw, (const _Float16*)scales,
                     (const _Float16*)zeros, (const _Float16*)bias, (_Float16*)out, m_base, M, K, N, ep);
}

template <int W, int MT, int NW>
int launch_spg(int spg, const void* act, const void* qw, const void* scales, const void* zeros,
               const void* bias, void* out, int m_base, int M, int K, int N,
               const xmk::Int4Epilogue& ep, hipStream_t st) {
  switch (spg) {
    case 1: launch<W, MT, 1, NW>(act, qw, scales, zeros, bias, out, m_base, M, K, N, ep, st); break;
    case 2: launch<W, MT, 2, NW>(act, qw, scales, zeros, bias, out, m_base, M, K, N, ep, st); break;
    case 4: launch<W, MT, 4, NW>(act, qw, scales, zeros, bias, out, m_base, M, K, N, ep, st); break;
    case 8: launch<W, MT, 8, NW>(act, qw, scales, zeros, bias, out, m_base, M, K, N, ep, st); break;
    default: return xmk::fail(XMK_UNIMPLEMENTED, "int4_gemm: group must be 32, 64, 128 or 256");
  }
  return XMK_OK;
}

}  // namespace

int xmk::int4_gemm_launch(const void* act, const void* qweight, const void* scales,
                          const void* zeros, const void* bias, void* out, int64_t m, int64_t k,
                          int64_t n, int64_t group, const Int4Epilogue& ep, hipStream_t st) {
  if (!act || !qweight || !scales || !zeros || !out)
    return xmk::fail(XMK_INVALID_ARGUMENT, "int4_gemm: null pointer");
  if (m <= 0 || k <= 0 || n <= 0 || group <= 0)
    return xmk::fail(XMK_INVALID_ARGUMENT, "int4_gemm: non-positive size");
  if (n % 8 != 0 || group % 8 != 0 || k % group != 0)
    return xmk::fail(XMK_INVALID_ARGUMENT,
                     "int4_gemm: need n %% 8 == 0, group %% 8 == 0, k %% group == 0 (m=%lld k=%lld "
                     "n=%lld group=%lld)", (long long)m, (long long)k, (long long)n, (long long)group);
  if (group % 32 != 0 || group > 256)
    return xmk::fail(XMK_UNIMPLEMENTED, "int4_gemm: group must be 32, 64, 128 or 256");
  if (k > (1 << 24) || n > (1 << 24) || m > (1 << 24))
    return xmk::fail(XMK_INVALID_ARGUMENT, "int4_gemm: dimension too large");
  if (!xmk::aligned(act, 16) || !xmk::aligned(qweight, 16) || !xmk::aligned(scales, 2) ||
      !xmk::aligned(out, 2))
    return xmk::fail(XMK_INVALID_ARGUMENT, "int4_gemm: act and qweight must be 16-byte aligned");
  const int spg = (int)(group / 32);
  const int M = (int)m, K = (int)k, N = (int)n;
  // Words per lane: the widest load that still yields about one block per CU.
  int w = 4;
  if (N / 64 < 192) w = 2;
  if (N / 32 < 192) w = 1;
  xmk::trace("int4_gemm m=%d k=%d n=%d group=%d words_per_lane=%d", M, K, N, (int)group, w);
  for (int m_base = 0; m_base < M; m_base += 32) {
    const bool two = (M - m_base) > 16;
    int rc;
#define XMK_INT4_CASE(WW)                                                                            \
  rc = two ? launch_spg<WW, 2, 8>(spg, act, qweight, scales, zeros, bias, out, m_base, M, K, N, ep, st) \
           : launch_spg<WW, 1, 16>(spg, act, qweight, scales, zeros, bias, out, m_base, M, K, N, ep, st)
    if (w == 4) { XMK_INT4_CASE(4); }
    else if (w == 2) { XMK_INT4_CASE(2); }
    else { XMK_INT4_CASE(1); }
#undef XMK_INT4_CASE
    if (rc != XMK_OK) return rc;
  }
  return xmk::check_launch("int4_gemm");
}

extern "C" int xmk_int4_gemm(const void* act, const void* qweight, const void* scales,
                             const void* zeros, const void* bias, void* out, int64_t m, int64_t k,
                             int64_t n, int64_t group, void* stream) {
  return xmk::int4_gemm_launch(act, qweight, scales, zeros, bias, out, m, k, n, group,
                               xmk::Int4Epilogue{}, (hipStream_t)stream);
}

extern "C" int xmk_int4_dequant(const void* qweight, const void* scales, const void* zeros,
                                void* w_out, int64_t k, int64_t n, int64_t group, void* stream) {
  if (!qweight || !scales || !zeros || !w_out)
    return xmk::fail(XMK_INVALID_ARGUMENT, "int4_dequant: null pointer");
  if (k <= 0 || n <= 0 || group <= 0 || n % 8 != 0 || group % 8 != 0 || k % group != 0)
    return xmk::fail(XMK_INVALID_ARGUMENT,
                     "int4_dequant: need n %% 8 == 0, group %% 8 == 0, k %% group == 0");
  if (k > (1 << 24) || n > (1 << 24)) return xmk::fail(XMK_INVALID_ARGUMENT, "int4_dequant: too large");
  if (!xmk::aligned(qweight, 16) || !xmk::aligned(w_out, 8))
    return xmk::fail(XMK_INVALID_ARGUMENT, "int4_dequant: qweight must be 16-byte aligned");
  const int64_t total = (k / 8) * (n / 4);
  hipLaunchKernelGGL(int4_dequant_kernel, dim3((unsigned)xmk::ceil_div(total, 256)), dim3(256), 0,
                     (hipStream_t)stream, (const uint32_t*)qweight, (const _Float16*)scales,
                     (const _Float16*)zeros, (_Float16*)w_out, (int)k, (int)n, (int)group);
  return xmk::check_launch("int4_dequant");
}
