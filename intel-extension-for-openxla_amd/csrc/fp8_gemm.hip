// FP8 (OCP e4m3fn) GEMM: out = bf16(a_scale * b_scale * A B), fp32 accumulation.
//
// MFMA kernel: A [M,K] row-major and B stored [N,K] (both reduction-contiguous, the
// layout XLA's "__cublas$lt$matmul$f8" rewrite produces).  256x256 output tile per
// work-group, K walked in steps of 128 bytes, operand tiles staged global -> registers
// -> LDS (double-buffered, 16-byte chunks XOR-swizzled by row) and consumed by
// v_mfma_f32_32x32x64_f8f6f4: a lane supplies 32 consecutive k of one row per
// instruction.  The per-tensor scales are read from device memory in the epilogue.
// B stored [K,N] (rhs_transpose == 0) runs a plain tiled kernel.
#include <utility>

#include "common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef int intx8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int BKB = 128;  // K step in bytes (= fp8 elements)
constexpr uint32_t kOob = 0x80000000u;

struct Fp8Params {
  const uint8_t* a;
  const uint8_t* b;
  const float* a_scale;
  const float* b_scale;
  __bf16* out;
  int M, N, K;
  int tiles_m, tiles_n;
};

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

__device__ __forceinline__ floatx16 zero16() {
  return floatx16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)kOob, 0x00020000);
}

// One operand tile [ROWS][128 bytes]: chunk ch = tid + i NT -> row ch / 8, 16-byte chunk ch % 8.
template <int ROWS, int NT>
struct Stager {
  static constexpr int NCH = ROWS * 8 / NT;
  u32x4 r[NCH];
  uint32_t voff[NCH];
  int kin;  // first k byte of this thread's chunks within the step (same for all chunks)

  __device__ __forceinline__ void init(int64_t ld, int valid, int tid) {
    kin = (tid % 8) * 16;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int row = (tid + i * NT) / 8;
      voff[i] = row < valid ? (uint32_t)((int64_t)row * ld + kin) : kOob;
    }
  }
  __device__ __forceinline__ void load(const void* base, int kleft) {
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(base);
    const bool ok = kin < kleft;  // K % 16 == 0: a chunk is all in or all out
#pragma unroll
    for (int i = 0; i < NCH; ++i)
      r[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, ok ? voff[i] : kOob, 0, 0));
  }
  __device__ __forceinline__ void store(char* lds, int tid) const {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int ch = tid + i * NT;
      const int row = ch / 8, c = ch % 8;
      *reinterpret_cast<u32x4*>(lds + row * BKB + ((c ^ (row & 7)) << 4)) = r[i];
    }
  }
};

// Fragment for k-step ks (64 k): lane l gets row row0 + l%32, bytes 64 ks + 32 (l/32) .. +31.
__device__ __forceinline__ intx8 read_frag(const char* lds, int row0, int ks, int lane) {
  const int row = row0 + (lane & 31);
  const int c = ks * 4 + (lane >> 5) * 2;
  const u32x4 lo = *reinterpret_cast<const u32x4*>(lds + row * BKB + ((c ^ (row & 7)) << 4));
  const u32x4 hi = *reinterpret_cast<const u32x4*>(lds + row * BKB + (((c + 1) ^ (row & 7)) << 4));
  intx8 v;
  v[0] = (int)lo[0]; v[1] = (int)lo[1]; v[2] = (int)lo[2]; v[3] = (int)lo[3];
  v[4] = (int)hi[0]; v[5] = (int)hi[1]; v[6] = (int)hi[2]; v[7] = (int)hi[3];
  return v;
}

__device__ __forceinline__ floatx16 mfma_fp8(intx8 a, intx8 b, floatx16 c) {
  // cbsz = blgp = 0: both operands e4m3; block scales 127 = 2^0 (E8M0).
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 127, 0, 127);
}

template <int BM, int BN, int WGM, int WGN>
__global__ __launch_bounds__(WGM * WGN * 64) void fp8_gemm_kernel(Fp8Params p) {
  constexpr int NT = WGM * WGN * 64;
  constexpr int WTM = BM / WGM, WTN = BN / WGN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * BKB, B_BYTES = BN * BKB, STAGE = A_BYTES + B_BYTES;
  __shared__ __attribute__((aligned(16))) char lds[2 * STAGE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;

  int pid = blockIdx.x;
  const int ntiles = p.tiles_m * p.tiles_n;
  if (ntiles % 8 == 0) pid = (pid % 8) * (ntiles / 8) + pid / 8;  // one contiguous run of tiles per XCD
  constexpr int GM = 8;
  const int group = pid / (GM * p.tiles_n);
  const int first_m = group * GM;
  const int gsize = min(p.tiles_m - first_m, GM);
  const int tile_m = first_m + (pid % (GM * p.tiles_n)) % gsize;
  const int tile_n = (pid % (GM * p.tiles_n)) / gsize;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = zero16();

  Stager<BM, NT> sa;
  Stager<BN, NT> sb;
  sa.init(p.K, p.M - m0, tid);
  sb.init(p.K, p.N - n0, tid);
  const uint8_t* a_tile = p.a + (int64_t)m0 * p.K;
  const uint8_t* b_tile = p.b + (int64_t)n0 * p.K;
  const int KT = (p.K + BKB - 1) / BKB;

  sa.load(a_tile, p.K);
  sb.load(b_tile, p.K);
  sa.store(lds, tid);
  sb.store(lds + A_BYTES, tid);
  __syncthreads();

  intx8 fa[2][TM], fb[2][TN];
  auto read_frags = [&](const char* stage, int ks, int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[buf][i] = read_frag(stage, wm * WTM + i * 32, ks, lane);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[buf][j] = read_frag(stage + A_BYTES, wn * WTN + j * 32, ks, lane);
  };
  auto mma = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = mfma_fp8(fb[buf][j], fa[buf][i], acc[i][j]);
  };
  auto interleave = [&]() {
#pragma unroll
    for (int r = 0; r < 2 * (TM + TN); ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
  };

  read_frags(lds, 0, 0);
  for (int kt = 0; kt < KT; ++kt) {
    const char* cur = lds + (kt & 1) * STAGE;
    char* nxt = lds + ((kt + 1) & 1) * STAGE;
    const bool more = kt + 1 < KT;
    if (more) {
      a_tile += BKB;
      b_tile += BKB;
      sa.load(a_tile, p.K - (kt + 1) * BKB);
      sb.load(b_tile, p.K - (kt + 1) * BKB);
    }
    read_frags(cur, 1, 1);
    mma(0);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    if (more) {
      sa.store(nxt, tid);
      sb.store(nxt + A_BYTES, tid);
    }
    __syncthreads();
    if (more) read_frags(nxt, 0, 0);
    mma(1);
    if (more) interleave();
    __builtin_amdgcn_sched_barrier(0);
  }

  // acc[i][j][e] is out[m][n], m = m0 + wm WTM + 32 i + lane%32, n = n0 + wn WTN + 32 j + 8 (e/4) + 4 (lane/32) + e%4.
  const float scale = p.a_scale[0] * p.b_scale[0];
  static_for<TM>([&](auto I) {
    constexpr int i = decltype(I)::value;
    const int m = m0 + wm * WTM + i * 32 + (lane & 31);
    static_for<TN>([&](auto J) {
      constexpr int j = decltype(J)::value;
      const floatx16 t = acc[i][j];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * WTN + j * 32 + q * 8 + (lane >> 5) * 4;
        if (m < p.M && n < p.N) {  // N % 4 == 0: the four columns are all in range
          union { __bf16 e[4]; u32x2 w; } o;
          o.e[0] = (__bf16)(t[4 * q + 0] * scale);
          o.e[1] = (__bf16)(t[4 * q + 1] * scale);
          o.e[2] = (__bf16)(t[4 * q + 2] * scale);
          o.e[3] = (__bf16)(t[4 * q + 3] * scale);
          *reinterpret_cast<u32x2*>(p.out + (int64_t)m * p.N + n) = o.w;
        }
      }
    });
  });
}

// Plain tiled kernel for any layout / size: 64x64 tile, fp8 decoded with the hardware
// conversion while staging, fp32 FMA.
__global__ __launch_bounds__(256) void fp8_gemm_generic_kernel(Fp8Params p, int rhs_transpose) {
  __shared__ float As[16][65];
  __shared__ float Bs[16][65];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < p.K; k0 += 16) {
    for (int e = threadIdx.x; e < 16 * 64; e += 256) {
      const int kk = e / 64, r = e % 64, k = k0 + kk;
      float av = 0.f, bv = 0.f;
      if (k < p.K && m0 + r < p.M)
        av = __builtin_amdgcn_cvt_f32_fp8((int)p.a[(int64_t)(m0 + r) * p.K + k], 0);
      if (k < p.K && n0 + r < p.N) {
        const int64_t i = rhs_transpose ? (int64_t)(n0 + r) * p.K + k : (int64_t)k * p.N + (n0 + r);
        bv = __builtin_amdgcn_cvt_f32_fp8((int)p.b[i], 0);
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
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
  const float scale = p.a_scale[0] * p.b_scale[0];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m < p.M && n < p.N) p.out[(int64_t)m * p.N + n] = (__bf16)(acc[i][j] * scale);
    }
}

}  // namespace

extern "C" int xmk_fp8_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale,
                            void* out, int64_t m, int64_t n, int64_t k, int32_t rhs_transpose,
                            void* stream) {
  if (!a || !b || !a_scale || !b_scale || !out) return xmk::fail(XMK_INVALID_ARGUMENT, "fp8_gemm: null pointer");
  if (m <= 0 || n <= 0 || k <= 0) return xmk::fail(XMK_INVALID_ARGUMENT, "fp8_gemm: empty dimension");
  if (m > (1 << 30) || n > (1 << 30) || k > (1 << 30))
    return xmk::fail(XMK_INVALID_ARGUMENT, "fp8_gemm: dimension too large");
  Fp8Params p;
  p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.a_scale = a_scale; p.b_scale = b_scale;
  p.out = (__bf16*)out; p.M = (int)m; p.N = (int)n; p.K = (int)k;
  hipStream_t st = (hipStream_t)stream;
  const bool fast = rhs_transpose != 0 && k % 16 == 0 && n % 4 == 0 && xmk::aligned(a, 16) &&
                    xmk::aligned(b, 16) && xmk::aligned(out, 8) && 256 * k < (int64_t)kOob;
  if (fast) {
    const bool big = xmk::ceil_div(m, 256) * xmk::ceil_div(n, 256) >= 256;
    xmk::trace("fp8_gemm m=%lld n=%lld k=%lld -> %s", (long long)m, (long long)n, (long long)k,
               big ? "mfma_256x256" : "mfma_128x128");
    if (big) {
      p.tiles_m = (int)xmk::ceil_div(m, 256); p.tiles_n = (int)xmk::ceil_div(n, 256);
      hipLaunchKernelGGL((fp8_gemm_kernel<256, 256, 2, 2>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0, st, p);
    } else {
      p.tiles_m = (int)xmk::ceil_div(m, 128); p.tiles_n = (int)xmk::ceil_div(n, 128);
      hipLaunchKernelGGL((fp8_gemm_kernel<128, 128, 2, 2>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0, st, p);
    }
  } else {
    xmk::trace("fp8_gemm m=%lld n=%lld k=%lld rhs_t=%d -> generic_64x64", (long long)m, (long long)n,
               (long long)k, rhs_transpose);
    hipLaunchKernelGGL(fp8_gemm_generic_kernel, dim3((unsigned)xmk::ceil_div(n, 64), (unsigned)xmk::ceil_div(m, 64)),
                       dim3(256), 0, st, p, (int)rhs_transpose);
  }
  return xmk::check_launch("fp8_gemm");
}
