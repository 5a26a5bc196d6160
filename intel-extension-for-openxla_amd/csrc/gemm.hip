// bf16 / fp16 GEMM with fp32 accumulation and a fused epilogue:
//     out = act(alpha * op(lhs) op(rhs) + beta * c + bias)
//
// MFMA kernel (gemm_mfma_kernel): one work-group owns a BM x BN tile of the output
// and walks K in steps of 64.  Both operand tiles are staged global -> registers ->
// LDS (double-buffered, one barrier per K step) so that the global loads of step
// t+1 are in flight while the matrix cores work on step t.  An operand whose
// reduction index is contiguous in memory ("KC": A[M,K] row-major, B stored [N,K])
// is kept in LDS as [row][64 k] with the 16-byte chunks of a row XOR-swizzled by
// the row number, and read with one ds_read_b128 per fragment.  An operand whose
// free index is contiguous ("MC": B[K,N] row-major, A stored [K,M]) is kept as
// [k][cols] with 64 bytes of padding per row and read with the LDS transpose
// loads (ds_read_b64_tr_b16), which hand each lane four consecutive k of one
// column.  The products are issued with the operands swapped (D^T = B^T A^T) so
// that a lane ends up holding four consecutive output columns of one row.
//
// Everything the MFMA kernel cannot take (fp32 or int8 operands, unaligned
// pointers or strides) runs gemm_generic_kernel, a plain LDS-tiled kernel; this is
// where the reference falls back to oneDNN (onednn_matmul_utils.cc:394-491).
#include <hip/hip_bf16.h>

#include <utility>

#include "common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int BK = 64;  // K step, elements

enum : int { ACT_NONE = 0, ACT_RELU = 1, ACT_GELU = 2 };

struct GemmParams {
  const void* a;
  const void* b;
  void* out;
  const void* c;
  const void* bias;
  int M, N, K;
  int64_t lda, ldb, ldc;        // elements between stored rows
  int64_t sa, sb, sc;           // batch strides, elements
  float alpha, beta;
  int act;
  int tiles_m, tiles_n;
};

__device__ __forceinline__ float gelu_tanh(float x) {
  // 0.5 x (1 + tanh(u)) = x * sigmoid(2u) = x / (1 + exp(-2u)), u = sqrt(2/pi)(x + 0.044715 x^3)
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  return x / (1.0f + __expf(-2.0f * u));
}

__device__ __forceinline__ float apply_act(float v, int act) {
  if (act == ACT_RELU) return fmaxf(v, 0.0f);
  if (act == ACT_GELU) return gelu_tanh(v);
  return v;
}

template <typename T> struct Elem;
template <> struct Elem<__bf16> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ floatx16 mfma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_f32(__bf16 v) { return (float)v; }
  static __device__ __forceinline__ uint16_t from_f32(float v) {
    __bf16 h = (__bf16)v;
    return __builtin_bit_cast(uint16_t, h);
  }
};
template <> struct Elem<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ floatx16 mfma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_f32(_Float16 v) { return (float)v; }
  static __device__ __forceinline__ uint16_t from_f32(float v) {
    _Float16 h = (_Float16)v;
    return __builtin_bit_cast(uint16_t, h);
  }
};

// Compile-time loop: f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>).  Used where
// an index into a register array must be a constant no matter what the unroller decides.
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

// LDS footprint of one operand tile of `rows` rows/columns.
template <bool MC> __host__ __device__ constexpr int tile_bytes(int rows) {
  return MC ? BK * (rows * 2 + 64) : rows * BK * 2;
}

// Buffer descriptor over [base, base + 2 GiB): loads whose byte offset is >= 2^31 (the
// sentinel kOob) return zero, which is how out-of-range rows / k are zero-filled.
constexpr uint32_t kOob = 0x80000000u;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)kOob, 0x00020000);
}

// Staging of one operand tile: NCH 16-byte chunks per thread, global -> registers -> LDS.
// The tile origin (first row/column, current k) lives in the scalar base of the buffer
// descriptor; a thread's byte offsets inside the tile never change, so the K loop does
// no per-chunk address arithmetic.
template <bool MC, int ROWS, int NT>
struct Stager {
  static constexpr int CHUNKS = ROWS * BK / 8;
  static constexpr int NCH = CHUNKS / NT;
  static_assert(CHUNKS % NT == 0, "tile does not divide over the threads");
  u32x4 r[NCH];
  uint32_t voff[NCH];   // byte offset of chunk i from the tile origin, or kOob
  int kin[NCH];         // k of chunk i relative to the K step

  // ld: elements between stored rows; valid: rows/cols of the tile that exist.
  __device__ __forceinline__ void init(int64_t ld, int valid, int tid) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int ch = tid + i * NT;
      int row, k;
      if constexpr (!MC) {
        row = ch / 8;
        k = (ch % 8) * 8;
      } else {
        k = ch / (ROWS / 8);
        row = (ch % (ROWS / 8)) * 8;
      }
      const int64_t e = MC ? (int64_t)k * ld + row : (int64_t)row * ld + k;
      voff[i] = row < valid ? (uint32_t)(e * 2) : kOob;
      kin[i] = k;
    }
  }
  // base: address of the tile origin for this K step; kleft: K - k0 (k of the step that exist).
  __device__ __forceinline__ void load(const void* base, int kleft) {
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(base);
    if (kleft >= BK) {
#pragma unroll
      for (int i = 0; i < NCH; ++i)
        r[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff[i], 0, 0));
    } else {
#pragma unroll
      for (int i = 0; i < NCH; ++i)
        r[i] = __builtin_bit_cast(
            u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, kin[i] < kleft ? voff[i] : kOob, 0, 0));
    }
  }
  __device__ __forceinline__ void store(char* lds, int tid) const {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int ch = tid + i * NT;
      int off;
      if constexpr (!MC) {
        const int row = ch / 8, c = ch % 8;
        off = row * (BK * 2) + ((c ^ (row & 7)) << 4);
      } else {
        const int k = ch / (ROWS / 8), c = ch % (ROWS / 8);
        off = k * (ROWS * 2 + 64) + (c << 4);
      }
      *reinterpret_cast<u32x4*>(lds + off) = r[i];
    }
  }
};

// Fragment of a 32-row (or 32-column) operand slab for k-step ks (16 k): lane l gets
// row l%32, k = 16 ks + 8 (l/32) .. +7.
template <bool MC, int ROWS, typename V8>
__device__ __forceinline__ V8 read_frag(const char* lds, int row0, int ks, int lane) {
  if constexpr (!MC) {
    const int row = row0 + (lane & 31);
    const int c = ks * 2 + (lane >> 5);
    const u32x4 v = *reinterpret_cast<const u32x4*>(lds + row * (BK * 2) + ((c ^ (row & 7)) << 4));
    return __builtin_bit_cast(V8, v);
  } else {
    // Transpose load: within a 16-lane block, lane p addresses row (kb + p/4), columns
    // (cb + 4 (p%4)) .. +3 and receives column cb + p, rows kb .. kb+3.
    const int p = lane & 15;
    const int cb = row0 + ((lane >> 4) & 1) * 16;
    const int kb = ks * 16 + (lane >> 5) * 8;
    const char* a0 = lds + (kb + (p >> 2)) * (ROWS * 2 + 64) + (cb + 4 * (p & 3)) * 2;
    typedef short4v __attribute__((address_space(3))) * lds_ptr;
    const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(a0));
    const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(a0 + 4 * (ROWS * 2 + 64)));
    u32x4 v;
    v[0] = __builtin_bit_cast(u32x2, lo)[0];
    v[1] = __builtin_bit_cast(u32x2, lo)[1];
    v[2] = __builtin_bit_cast(u32x2, hi)[0];
    v[3] = __builtin_bit_cast(u32x2, hi)[1];
    return __builtin_bit_cast(V8, v);
  }
}

// Epilogue for four consecutive output columns n..n+3 of row m held by one lane.
template <typename T, bool OutF32>
__device__ __forceinline__ void store_quad(const GemmParams& p, floatx4 a, int m, int n,
                                           int64_t coff) {
  if (m >= p.M || n >= p.N) return;
  const int64_t off = coff + (int64_t)m * p.ldc + n;
  const bool full = n + 4 <= p.N;
  float v0 = p.alpha * a[0], v1 = p.alpha * a[1], v2 = p.alpha * a[2], v3 = p.alpha * a[3];
  if (p.c) {  // non-null only when beta != 0
    float c0 = 0.f, c1 = 0.f, c2 = 0.f, c3 = 0.f;
    if constexpr (OutF32) {
      const float* cp = reinterpret_cast<const float*>(p.c) + off;
      c0 = cp[0];
      if (full || n + 1 < p.N) c1 = cp[1];
      if (full || n + 2 < p.N) c2 = cp[2];
      if (full) c3 = cp[3];
    } else {
      const T* cp = reinterpret_cast<const T*>(p.c) + off;
      c0 = Elem<T>::to_f32(cp[0]);
      if (full || n + 1 < p.N) c1 = Elem<T>::to_f32(cp[1]);
      if (full || n + 2 < p.N) c2 = Elem<T>::to_f32(cp[2]);
      if (full) c3 = Elem<T>::to_f32(cp[3]);
    }
    v0 += p.beta * c0; v1 += p.beta * c1; v2 += p.beta * c2; v3 += p.beta * c3;
  }
  if (p.bias) {
    const T* bp = reinterpret_cast<const T*>(p.bias) + n;
    v0 += Elem<T>::to_f32(bp[0]);
    if (full || n + 1 < p.N) v1 += Elem<T>::to_f32(bp[1]);
    if (full || n + 2 < p.N) v2 += Elem<T>::to_f32(bp[2]);
    if (full) v3 += Elem<T>::to_f32(bp[3]);
  }
  v0 = apply_act(v0, p.act); v1 = apply_act(v1, p.act);
  v2 = apply_act(v2, p.act); v3 = apply_act(v3, p.act);
  if constexpr (OutF32) {
    float* op = reinterpret_cast<float*>(p.out) + off;
    if (full && (off % 4 == 0)) {
      *reinterpret_cast<floatx4*>(op) = floatx4{v0, v1, v2, v3};
    } else {
      op[0] = v0;
      if (n + 1 < p.N) op[1] = v1;
      if (n + 2 < p.N) op[2] = v2;
      if (n + 3 < p.N) op[3] = v3;
    }
  } else {
    uint16_t* op = reinterpret_cast<uint16_t*>(p.out) + off;
    const uint16_t h0 = Elem<T>::from_f32(v0), h1 = Elem<T>::from_f32(v1);
    const uint16_t h2 = Elem<T>::from_f32(v2), h3 = Elem<T>::from_f32(v3);
    if (full && (off % 4 == 0)) {
      u32x2 w;
      w[0] = (uint32_t)h0 | ((uint32_t)h1 << 16);
      w[1] = (uint32_t)h2 | ((uint32_t)h3 << 16);
      *reinterpret_cast<u32x2*>(op) = w;
    } else {
      op[0] = h0;
      if (n + 1 < p.N) op[1] = h1;
      if (n + 2 < p.N) op[2] = h2;
      if (n + 3 < p.N) op[3] = h3;
    }
  }
}

// T: element type; OutF32: fp32 output (else T); A_MC / B_MC: operand's free index is
// contiguous; BM x BN tile; WGM x WGN waves.
template <typename T, bool OutF32, bool A_MC, bool B_MC, int BM, int BN, int WGM, int WGN>
__global__ __launch_bounds__(WGM * WGN * 64) void gemm_mfma_kernel(GemmParams p) {
  constexpr int NT = WGM * WGN * 64;
  constexpr int WTM = BM / WGM, WTN = BN / WGN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = tile_bytes<A_MC>(BM), B_BYTES = tile_bytes<B_MC>(BN);
  constexpr int STAGE = A_BYTES + B_BYTES;
  typedef typename Elem<T>::vec8 V8;
  __shared__ __attribute__((aligned(16))) char lds[2 * STAGE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;

  // Tile order: consecutive block ids land on different XCDs (8 of them, each with its
  // own L2), so give each XCD a contiguous run of tiles, and walk tiles in groups of 8
  // tile-rows so that a run re-uses the same A rows and B columns.
  int pid = blockIdx.x;
  const int ntiles = p.tiles_m * p.tiles_n;
  if (ntiles % 8 == 0) pid = (pid % 8) * (ntiles / 8) + pid / 8;
  constexpr int GM = 8;
  const int group = pid / (GM * p.tiles_n);
  const int first_m = group * GM;
  const int gsize = min(p.tiles_m - first_m, GM);
  const int tile_m = first_m + (pid % (GM * p.tiles_n)) % gsize;
  const int tile_n = (pid % (GM * p.tiles_n)) / gsize;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int64_t bz = blockIdx.z;
  const T* A = reinterpret_cast<const T*>(p.a) + bz * p.sa;
  const T* B = reinterpret_cast<const T*>(p.b) + bz * p.sb;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = zero16();

  Stager<A_MC, BM, NT> sa;
  Stager<B_MC, BN, NT> sb;
  const int KT = (p.K + BK - 1) / BK;
  sa.init(p.lda, p.M - m0, tid);
  sb.init(p.ldb, p.N - n0, tid);
  // Tile origins; one K step further is +BK elements (KC) or +BK rows (MC).
  const T* a_tile = A_MC ? A + m0 : A + (int64_t)m0 * p.lda;
  const T* b_tile = B_MC ? B + n0 : B + (int64_t)n0 * p.ldb;
  const int64_t a_step = A_MC ? BK * p.lda : BK;
  const int64_t b_step = B_MC ? BK * p.ldb : BK;

  sa.load(a_tile, p.K);
  sb.load(b_tile, p.K);
  sa.store(lds, tid);
  sb.store(lds + A_BYTES, tid);
  __syncthreads();

  // Fragments are double-buffered in registers: while the matrix cores work on k-step
  // ks, the LDS reads of k-step ks+1 are in flight.  The next K tile is written to the
  // other LDS buffer during k-step 2 and the barrier sits before k-step 3, so that
  // k-step 3 can already prefetch the first fragments of the next tile.
  V8 fa[2][TM], fb[2][TN];
  auto read_frags = [&](const char* stage, int ks, int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[buf][i] = read_frag<A_MC, BM, V8>(stage, wm * WTM + i * 32, ks, lane);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[buf][j] = read_frag<B_MC, BN, V8>(stage + A_BYTES, wn * WTN + j * 32, ks, lane);
  };
  auto mma = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = Elem<T>::mfma(fb[buf][j], fa[buf][i], acc[i][j]);
  };
  // One LDS read per MFMA until the reads of the step are issued.
  constexpr int READS = (A_MC ? 2 : 1) * TM + (B_MC ? 2 : 1) * TN;
  auto interleave = [&]() {
#pragma unroll
    for (int r = 0; r < READS; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 DS read
    }
  };

  read_frags(lds, 0, 0);
  for (int kt = 0; kt < KT; ++kt) {
    const char* cur = lds + (kt & 1) * STAGE;
    char* nxt = lds + ((kt + 1) & 1) * STAGE;
    const bool more = kt + 1 < KT;
    if (more) {
      a_tile += a_step;
      b_tile += b_step;
      sa.load(a_tile, p.K - (kt + 1) * BK);
      sb.load(b_tile, p.K - (kt + 1) * BK);
    }
    read_frags(cur, 1, 1);
    mma(0);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    read_frags(cur, 2, 0);
    mma(1);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    read_frags(cur, 3, 1);
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

  // Epilogue.  acc[i][j][e] is out[m][n] with m = m0 + wm WTM + 32 i + lane%32 and
  // n = n0 + wn WTN + 32 j + 8 (e/4) + 4 (lane/32) + e%4.
  const int64_t coff = bz * p.sc;
  static_for<TM>([&](auto I) {
    constexpr int i = decltype(I)::value;
    const int m = m0 + wm * WTM + i * 32 + (lane & 31);
    static_for<TN>([&](auto J) {
      constexpr int j = decltype(J)::value;
      const floatx16 t = acc[i][j];
      const int nb = n0 + wn * WTN + j * 32 + (lane >> 5) * 4;
      store_quad<T, OutF32>(p, floatx4{t[0], t[1], t[2], t[3]}, m, nb, coff);
      store_quad<T, OutF32>(p, floatx4{t[4], t[5], t[6], t[7]}, m, nb + 8, coff);
      store_quad<T, OutF32>(p, floatx4{t[8], t[9], t[10], t[11]}, m, nb + 16, coff);
      store_quad<T, OutF32>(p, floatx4{t[12], t[13], t[14], t[15]}, m, nb + 24, coff);
    });
  });
}

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
};

__global__ __launch_bounds__(256) void gemm_generic_kernel(GenericParams p) {
  __shared__ float As[16][65];
  __shared__ float Bs[16][65];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int64_t bz = blockIdx.z;
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
      if (p.bias) v += load_as_f32(p.bias, p.kin, n);
      v = apply_act(v, p.act);
      switch (p.kout) {
        case G_BF16: reinterpret_cast<__bf16*>(p.out)[off] = (__bf16)v; break;
        case G_F16: reinterpret_cast<_Float16*>(p.out)[off] = (_Float16)v; break;
        default: reinterpret_cast<float*>(p.out)[off] = v; break;
      }
    }
  }
}

// ------------------------------------------------------------------ host side

// Tile policies, the counterpart of the reference's gemm_policy list
// (xetla/gemm/gemm_dispatch.h:183-214).
struct Policy {
  const char* name;
  int bm, bn, wgm, wgn;
};
constexpr Policy kPolicies[] = {
    {"mfma_256x256_w2x2", 256, 256, 2, 2},
    {"mfma_128x128_w2x2", 128, 128, 2, 2},
    {"mfma_64x64_w2x2", 64, 64, 2, 2},
};
constexpr int kNumPolicies = sizeof(kPolicies) / sizeof(kPolicies[0]);

// Largest tile that still gives every CU of the device (256) work; the role of
// selectXetlaGemmConfig (xetla/gemm/gemm.cc:286-308), without a per-shape table.
int select_policy(int64_t m, int64_t n, int64_t k) {
  (void)k;
  for (int i = 0; i < kNumPolicies; ++i) {
    const int64_t tiles = xmk::ceil_div(m, kPolicies[i].bm) * xmk::ceil_div(n, kPolicies[i].bn);
    if (tiles >= 256 || i == kNumPolicies - 1) return i;
  }
  return kNumPolicies - 1;
}

template <typename T, bool OutF32, bool A_MC, bool B_MC, int BM, int BN, int WGM, int WGN>
void launch_mfma(const GemmParams& p, int batch, hipStream_t st) {
  hipLaunchKernelGGL((gemm_mfma_kernel<T, OutF32, A_MC, B_MC, BM, BN, WGM, WGN>),
                     dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(WGM * WGN * 64), 0, st, p);
}

template <typename T, bool OutF32, bool A_MC, bool B_MC>
void launch_policy(int pol, GemmParams& p, int batch, hipStream_t st) {
  p.tiles_m = (int)xmk::ceil_div(p.M, kPolicies[pol].bm);
  p.tiles_n = (int)xmk::ceil_div(p.N, kPolicies[pol].bn);
  switch (pol) {
    case 0: launch_mfma<T, OutF32, A_MC, B_MC, 256, 256, 2, 2>(p, batch, st); break;
    case 1: launch_mfma<T, OutF32, A_MC, B_MC, 128, 128, 2, 2>(p, batch, st); break;
    default: launch_mfma<T, OutF32, A_MC, B_MC, 64, 64, 2, 2>(p, batch, st); break;
  }
}

template <typename T, bool OutF32>
void launch_layout(bool a_mc, bool b_mc, int pol, GemmParams& p, int batch, hipStream_t st) {
  if (!a_mc && !b_mc) launch_policy<T, OutF32, false, false>(pol, p, batch, st);
  else if (!a_mc && b_mc) launch_policy<T, OutF32, false, true>(pol, p, batch, st);
  else if (a_mc && !b_mc) launch_policy<T, OutF32, true, false>(pol, p, batch, st);
  else launch_policy<T, OutF32, true, true>(pol, p, batch, st);
}

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
  (void)rhs_transpose;
  const bool sixteen = dtype_in == XMK_BF16 || dtype_in == XMK_F16;
  if (!sixteen || !(dtype_out == dtype_in || dtype_out == XMK_F32)) return "generic_64x64";
  return kPolicies[select_policy(m, n, k)].name;
}

extern "C" int xmk_gemm(const xmk_gemm_desc* d, void* stream) {
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

  hipStream_t st = (hipStream_t)stream;
  const bool sixteen = din == XMK_BF16 || din == XMK_F16;
  const bool fast = sixteen && xmk::aligned(lhs.data, 16) && xmk::aligned(rhs.data, 16) &&
                    xmk::aligned(out.data, 16) && lhs.leading_dim_stride % 8 == 0 &&
                    rhs.leading_dim_stride % 8 == 0 && lhs.batch_stride % 8 == 0 &&
                    rhs.batch_stride % 8 == 0 && lhs.num_cols % 8 == 0 && rhs.num_cols % 8 == 0;
  if (fast) {
    GemmParams p;
    p.a = lhs.data; p.b = rhs.data; p.out = out.data; p.c = d->beta != 0.0f ? d->c : nullptr;
    p.bias = wants_bias ? d->bias : nullptr;
    p.M = (int)m; p.N = (int)n; p.K = (int)k;
    p.lda = lhs.leading_dim_stride; p.ldb = rhs.leading_dim_stride; p.ldc = out.leading_dim_stride;
    p.sa = lhs.batch_stride; p.sb = rhs.batch_stride; p.sc = out.batch_stride;
    p.alpha = d->alpha; p.beta = d->beta; p.act = act;
    const bool a_mc = lhs.transpose != 0;   // stored [K, M]
    const bool b_mc = rhs.transpose == 0;   // stored [K, N]
    const int pol = select_policy(m, n, k);
    xmk::trace("gemm m=%lld n=%lld k=%lld batch=%lld lhs_t=%d rhs_t=%d epilogue=%d beta=%g -> %s",
               (long long)m, (long long)n, (long long)k, (long long)d->batch_size, lhs.transpose,
               rhs.transpose, d->epilogue, d->beta, kPolicies[pol].name);
    const int batch = (int)d->batch_size;
    if (din == XMK_BF16) {
      if (dout == XMK_F32) launch_layout<__bf16, true>(a_mc, b_mc, pol, p, batch, st);
      else launch_layout<__bf16, false>(a_mc, b_mc, pol, p, batch, st);
    } else {
      if (dout == XMK_F32) launch_layout<_Float16, true>(a_mc, b_mc, pol, p, batch, st);
      else launch_layout<_Float16, false>(a_mc, b_mc, pol, p, batch, st);
    }
    return xmk::check_launch("gemm");
  }

  if (din == XMK_S8 && (d->alpha != 1.0f || d->beta != 0.0f || d->epilogue != XMK_EPI_DEFAULT))
    return xmk::fail(XMK_UNIMPLEMENTED, "gemm: s8 x s8 -> s32 supports alpha=1, beta=0, no epilogue");
  GenericParams g;
  g.a = lhs.data; g.b = rhs.data; g.out = out.data; g.c = d->beta != 0.0f ? d->c : nullptr;
  g.bias = wants_bias ? d->bias : nullptr;
  g.M = (int)m; g.N = (int)n; g.K = (int)k;
  g.lda = lhs.leading_dim_stride; g.ldb = rhs.leading_dim_stride; g.ldc = out.leading_dim_stride;
  g.sa = lhs.batch_stride; g.sb = rhs.batch_stride; g.sc = out.batch_stride;
  g.ta = lhs.transpose; g.tb = rhs.transpose;
  g.kin = generic_kind(din); g.kout = generic_kind(dout);
  g.alpha = d->alpha; g.beta = d->beta; g.act = act;
  xmk::trace("gemm m=%lld n=%lld k=%lld -> generic_64x64", (long long)m, (long long)n, (long long)k);
  hipLaunchKernelGGL(gemm_generic_kernel,
                     dim3((unsigned)xmk::ceil_div(n, 64), (unsigned)xmk::ceil_div(m, 64),
                          (unsigned)d->batch_size),
                     dim3(256), 0, st, g);
  return xmk::check_launch("gemm");
}
