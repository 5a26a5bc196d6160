// MFMA GEMM kernel and its launch templates (included by gemm.hip for the host API and by the
// gemm_inst_*.hip units, each of which instantiates one (element type, output type) pair so
// that the instantiations compile in parallel).
#pragma once
#include <hip/hip_bf16.h>

#include <cstdlib>
#include <utility>

#include "common.h"

namespace gemm_impl {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));


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
  // Shared-lhs multi-output form (three GEMMs with one A): batch member z > 0 writes to
  // out_alt[z - 1] instead of out + z * sc and reads bias + z * sbias.  Null when unused.
  void* out_alt[2];
  int64_t sbias;
  // Gathering kernel only: elements per load (1, 2, 4 or 8) that the alignment of each operand's
  // pointer, leading dimension, batch stride and row length allows.
  int vec_a, vec_b;
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

// Buffer descriptor over [base, base + 2 GiB): loads whose byte offset is >= 2^31 (the
// sentinel kOob) return zero, which is how out-of-range rows / k are zero-filled.
constexpr uint32_t kOob = 0x80000000u;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)kOob, 0x00020000);
}

typedef __attribute__((address_space(3))) void* lds_void_ptr;

// XOR applied to the 16-byte chunk index inside an LDS row, chosen so that the lanes the LDS serves
// together touch different banks (256 bytes of banks).
//   KC, BK = 64: rows of 128 bytes (8 chunks); KC, BK = 32: rows of 64 bytes (4 chunks); read with
//       ds_read_b128, 16 lanes = 16 rows of one chunk column.  Two (four) rows share 256 bytes of banks and
//       are apart by their position there, so the XOR counts pairs (quadruples) of rows.
//   MC: rows of ROWS * 2 bytes, read with the LDS transpose loads.  16-bit elements (EB = 2,
//       ds_read_b64_tr_b16): 32 lanes take 64 bytes of each of 4 consecutive k rows, so rows of 256 bytes and
//       more move by whole 64-byte groups, (k & 3) << 2; with 128-byte rows two rows share the banks and
//       (k & 3) << 1 separates the four.  8-bit elements (EB = 1, ds_read_b64_tr_b8): 32 lanes take 32 bytes of
//       each of 8 consecutive k rows, (k & 7) << 1 (rows of 256 bytes and more).  The XOR is even so that 32-byte pairs
//       stay together.
template <bool MC, int ROWS, int BK, int EB = 2>
__device__ __forceinline__ int swz(int row_or_k) {
  if constexpr (!MC) return BK == 64 ? ((row_or_k >> 1) & 7) : ((row_or_k >> 2) & 3);
  else if constexpr (ROWS < 128) return (row_or_k & 3) << 1;  // 8 chunks per row: the XOR stays below 8
  else if constexpr (EB == 1) return (row_or_k & 7) << 1;
  else return (row_or_k & 3) << 2;
}

// One operand tile = BK k x ROWS rows/cols = ROWS * BK * 2 bytes of LDS in both layouts.
// A wave issues NL loads of 1 KiB per K step; load j = i * NWAVES + wave (i = 0..NL-1) fills
// LDS bytes [1024 j, 1024 j + 1024).  The swizzle is chosen so that a lane fetches the same
// chunk column in every load: its global byte offset is voff + i * sstride, with voff in one
// VGPR and the per-load part in the instruction's scalar offset.  Row/column validity is
// kept as one lane mask per load (scalar registers).
template <bool MC, int ROWS, int BK, int NWAVES, int EB = 2>
struct Loader {
  static constexpr int RB = MC ? ROWS * 2 : BK * 2;  // LDS row, bytes
  static constexpr int CPR = RB / 16;                // chunks per LDS row
  static constexpr int RPL = 1024 / RB;              // LDS rows per load
  static constexpr int NL = ROWS * BK * 2 / 1024 / NWAVES;
  static constexpr int LSTRIDE = NWAVES * RPL;       // LDS rows between consecutive loads of a wave
  static_assert(NL >= 1, "tile too small for this many waves");
  static_assert(LSTRIDE % 16 == 0 || (LSTRIDE % 8 == 0 && (MC || BK == 32)), "swizzle must repeat from load to load");
  uint32_t voff;     // byte offset of this lane's chunk in load 0, from the tile origin
  uint32_t sstride;  // bytes between consecutive loads of this wave (uniform)
  int kin0;          // k (inside the K step) of this lane's chunk in load 0
  bool ok[NL];       // this lane's row / column exists
  uint32_t okoff[NL];  // ok[i] ? voff : kOob -- the offset of load i in a K step that lies fully inside K

  __device__ __forceinline__ void init(int64_t ld, int valid, int wave, int lane) {
    const int lrow = wave * RPL + lane / CPR;  // LDS row in load 0: operand row (KC) or k (MC)
    const int chunk = (lane % CPR) ^ swz<MC, ROWS, BK, EB>(lrow);
    voff = (uint32_t)(((int64_t)lrow * ld + chunk * 8) * 2);
    sstride = (uint32_t)(LSTRIDE * ld * 2);
    if constexpr (!MC) {
      kin0 = chunk * 8;
#pragma unroll
      for (int i = 0; i < NL; ++i) ok[i] = lrow + i * LSTRIDE < valid;
    } else {
      kin0 = lrow;
#pragma unroll
      for (int i = 0; i < NL; ++i) ok[i] = chunk * 8 < valid;
    }
#pragma unroll
    for (int i = 0; i < NL; ++i) okoff[i] = ok[i] ? voff : kOob;
  }
  // Issues load i.  base: address of the tile origin for this K step; kleft: k of the step that
  // exist (<= 0 past the end of K: every lane is then out of range and the load writes zeros).
  // CHECK_K = false: the caller knows that the whole K step exists (kleft >= BK).
  template <bool CHECK_K = true>
  __device__ __forceinline__ void issue_one(int i, __amdgpu_buffer_rsrc_t rsrc, int kleft, char* lds_tile,
                                            int wave) const {
    const int k = MC ? kin0 + i * LSTRIDE : kin0;
    const uint32_t off = CHECK_K ? ((ok[i] && k < kleft) ? voff : kOob) : okoff[i];
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr)(lds_tile + (i * NWAVES + wave) * 1024), 16,
                                             off, i * sstride, 0, 0);
  }
  __device__ __forceinline__ void issue(const void* base, int kleft, char* lds_tile, int wave) const {
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(base);
#pragma unroll
    for (int i = 0; i < NL; ++i) issue_one(i, rsrc, kleft, lds_tile, wave);
  }
  // The same placement for operands the direct loads cannot take (rows that do not start on a
  // 16-byte boundary, a row length that is not a multiple of 8): load i's chunk is gathered element
  // by element, zero where the row, column or k does not exist, and written with one 16-byte LDS
  // store.  Nothing outside the matrix is read.  base: tile origin for this K step; valid: rows
  // (KC) or columns (MC) of the tile that exist; kleft as in issue_one; vec: elements per load
  // (wave-uniform; every group of `vec` elements is aligned and lies inside the row or outside as a whole).
  __device__ __forceinline__ void gather_one(int i, const uint16_t* base, int64_t ld, int valid, int kleft,
                                             char* lds_tile, int wave, int lane, int vec) const {
    scatter_one(i, gather_load(i, base, ld, valid, kleft, wave, lane, vec), lds_tile, wave, lane);
  }
  __device__ __forceinline__ void scatter_one(int i, u32x4 v, char* lds_tile, int wave, int lane) const {
    *reinterpret_cast<u32x4*>(lds_tile + (i * NWAVES + wave) * 1024 + lane * 16) = v;
  }
  __device__ __forceinline__ u32x4 gather_load(int i, const uint16_t* base, int64_t ld, int valid, int kleft,
                                               int wave, int lane, int vec) const {
    const int lrow = wave * RPL + lane / CPR + i * LSTRIDE;                       // LSTRIDE % 8 == 0:
    const int c0 = ((lane % CPR) ^ swz<MC, ROWS, BK, EB>(wave * RPL + lane / CPR)) * 8;  // same swizzle for every i
    const int row = MC ? c0 : lrow;   // operand row / column of element 0
    const int k = MC ? lrow : c0;     // k (inside the K step) of element 0
    const uint16_t* src = MC ? base + (int64_t)k * ld + row : base + (int64_t)row * ld + k;
    const bool line = MC ? k < kleft : row < valid;  // the stored row this chunk lies in exists
    const int left = MC ? valid - row : kleft - k;    // elements of that row from element 0 on
    u32x4 v = {0u, 0u, 0u, 0u};
    if (vec == 8) {
      if (line && left > 0) v = *reinterpret_cast<const u32x4*>(src);
    } else if (vec == 4) {
#pragma unroll
      for (int j = 0; j < 2; ++j)
        if (line && 4 * j < left) {
          const u32x2 w = *reinterpret_cast<const u32x2*>(src + 4 * j);
          v[2 * j] = w[0];
          v[2 * j + 1] = w[1];
        }
    } else if (vec == 2) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (line && 2 * j < left) v[j] = *reinterpret_cast<const uint32_t*>(src + 2 * j);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (line && j < left) v[j >> 1] |= (uint32_t)src[j] << (16 * (j & 1));
    }
    return v;
  }
};

// Per-lane LDS byte offsets of an operand's fragments, computed once.  A fragment of the
// 32-row (or 32-column) slab t for k-step ks (16 k) gives lane l row l%32, k = 16 ks + 8 (l/32)..+7.
//   KC: one 16-byte read at base[ks] + t * 32 * RB          (the XOR depends on ks, not on t)
//   MC: two transpose reads (k .. k+3 and k+4 .. k+7 of one column) at base[t][h] + ks * 16 * RB
//       (the XOR depends on t and h, not on ks)
template <bool MC, int ROWS, int BK, int T>
struct FragAddr {
  static constexpr int KS = BK / 16;
  int base[MC ? T : KS][MC ? 2 : 1];
  __device__ __forceinline__ void init(int row0, int lane) {
    if constexpr (!MC) {
      const int row = row0 + (lane & 31);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        base[ks][0] = row * (BK * 2) + (((ks * 2 + (lane >> 5)) ^ swz<false, ROWS, BK>(row)) << 4);
    } else {
      // Within a 16-lane block, lane p addresses row (kb + p/4), columns (cb + 4 (p%4)) .. +3
      // and receives column cb + p, rows kb .. kb+3.
      const int p = lane & 15;
#pragma unroll
      for (int t = 0; t < T; ++t) {
        const int col = row0 + t * 32 + ((lane >> 4) & 1) * 16 + 4 * (p & 3);
        const int chunk = col >> 3, within = (col & 7) * 2;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int k = (lane >> 5) * 8 + (p >> 2) + 4 * h;  // + 16 ks, which does not change k & 7
          base[t][h] = k * (ROWS * 2) + ((chunk ^ swz<true, ROWS, BK>(k)) << 4) + within;
        }
      }
    }
  }
  template <typename V8>
  __device__ __forceinline__ V8 read(const char* __restrict__ tile, int t, int ks) const {
    if constexpr (!MC) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(tile + base[ks][0] + t * 32 * (BK * 2));
      return __builtin_bit_cast(V8, v);
    } else {
      typedef short4v __attribute__((address_space(3))) * lds_ptr;
      const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile + base[t][0] + ks * 16 * (ROWS * 2)));
      const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile + base[t][1] + ks * 16 * (ROWS * 2)));
      u32x4 v;
      v[0] = __builtin_bit_cast(u32x2, lo)[0];
      v[1] = __builtin_bit_cast(u32x2, lo)[1];
      v[2] = __builtin_bit_cast(u32x2, hi)[0];
      v[3] = __builtin_bit_cast(u32x2, hi)[1];
      return __builtin_bit_cast(V8, v);
    }
  }
};

// s_waitcnt immediate (gfx9 encoding) that waits until at most n vector-memory loads are
// outstanding and does not wait on the other counters.
__host__ __device__ constexpr int vmcnt_imm(int n) {
  return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4) | (0xf << 8);
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

// The epilogue's arithmetic for four consecutive columns n..n+3 of row m that lie inside the matrix.
// PLAIN: alpha == 1 and no addend, bias or activation.
template <typename T, bool PLAIN>
__device__ __forceinline__ floatx4 quad_values(const GemmParams& p, floatx4 a, int m, int n, int64_t coff) {
  if constexpr (PLAIN) return a;
  float v0 = p.alpha * a[0], v1 = p.alpha * a[1], v2 = p.alpha * a[2], v3 = p.alpha * a[3];
  if (p.c) {
    const u32x2 cw = *reinterpret_cast<const u32x2*>(reinterpret_cast<const T*>(p.c) + coff + (int64_t)m * p.ldc + n);
    const T* cp = reinterpret_cast<const T*>(&cw);
    v0 += p.beta * Elem<T>::to_f32(cp[0]); v1 += p.beta * Elem<T>::to_f32(cp[1]);
    v2 += p.beta * Elem<T>::to_f32(cp[2]); v3 += p.beta * Elem<T>::to_f32(cp[3]);
  }
  if (p.bias) {
    const T* bp = reinterpret_cast<const T*>(p.bias) + n;
    v0 += Elem<T>::to_f32(bp[0]); v1 += Elem<T>::to_f32(bp[1]);
    v2 += Elem<T>::to_f32(bp[2]); v3 += Elem<T>::to_f32(bp[3]);
  }
  return floatx4{apply_act(v0, p.act), apply_act(v1, p.act), apply_act(v2, p.act), apply_act(v3, p.act)};
}

// Epilogue of a tile that lies fully inside a 16-bit output matrix: each wave rounds its WTM x WTN
// part, lays it out row-major in its own LDS region, and copies the region out with 16-byte stores
// that cover whole row segments (the accumulator layout itself gives a lane 8 bytes in each of 32
// different rows per store).  XOR on the 16-byte chunk index keeps both passes off the same banks.
// vec: elements per global store (8, 4, 2 or 1) that the output's alignment allows; a lane always
// owns 8 consecutive elements of a row.
template <typename T, bool PLAIN, int WTM, int WTN, int TM, int TN>
__device__ __forceinline__ void store_tile_via_lds(const GemmParams& q, const floatx16 (&acc)[TM][TN], char* region,
                                                   int m_base, int n_base, int64_t coff, int lane, int vec = 8) {
  constexpr int RBY = WTN * 2;       // bytes per row of the region
  constexpr int CPRW = RBY / 16;     // 16-byte chunks per row (4, 8 or 16)
  constexpr int RDIV = 16 / CPRW;    // rows that share one 256-byte bank sweep
  static_assert(CPRW == 4 || CPRW == 8 || CPRW == 16, "unsupported wave tile width");
  const int r1 = lane & 31;
  const int s1 = (r1 / RDIV) & (CPRW - 1);
  static_for<TM>([&](auto I) {
    constexpr int i = decltype(I)::value;
    static_for<TN>([&](auto J) {
      constexpr int j = decltype(J)::value;
      const floatx16 t = acc[i][j];
      static_for<4>([&](auto Q) {
        constexpr int qd = decltype(Q)::value;
        const floatx4 v = quad_values<T, PLAIN>(q, floatx4{t[4 * qd], t[4 * qd + 1], t[4 * qd + 2], t[4 * qd + 3]},
                                                m_base + i * 32 + r1, n_base + j * 32 + 8 * qd + 4 * (lane >> 5), coff);
        u32x2 w;
        w[0] = (uint32_t)Elem<T>::from_f32(v[0]) | ((uint32_t)Elem<T>::from_f32(v[1]) << 16);
        w[1] = (uint32_t)Elem<T>::from_f32(v[2]) | ((uint32_t)Elem<T>::from_f32(v[3]) << 16);
        *reinterpret_cast<u32x2*>(region + (i * 32 + r1) * RBY + (((4 * j + qd) ^ s1) << 4) + (lane >> 5) * 8) = w;
      });
    });
  });
  constexpr int RPI = 64 / CPRW;  // rows per copy instruction
  uint16_t* out = reinterpret_cast<uint16_t*>(q.out) + coff + (int64_t)m_base * q.ldc + n_base + (lane % CPRW) * 8;
#pragma unroll 4
  for (int it = 0; it < WTM / RPI; ++it) {
    const int row = it * RPI + lane / CPRW;
    const int chunk = (lane % CPRW) ^ ((row / RDIV) & (CPRW - 1));
    const u32x4 v = *reinterpret_cast<const u32x4*>(region + row * RBY + (chunk << 4));
    uint16_t* dst = out + (int64_t)row * q.ldc;
    if (vec == 8) {
      *reinterpret_cast<u32x4*>(dst) = v;
    } else if (vec == 4) {
      *reinterpret_cast<u32x2*>(dst) = u32x2{v[0], v[1]};
      *reinterpret_cast<u32x2*>(dst + 4) = u32x2{v[2], v[3]};
    } else if (vec == 2) {
#pragma unroll
      for (int j = 0; j < 4; ++j) *reinterpret_cast<uint32_t*>(dst + 2 * j) = v[j];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) dst[j] = (uint16_t)(v[j >> 1] >> (16 * (j & 1)));
    }
  }
}

// T: element type; OutF32: fp32 output (else T); A_MC / B_MC: operand's free index is
// contiguous; BM x BN tile; WGM x WGN waves; BK: K step (32 or 64); NSTAGE: LDS stages.
// SLOW: operands are gathered element by element (Loader::gather_one) instead of loaded directly
// into LDS; for leading dimensions and row lengths the direct loads cannot take.
template <typename T, bool OutF32, bool A_MC, bool B_MC, int BM, int BN, int WGM, int WGN, int BK, int NSTAGE,
          bool SLOW = false>
__global__ __launch_bounds__(WGM * WGN * 64) void gemm_mfma_kernel(GemmParams p) {
  constexpr int WTM = BM / WGM, WTN = BN / WGN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int NWAVES = WGM * WGN;
  constexpr int KS = BK / 16;  // 16-wide k-steps per K step
  constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  constexpr int STAGE = A_BYTES + B_BYTES;
  typedef typename Elem<T>::vec8 V8;
  typedef Loader<A_MC, BM, BK, NWAVES> LoaderA;
  typedef Loader<B_MC, BN, BK, NWAVES> LoaderB;
  __shared__ __attribute__((aligned(1024))) char lds[NSTAGE * STAGE];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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

  LoaderA la;
  LoaderB lb;
  const int KT = (p.K + BK - 1) / BK;
  la.init(p.lda, p.M - m0, wave, lane);
  lb.init(p.ldb, p.N - n0, wave, lane);
  // Tile origins; one K step further is +BK elements (KC) or +BK rows (MC).
  const T* a_tile = A_MC ? A + m0 : A + (int64_t)m0 * p.lda;
  const T* b_tile = B_MC ? B + n0 : B + (int64_t)n0 * p.ldb;
  const int64_t a_step = A_MC ? BK * p.lda : BK;
  const int64_t b_step = B_MC ? BK * p.ldb : BK;
  constexpr int LOADS = LoaderA::NL + LoaderB::NL;  // per wave per K step

  // Prologue: K steps 0 .. NSTAGE-2 go to stages 0 .. NSTAGE-2.  Loads past the end of K are
  // out of range and write zeros, so every step issues the same number of loads and the
  // vmcnt arithmetic below is uniform.
#pragma unroll
  for (int st = 0; st < NSTAGE - 1; ++st) {
    if constexpr (SLOW) {
#pragma unroll
      for (int i = 0; i < LoaderA::NL; ++i)
        la.gather_one(i, reinterpret_cast<const uint16_t*>(a_tile), p.lda, p.M - m0, p.K - st * BK,
                      lds + st * STAGE, wave, lane, p.vec_a);
#pragma unroll
      for (int i = 0; i < LoaderB::NL; ++i)
        lb.gather_one(i, reinterpret_cast<const uint16_t*>(b_tile), p.ldb, p.N - n0, p.K - st * BK,
                      lds + st * STAGE + A_BYTES, wave, lane, p.vec_b);
    } else {
      la.issue(a_tile, p.K - st * BK, lds + st * STAGE, wave);
      lb.issue(b_tile, p.K - st * BK, lds + st * STAGE + A_BYTES, wave);
    }
    a_tile += a_step;
    b_tile += b_step;
  }
  if constexpr (SLOW) __builtin_amdgcn_s_waitcnt(0xc07f);                   // the gathers' LDS stores are done
  else __builtin_amdgcn_s_waitcnt(vmcnt_imm((NSTAGE - 2) * LOADS));         // step 0 has landed (loads return in order)
  __builtin_amdgcn_s_barrier();

  FragAddr<A_MC, BM, BK, TM> faddr;
  FragAddr<B_MC, BN, BK, TN> fbddr;
  faddr.init(wm * WTM, lane);
  fbddr.init(wn * WTN, lane);

  // Fragments are double-buffered in registers: while the matrix cores work on k-step ks,
  // the LDS reads of k-step ks+1 are in flight.
  V8 fa[2][TM], fb[2][TN];
  auto read_frags = [&](const char* __restrict__ stage, int ks, int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[buf][i] = faddr.template read<V8>(stage, i, ks);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[buf][j] = fbddr.template read<V8>(stage + A_BYTES, j, ks);
  };
  auto mma = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int jj = (i & 1) ? TN - 1 - j : j;  // boustrophedon: consecutive MFMAs share one operand
        acc[i][jj] = Elem<T>::mfma(fb[buf][jj], fa[buf][i], acc[i][jj]);
      }
  };
  constexpr int READS = (A_MC ? 2 : 1) * TM + (B_MC ? 2 : 1) * TN;
  constexpr int NMFMA = TM * TN;
  // Instruction mix of one k-step: after every MFMA one LDS read (while there are any) and,
  // spread evenly over the MFMAs, `nloads` global loads.
  auto interleave = [&](int nloads) {
#pragma unroll
    for (int r = 0; r < NMFMA; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 // 1 MFMA
      if (r < READS) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 DS read
      if ((r + 1) * nloads / NMFMA > r * nloads / NMFMA)
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);               // 1 VMEM read
    }
  };
  // One K step: compute from stage `cur`, prefetch the first fragments of stage `nxt`, and fill
  // stage `wr` with K step kt + NSTAGE - 1.  The three stages are distinct; saying so
  // (__restrict__) lets the compiler keep the LDS-DMA loads in flight across the fragment reads
  // instead of waiting for them before every LDS read.  What must be waited for is written out:
  // before the barrier, all but the youngest (NSTAGE-2) steps' loads of this wave have landed
  // (loads return in order), so step kt + 1 is complete once every wave has arrived, and this
  // wave's reads of `cur` are done, so `cur` may be overwritten by the loads the next step issues.
  auto k_step = [&](auto CHECK, const char* __restrict__ cur, const char* __restrict__ nxt, char* __restrict__ wr,
                    int kt) {
    constexpr bool CHECK_K = decltype(CHECK)::value;
    const int kleft = p.K - (kt + NSTAGE - 1) * BK;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(a_tile), rb = make_rsrc(b_tile);
    // Gathering kernel: the whole K step's operand chunks are loaded into registers up front and go
    // to LDS after the step's MFMAs, which cover most of the load latency.
    u32x4 ga[SLOW ? LoaderA::NL : 1], gb[SLOW ? LoaderB::NL : 1];
    if constexpr (SLOW) {
#pragma unroll
      for (int i = 0; i < LoaderA::NL; ++i)
        ga[i] = la.gather_load(i, reinterpret_cast<const uint16_t*>(a_tile), p.lda, p.M - m0, kleft, wave, lane, p.vec_a);
#pragma unroll
      for (int i = 0; i < LoaderB::NL; ++i)
        gb[i] = lb.gather_load(i, reinterpret_cast<const uint16_t*>(b_tile), p.ldb, p.N - n0, kleft, wave, lane, p.vec_b);
    }
    static_for<KS>([&](auto KSI) {
      constexpr int ks = decltype(KSI)::value;
      // this k-step's share of the loads
      constexpr int la0 = LoaderA::NL * ks / KS, la1 = LoaderA::NL * (ks + 1) / KS;
      constexpr int lb0 = LoaderB::NL * ks / KS, lb1 = LoaderB::NL * (ks + 1) / KS;
      if constexpr (ks + 1 == KS) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((NSTAGE - 3) * LOADS + LoaderA::NL * ks / KS + LoaderB::NL * ks / KS) &
                                   ~(0xf << 8));  // and lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
      }
      if constexpr (!SLOW) {
#pragma unroll
        for (int i = la0; i < la1; ++i) la.template issue_one<CHECK_K>(i, ra, kleft, wr, wave);
#pragma unroll
        for (int i = lb0; i < lb1; ++i) lb.template issue_one<CHECK_K>(i, rb, kleft, wr + A_BYTES, wave);
      }
      if constexpr (ks + 1 < KS) read_frags(cur, ks + 1, (ks + 1) & 1);
      else read_frags(nxt, 0, KS & 1);
      mma(ks & 1);
      interleave(SLOW ? 0 : (la1 - la0) + (lb1 - lb0));
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (SLOW && ks + 1 == KS) {
#pragma unroll
        for (int i = 0; i < LoaderA::NL; ++i) la.scatter_one(i, ga[i], wr, wave, lane);
#pragma unroll
        for (int i = 0; i < LoaderB::NL; ++i) lb.scatter_one(i, gb[i], wr + A_BYTES, wave, lane);
        __builtin_amdgcn_sched_barrier(0);
      }
    });
    a_tile += a_step;
    b_tile += b_step;
  };

  static_assert(KS % 2 == 0, "fragment double-buffering assumes an even number of k-steps");
  static_assert(NSTAGE >= 3, "the barrier leaves the running step's loads in flight");
  read_frags(lds, 0, 0);
  // Step kt loads K step kt + NSTAGE - 1: all of it exists until that index reaches the last
  // (possibly partial) step, so only the final NSTAGE - 1 iterations (and a partial last K step)
  // need the per-lane K test.
  const int kt_full = min(KT, p.K / BK - (NSTAGE - 1));
  int kt = 0;
  for (; kt < kt_full; ++kt)
    k_step(std::false_type{}, lds + (kt % NSTAGE) * STAGE, lds + ((kt + 1) % NSTAGE) * STAGE,
           lds + ((kt + NSTAGE - 1) % NSTAGE) * STAGE, kt);
  for (; kt < KT; ++kt)
    k_step(std::true_type{}, lds + (kt % NSTAGE) * STAGE, lds + ((kt + 1) % NSTAGE) * STAGE,
           lds + ((kt + NSTAGE - 1) % NSTAGE) * STAGE, kt);
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // drain the zero-fill loads before LDS is released

  // Epilogue.  acc[i][j][e] is out[m][n] with m = m0 + wm WTM + 32 i + lane%32 and
  // n = n0 + wn WTN + 32 j + 8 (e/4) + 4 (lane/32) + e%4.
  const int64_t coff = bz * p.sc;
  GemmParams q = p;  // this batch member's view of the output and bias
  if (p.out_alt[0] && bz > 0) q.out = p.out_alt[bz - 1];
  if (p.bias) q.bias = reinterpret_cast<const T*>(p.bias) + bz * p.sbias;
  if constexpr (!OutF32) {
    static_assert(NSTAGE * STAGE >= BM * BN * 2, "the output tile is staged in the operand stages");
    const bool inside = m0 + BM <= p.M && n0 + BN <= p.N &&
                        (!p.c || (p.ldc % 4 == 0 && (reinterpret_cast<uintptr_t>(p.c) + coff * 2) % 8 == 0));
    if (inside) {                      // uniform over the work-group
      __builtin_amdgcn_s_barrier();    // every wave has read its last fragments
      char* region = lds + wave * (WTM * WTN * 2);
      const int mb = m0 + wm * WTM, nb = n0 + wn * WTN;
      int vec = 8;  // widest store that every row start of this batch member's output allows
      while (vec > 1 && (p.ldc % vec != 0 || (reinterpret_cast<uintptr_t>(q.out) + coff * 2) % (2 * vec) != 0))
        vec >>= 1;
      if (p.alpha == 1.0f && !p.c && !p.bias && p.act == ACT_NONE)
        store_tile_via_lds<T, true, WTM, WTN, TM, TN>(q, acc, region, mb, nb, coff, lane, vec);
      else
        store_tile_via_lds<T, false, WTM, WTN, TM, TN>(q, acc, region, mb, nb, coff, lane, vec);
      return;
    }
  }
  static_for<TM>([&](auto I) {
    constexpr int i = decltype(I)::value;
    const int m = m0 + wm * WTM + i * 32 + (lane & 31);
    static_for<TN>([&](auto J) {
      constexpr int j = decltype(J)::value;
      const floatx16 t = acc[i][j];
      const int nb = n0 + wn * WTN + j * 32 + (lane >> 5) * 4;
      store_quad<T, OutF32>(q, floatx4{t[0], t[1], t[2], t[3]}, m, nb, coff);
      store_quad<T, OutF32>(q, floatx4{t[4], t[5], t[6], t[7]}, m, nb + 8, coff);
      store_quad<T, OutF32>(q, floatx4{t[8], t[9], t[10], t[11]}, m, nb + 16, coff);
      store_quad<T, OutF32>(q, floatx4{t[12], t[13], t[14], t[15]}, m, nb + 24, coff);
    });
  });
}

// Tile policies, the counterpart of the reference's gemm_policy list
// (xetla/gemm/gemm_dispatch.h:183-214).
struct Policy {
  const char* name;
  int bm, bn, wgm, wgn, bk, stages;
};
constexpr Policy kPolicies[] = {
    {"mfma_256x256x32_w2x2_s4", 256, 256, 2, 2, 32, 4},
    {"mfma_128x128x64_w2x2_s3", 128, 128, 2, 2, 64, 3},
    {"mfma_128x64x64_w2x2_s4", 128, 64, 2, 2, 64, 4},
    {"mfma_64x64x64_w2x2_s4", 64, 64, 2, 2, 64, 4},
    {"mfma_256x128x64_w2x2_s3", 256, 128, 2, 2, 64, 3},
    // not a matrix-core tile: the streaming kernel for up to eight rows (gemm_rows.hip), eight waves
    // that split the reduction of a 512-column block
    {"stream_rows_8x512_w8", 8, 512, 8, 1, 8, 2},
};
constexpr int kNumPolicies = sizeof(kPolicies) / sizeof(kPolicies[0]);
constexpr int kRowsPolicy = kNumPolicies - 1;
constexpr int kRowsMaxM = 8;            // rows the streaming kernel takes
constexpr int kRowsMinBN = 64;          // its output columns per work-group: 64, 128, 256 or 512
constexpr int kRowsEnoughBlocks = 192;  // work-groups from which on a launch pulls the memory system's rate
// The streaming kernel is the default where 128-column blocks are already that many work-groups, i.e. from
// 24.5 thousand columns on (the vocabulary projections).  Measured, fp16, k = 4096, microseconds, best
// matrix-core choice against best streaming choice: n = 50400, m = 4: 96.9 / 71.9 (5.75 TB/s); n = 16384,
// m = 1: 27.7 / 28.5, m = 4: 27.4 / 31.1; n = 12288, m = 8: 25.9 / 32.2; n = 4096, k = 16384, m = 4:
// 30.1 / 36.8: below that width a launch is over before the stream has paid for its start and end.
constexpr int kRowsDefaultBN = 128;
// B stored [N, K] streams in blocks of 64 output columns and is the default for up to four rows from 12288
// columns on (fp16, k = 4096, microseconds, matrix-core kernel against streaming: n = 50400, m = 1: 89.2 /
// 78.6, m = 4: 90.1 / 80.8, m = 8: 91.4 / 95.6; n = 32000, m = 4: 61.6 / 49.5; n = 16384, m = 4: 33.6 / 25.5).
constexpr int kColsBN = 64;
constexpr int kColsMaxK = 16384;  // reduction length its register-resident pieces of A allow
enum : int { kRowsNone = 0, kRowsMC = 1, kRowsKC = 2 };  // which streaming kernel the operands allow

// Tile choice, the role of selectXetlaGemmConfig (xetla/gemm/gemm.cc:286-308).  Shapes listed in the tuned table
// (gemm_policy_table.h, written by autotune_gemm.py from measurements) take the policy
// recorded there, as the reference's configMap does (gemm.cc:31-285).
// XMK_GEMM_POLICY=<index> forces one policy for every shape (what the autotuner uses).
// ksplit: K slices to use when the caller supplies scratch (xmk_gemm_ws); 0 = no tuned value, the
// planner's own rule decides.  With ksplit > 1 `policy` is the tile of the slices.
struct TunedShape {
  int m, n, k, policy, ksplit;
};
#include "gemm_policy_table.h"
inline const TunedShape* tuned_shape(int64_t m, int64_t n, int64_t k) {
  for (const TunedShape& t : kTunedShapes)
    if (t.m == m && t.n == n && t.k == k) return &t;
  return nullptr;
}
inline bool rows_streams_by_default(int rows_kind, int64_t m, int64_t n) {
  return (rows_kind == kRowsMC && xmk::ceil_div(n, (int64_t)kRowsDefaultBN) >= kRowsEnoughBlocks) ||
         (rows_kind == kRowsKC && m <= 4 && xmk::ceil_div(n, (int64_t)kColsBN) >= kRowsEnoughBlocks);
}
// XMK_GEMM_POLICY=<index>, or -1.  Read at every call (a getenv costs far less than a launch), so that the
// autotuner can walk the policies inside one process.
inline int forced_policy() {
  if (const char* e = getenv("XMK_GEMM_POLICY")) {
    const int v = atoi(e);
    if (*e && v >= 0 && v < kNumPolicies) return v;
  }
  return -1;
}
// rows_kind: which streaming kernel the operands allow (gemm_rows_applicable); it is never chosen otherwise.
// tuned_ok: the operands have the layout the tuned table was measured with (B stored [K, N]).
inline int select_policy(int64_t m, int64_t n, int64_t k, int64_t batch = 1, int rows_kind = kRowsNone,
                         bool tuned_ok = true) {
  const bool rows_ok = rows_kind != kRowsNone;
  auto usable = [&](int v) { return v >= 0 && v < kNumPolicies && (v != kRowsPolicy || rows_ok); };
  if (const int v = forced_policy(); usable(v)) return v;
  if (batch == 1 && tuned_ok)
    if (const TunedShape* t = tuned_shape(m, n, k); t && t->ksplit <= 1 && usable(t->policy)) return t->policy;
  // A few rows against a very wide matrix: stream it.
  if (batch == 1 && rows_streams_by_default(rows_kind, m, n)) return kRowsPolicy;
  // Heuristic: the policy with the best estimated throughput = (what the tile sustains when the
  // device is full) x (share of the 256 CUs busy over the tile waves) x (share of the tiles' area
  // inside the matrix).  The per-tile figures are measured large-shape rates relative to 256x256.
  static constexpr float kTileRate[kRowsPolicy] = {1.0f, 0.75f, 0.60f, 0.55f, 0.90f};
  int best = kRowsPolicy - 1;
  float best_score = -1.0f;
  for (int i = 0; i < kRowsPolicy; ++i) {
    const int64_t tiles = xmk::ceil_div(m, kPolicies[i].bm) * xmk::ceil_div(n, kPolicies[i].bn) * batch;
    const int64_t waves = xmk::ceil_div(tiles, 256);
    const float busy = (float)tiles / (float)(waves * 256);
    const float inside = (float)((double)m * (double)n / ((double)tiles * kPolicies[i].bm * kPolicies[i].bn));
    const float score = kTileRate[i] * busy * inside;
    if (score > best_score) {
      best = i;
      best_score = score;
    }
  }
  return best;
}

template <typename T, bool OutF32, bool A_MC, bool B_MC, int BM, int BN, int WGM, int WGN, int BK, int NSTAGE,
          bool SLOW = false>
void launch_mfma(const GemmParams& p, int batch, hipStream_t st) {
  hipLaunchKernelGGL((gemm_mfma_kernel<T, OutF32, A_MC, B_MC, BM, BN, WGM, WGN, BK, NSTAGE, SLOW>),
                     dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(WGM * WGN * 64), 0, st, p);
}

template <typename T, bool OutF32, bool A_MC, bool B_MC>
void launch_policy(int pol, GemmParams& p, int batch, hipStream_t st) {
  p.tiles_m = (int)xmk::ceil_div(p.M, kPolicies[pol].bm);
  p.tiles_n = (int)xmk::ceil_div(p.N, kPolicies[pol].bn);
  switch (pol) {
    case 0: launch_mfma<T, OutF32, A_MC, B_MC, 256, 256, 2, 2, 32, 4>(p, batch, st); break;
    case 1: launch_mfma<T, OutF32, A_MC, B_MC, 128, 128, 2, 2, 64, 3>(p, batch, st); break;
    case 2: launch_mfma<T, OutF32, A_MC, B_MC, 128, 64, 2, 2, 64, 4>(p, batch, st); break;
    case 4: launch_mfma<T, OutF32, A_MC, B_MC, 256, 128, 2, 2, 64, 3>(p, batch, st); break;
    default: launch_mfma<T, OutF32, A_MC, B_MC, 64, 64, 2, 2, 64, 4>(p, batch, st); break;
  }
}

template <typename T, bool OutF32>
void launch_layout_impl(bool a_mc, bool b_mc, int pol, GemmParams& p, int batch, hipStream_t st) {
  if (!a_mc && !b_mc) launch_policy<T, OutF32, false, false>(pol, p, batch, st);
  else if (!a_mc && b_mc) launch_policy<T, OutF32, false, true>(pol, p, batch, st);
  else if (a_mc && !b_mc) launch_policy<T, OutF32, true, false>(pol, p, batch, st);
  else launch_policy<T, OutF32, true, true>(pol, p, batch, st);
}


// The gathering variant (operands the direct loads cannot take) has one tile, 128x128x32 in 3
// stages: its loads go through registers and are waited for inside the K step, so what hides their
// latency is occupancy -- 48 KB of LDS and about 150 registers let three work-groups share a CU.
constexpr Policy kGatherPolicy = {"mfma_128x128x32_w2x2_s3_gather", 128, 128, 2, 2, 32, 3};
template <typename T, bool OutF32, bool A_MC, bool B_MC>
void launch_policy_gather(GemmParams& p, int batch, hipStream_t st) {
  p.tiles_m = (int)xmk::ceil_div(p.M, kGatherPolicy.bm);
  p.tiles_n = (int)xmk::ceil_div(p.N, kGatherPolicy.bn);
  launch_mfma<T, OutF32, A_MC, B_MC, 128, 128, 2, 2, 32, 3, true>(p, batch, st);
}

template <typename T, bool OutF32>
void launch_layout_gather_impl(bool a_mc, bool b_mc, GemmParams& p, int batch, hipStream_t st) {
  if (!a_mc && !b_mc) launch_policy_gather<T, OutF32, false, false>(p, batch, st);
  else if (!a_mc && b_mc) launch_policy_gather<T, OutF32, false, true>(p, batch, st);
  else if (a_mc && !b_mc) launch_policy_gather<T, OutF32, true, false>(p, batch, st);
  else launch_policy_gather<T, OutF32, true, true>(p, batch, st);
}

// Explicitly instantiated in gemm_inst_*.hip.
template <typename T, bool OutF32>
void launch_layout(bool a_mc, bool b_mc, int pol, GemmParams& p, int batch, hipStream_t st);
template <typename T, bool OutF32>
void launch_layout_gather(bool a_mc, bool b_mc, GemmParams& p, int batch, hipStream_t st);

}  // namespace gemm_impl
