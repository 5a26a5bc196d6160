// Fused multi-head attention forward (flash attention) for bf16 / fp16:
//     O = softmax(scale * Q K^T + bias + mask) V,   optional LSE = m + log l.
//
// One work-group = NW waves, each owning 32 query rows of one (batch, head) unit; K and V are
// staged in LDS in tiles of 64 keys and consumed in half tiles of 32 keys.  Both products are
// issued transposed so that a lane owns ONE query row for the whole kernel:
//   S^T = K Q^T : A operand = K fragment (rows = keys) read from LDS, B operand = Q fragment
//                 kept in registers; the 32x32 accumulator layout puts query l%32 in lane l
//                 and keys in the lane's registers, so the row max is a register reduction
//                 plus one exchange with lane l^32 (which holds the other keys).
//   O^T += V^T P^T : P stays in registers (the S accumulator registers, converted, ARE the B
//                 operand); V is staged untransposed [key][h] and read with the LDS transpose
//                 loads, which deliver four consecutive keys of one h.
// K and V half tiles go from global memory straight into LDS (buffer_load ... lds), a ring of four
// stages each, the loads of the next three half tiles in flight while the current one is computed.
//
// The loop is a three-stage software pipeline over half tiles h (32 keys): in one step the matrix
// cores run the P V product of half tile h-1 and the S product of half tile h+1 while the vector
// ALU turns S_h into P_h (row max, exponentials, rounding, row sums).  The matrix instructions of
// a step depend on no vector result of the same step.  The step is written out as one slot per
// matrix instruction (its LDS fragment reads a few slots ahead, a fixed share of the vector work),
// the slots separated by scheduling fences: an 8-pass matrix instruction leaves about seven vector
// issue slots, which is what the softmax of its share of the scores needs.
//
// Online softmax in the exp2 domain: the scale is folded into the exponent (one FMA per
// element), the running reference max only moves when a row max exceeds it by more than
// 2^8 (so O is rescaled in few steps), and O is divided by l once at the end.  Causal: key >
// query masked (top-left aligned), key tiles past the diagonal are never visited, a wave skips
// the half tiles past its own rows, work-groups are issued heaviest first.
#pragma once
#include <algorithm>
#include <type_traits>
#include <utility>

#include "common.h"

namespace fmha_fwd_impl {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* lds_void_ptr;

constexpr int BC = 64;  // keys per K / V tile
constexpr uint32_t kOob = 0x80000000u;
constexpr float kLog2e = 1.4426950408889634f;

struct FmhaParams {
  const void* q;
  const void* k;
  const void* v;
  const void* bias;
  void* out;
  float* lse;
  int H, F, T;
  int nqb;       // query blocks per unit
  int total;     // work-groups with work: units * nqb
  int per_xcd;   // ceil(total / 8)
  int ug;        // units dealt together inside an XCD's range
  float scale2;  // head_scale * log2(e), > 0
};

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

template <typename T> struct Elem;
template <> struct Elem<__bf16> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ floatx16 mfma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // acc + a + b in fp32
  static __device__ __forceinline__ float dot2_ones(__bf16 a, __bf16 b, float acc) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(v2{a, b}, v2{(__bf16)1.0f, (__bf16)1.0f}, acc, false);
  }
};
template <> struct Elem<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ floatx16 mfma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float dot2_ones(_Float16 a, _Float16 b, float acc) {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(v2{a, b}, v2{(_Float16)1.0f, (_Float16)1.0f}, acc, false);
  }
};

__device__ __forceinline__ floatx16 zero16() {
  return floatx16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
}

// x *= alpha for an MFMA accumulator.  With the accumulators in the AGPR half of the register file
// (XMK_FMHA_AGPR, the build of the head-size-256 class) it is written out so that the register
// allocator keeps them in that file through the rare rescale path instead of moving all of them
// between files in every iteration; the leading and trailing waits cover the MFMA -> VALU and
// VALU -> MFMA hazards, which the compiler cannot see through the asm text.
__device__ __forceinline__ void scale_acc(floatx16& x, float alpha) {
#ifdef XMK_FMHA_AGPR
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    float e = x[i], tmp;
    if (i == 0)
      asm volatile("s_nop 7\n s_nop 7\n s_nop 7\n s_nop 7\n v_accvgpr_read_b32 %1, %0\n v_mul_f32 %1, %1, %2\n v_accvgpr_write_b32 %0, %1"
                   : "+a"(e), "=&v"(tmp) : "v"(alpha));
    else if (i == 15)
      asm volatile("v_accvgpr_read_b32 %1, %0\n v_mul_f32 %1, %1, %2\n v_accvgpr_write_b32 %0, %1\n s_nop 7\n s_nop 7"
                   : "+a"(e), "=&v"(tmp) : "v"(alpha));
    else
      asm volatile("v_accvgpr_read_b32 %1, %0\n v_mul_f32 %1, %1, %2\n v_accvgpr_write_b32 %0, %1"
                   : "+a"(e), "=&v"(tmp) : "v"(alpha));
    x[i] = e;
  }
#else
  x *= alpha;
#endif
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load(__amdgpu_buffer_rsrc_t r, uint32_t voff) {
  return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
}
// s_waitcnt immediate (gfx9 encoding): vmcnt(n), lgkmcnt(0), expcnt untouched.
__host__ __device__ constexpr int wait_vm_lgkm0(int n) { return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4); }

// Constraint that pins an MFMA accumulator where the matrix instructions of this build keep it.
#ifdef XMK_FMHA_AGPR
#define XMK_ACC(x) "+a"(x)
#else
#define XMK_ACC(x) "+v"(x)
#endif
constexpr int kAhead = 3;  // matrix instructions by which the LDS fragment reads run ahead

// T: element type; HP: head size padded to 64 / 128 / 256; NW: waves per work-group; WPS: waves
// per SIMD the register budget is set for.
// BIAS: 0 none; 1 read from global memory element by element (any shape and alignment); 2 staged
// through LDS one [rows x 64 keys] tile per key tile (T % 8 == 0, 16-byte aligned bias).
template <typename T, int HP, int NW, int WPS, bool CAUSAL, int BIAS>
__global__ __launch_bounds__(NW * 64, WPS) void fmha_fwd_kernel(FmhaParams p) {
  typedef typename Elem<T>::vec8 V8;
  constexpr int BR = NW * 32;                // query rows per work-group
  constexpr int ROWB = HP * 2;               // bytes of one K / V row in LDS
  constexpr int CPR = ROWB / 16;             // 16-byte chunks per row
  constexpr int KMASK = 15;                  // the K swizzle repeats every KMASK + 1 rows
  constexpr int HALF = 32 * ROWB;            // one K or V half tile (32 keys): one LDS stage
  constexpr int NST = 4;                     // stages of the K ring and of the V ring
  constexpr int RPL = 1024 / ROWB;           // tile rows per 1 KiB load
  constexpr int NL = HALF / 1024 / NW;       // loads per wave per half tile
  constexpr int LROWS = NW * RPL;            // tile rows between consecutive loads of a wave
  constexpr int KV = (LROWS % (KMASK + 1) == 0) ? 1 : 2;  // distinct K swizzles among a wave's loads
  constexpr int KS = HP / 16;                // k-steps of the S product
  constexpr int HT = HP / 32;                // 32-wide h tiles of O
  static_assert(BR % BC == 0, "a query block spans whole key tiles");
  static_assert(NL >= 1 && NL * LROWS == 32 && LROWS % 8 == 0 && (2 * LROWS) % (KMASK + 1) == 0, "half tile / wave split");
  constexpr int BTILE = 32 * BC * 2;         // one wave's bias tile: its 32 query rows x 64 keys
  __shared__ __attribute__((aligned(1024))) char lds[2 * NST * HALF + (BIAS == 2 ? NW * BTILE : 0)];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, l32 = lane & 31;
  // Work-groups are dealt round-robin to the 8 XCDs, each with its own L2.  Give every XCD a
  // contiguous range of (unit, query block) pairs, so that the query blocks of one unit, which
  // stream the same K and V, run on one XCD at about the same time.
  const int wg = (int)(blockIdx.x % 8) * p.per_xcd + (int)(blockIdx.x / 8);
  if (wg >= p.total) return;
  // Inside the range, units go four at a time, query blocks outermost and heaviest (latest) first: the four
  // units' work-groups of one causal weight are dealt together, so an XCD's slots run dry at about the same
  // time (unit by unit, the last unit's heaviest block would start when most slots are about to finish).
  const int UG = p.ug;
  const int ublk = wg / (UG * p.nqb), r = wg % (UG * p.nqb);
  const int gb = min(UG, p.total / p.nqb - ublk * UG);  // units in this group (the last may hold fewer)
  const int unit = ublk * UG + r % gb;
  const int qb = p.nqb - 1 - r / gb;
  const int q0 = qb * BR;
  const int H = p.H, F = p.F, Tk = p.T;

  using std::false_type;
  using std::true_type;

  const T* Q = reinterpret_cast<const T*>(p.q) + (int64_t)unit * F * H;
  const T* K = reinterpret_cast<const T*>(p.k) + (int64_t)unit * Tk * H;
  const T* V = reinterpret_cast<const T*>(p.v) + (int64_t)unit * Tk * H;

  // ---- Q fragments (B operand of S^T): this wave holds query rows wq0 + l%32, fragment s covers
  // h = 16 s + 8 g .. +7.
  const int wq0 = q0 + wave * 32;
  const int qrow = wq0 + l32;
  // They come in through LDS (prologue below): read from global memory in this layout, neighbouring lanes hold
  // different rows and every lane is a cache access of its own, four times the load-path time of a tile load.
  V8 qf[KS];

  // ---- K / V half-tile loads, global -> LDS.  Load j = i * NW + wave fills LDS bytes [1024 j, +1024)
  // of the stage, i.e. half-tile rows j * RPL ..; lane l lands at row j * RPL + l / CPR, chunk l % CPR,
  // and fetches the global chunk that belongs there under the stage's swizzle.
  // K rows: chunk ^= kswz(key), so that the 16 lanes of a fragment read (16 consecutive keys, one chunk column)
  // touch 16 different bank groups: with 128-byte rows two keys share 256 bytes of banks and the key's parity
  // already separates them.
  auto kswz = [](int key) { return CPR >= 16 ? (key & 15) : ((key >> 1) & 7); };
  const int lrow = wave * RPL + lane / CPR;  // half-tile row of this lane in load 0; load i: + i * LROWS
  uint32_t koff[KV];
#pragma unroll
  for (int v = 0; v < KV; ++v) {
    const int row = lrow + v * LROWS;
    const int chunk = (lane % CPR) ^ kswz(row);
    koff[v] = chunk * 8 < H ? (uint32_t)((lrow * H + chunk * 8) * 2) : kOob;
  }
  // V rows: chunk ^= vswz(key).  A transpose read touches 4 chunks of each of 4 consecutive keys;
  // the XOR moves each key's group of 4 chunks to its own banks.
  auto vswz = [](int key) { return CPR >= 16 ? (key & 3) << 2 : (key & 2) << 1; };
  const int vchunk = (lane % CPR) ^ vswz(lrow);
  const uint32_t voff = vchunk * 8 < H ? (uint32_t)((lrow * H + vchunk * 8) * 2) : kOob;
  const uint32_t lstride = (uint32_t)(LROWS * H * 2);  // global bytes between a wave's loads
  // Half tile hh (32 rows from row 32 hh of K or V) into `stage`.  Rows past T load zeros, in two ways.
  // RANGED: every load gets a buffer descriptor of its own that ends with the last row (a handful of
  // scalar instructions; a half tile wholly past T then touches no memory at all), so that the plain
  // steps can run up to the end of the keys.  Otherwise one descriptor per half tile, the loads apart by
  // a scalar offset, which the hardware does not range-check: rows past T become out-of-range lane offsets.
  auto issue_half = [&](auto RANGED, const T* base, int hh, char* __restrict__ stage, const uint32_t* offs, int noffs) {
    const int rows_left = Tk - 32 * hh;  // may be <= 0 for the second half of the last tile
    if constexpr (decltype(RANGED)::value) {
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int rl = max(rows_left - i * LROWS, 0);
        const __amdgpu_buffer_rsrc_t r = make_rsrc(base + (int64_t)(32 * hh + i * LROWS) * H, (uint32_t)rl * (uint32_t)(H * 2));
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void_ptr)(stage + (i * NW + wave) * 1024), 16, offs[i % noffs], 0,
                                                 0, 0);
      }
    } else {
      const __amdgpu_buffer_rsrc_t r = make_rsrc(base + (int64_t)(32 * hh) * H, 0x7fffffffu);
      const bool full = rows_left >= 32;
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const uint32_t off = (full || lrow + i * LROWS < rows_left) ? offs[i % noffs] : kOob;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void_ptr)(stage + (i * NW + wave) * 1024), 16, off,
                                                 i * lstride, 0, 0);
      }
    }
  };

  // The 32 query rows of wave i as a half tile in K's layout (rows past F: zeros).
  auto issue_q = [&](int i_half, char* __restrict__ stage) {
    const int rows_left = F - q0 - 32 * i_half;
    const __amdgpu_buffer_rsrc_t r = make_rsrc(Q + (int64_t)(q0 + 32 * i_half) * H, 0x7fffffffu);
    const bool full = rows_left >= 32;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const uint32_t off = (full || lrow + i * LROWS < rows_left) ? koff[i % KV] : kOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void_ptr)(stage + (i * NW + wave) * 1024), 16, off, i * lstride, 0, 0);
    }
  };

  // ---- per-lane LDS offsets of the fragments
  // K fragment (step s): key row l%32 of the half tile, logical chunk 2 s + g.
  int kbase[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) kbase[s] = l32 * ROWB + (((2 * s + g) ^ kswz(l32)) << 4);
  // V^T fragment (key group u of the half tile, h tile ht): two transpose reads; within a 16-lane block
  // lane pl addresses key row 16 u + 4 g + pl/4 (+8 for the second read), h = cb + 4 (pl%4) .. +3.
  int vbase[HT][2];
  {
    const int pl = lane & 15;
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) {
      const int col = 32 * ht + ((lane >> 4) & 1) * 16 + 4 * (pl & 3);
      const int chunk = col >> 3, within = (col & 7) * 2;
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const int key = 4 * g + (pl >> 2) + 8 * h2;  // + 16 u: does not change key & 3
        vbase[ht][h2] = key * ROWB + ((chunk ^ vswz(key)) << 4) + within;
      }
    }
  }

  // ---- bias tile (BIAS == 2): each wave keeps the [32 rows x 64 keys] tile of its own query rows in
  // its own 4 KiB of LDS, loaded with four 1 KiB direct loads (8 rows of 128 bytes each) one tile
  // ahead.  Row r stores its 16-byte chunk c at position c ^ ((r >> 1) & 7), so that the 8-byte reads
  // of 32 lanes (32 rows, one chunk column) spread over the banks.
  uint32_t boff[4];  // global byte offset of this lane's chunk in load i, from bias row q0, key 0
  int bkey[4];       // first key (within the tile) of that chunk
  int bread[8];      // LDS byte offset of the 4 keys 32 kt + 8 q + 4 g .. +3 of this lane's row: [4 kt + q]
  const T* bias_base = nullptr;
  if constexpr (BIAS == 2) {
    bias_base = reinterpret_cast<const T*>(p.bias) + ((int64_t)unit * F + q0) * Tk;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 8 * i + (lane >> 3);
      const int c = (lane & 7) ^ ((row >> 1) & 7);
      bkey[i] = c * 8;
      boff[i] = wq0 + row < F ? (uint32_t)((((int64_t)(wave * 32 + row)) * Tk + c * 8) * 2) : kOob;
    }
#pragma unroll
    for (int r = 0; r < 8; ++r) bread[r] = l32 * 128 + ((r ^ ((l32 >> 1) & 7)) << 4) + g * 8;
  }
  // Loads the bias tile of the key tile that starts at t0.  T % 8 == 0, so a chunk lies inside
  // the row or past its end as a whole; rows past F and chunks past T load zeros.
  auto issue_bias = [&](int t0, char* __restrict__ btile) {
    const __amdgpu_buffer_rsrc_t r = make_rsrc(bias_base, 0x7fffffffu);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t off = (t0 + bkey[i] < Tk && boff[i] != kOob) ? boff[i] + (uint32_t)t0 * 2 : kOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void_ptr)(btile + i * 1024), 16, off, 0, 0, 0);
    }
  };
  auto bias_value = [](u32x2 w, int e) -> float {
    const uint32_t d = w[e >> 1];
    if constexpr (sizeof(T) == 2 && __is_same(T, __bf16)) {
      return __builtin_bit_cast(float, (e & 1) ? (d & 0xffff0000u) : (d << 16));
    } else {
      return (float)__builtin_bit_cast(_Float16, (uint16_t)((e & 1) ? (d >> 16) : (d & 0xffffu)));
    }
  };

  floatx16 ot[HT];
  float m_run = -INFINITY;
  float l_run = 0.0f;  // this lane's share (its 16 keys of every half tile) of the row sum
#pragma unroll
  for (int i = 0; i < HT; ++i) ot[i] = zero16();
  const float inv_scale = kLog2e / p.scale2;  // bias is added in score units: (s + b / scale) * scale

  const int kend = CAUSAL ? min(Tk, q0 + BR) : Tk;  // keys this work-group can see
  const int nblk = (kend + BC - 1) / BC;            // key tiles
  // Half tiles this wave has to look at: those that start at or before its last query row and before
  // the last key.
  const int nh_all = (kend + 31) / 32;
  const int nh = CAUSAL ? min(nh_all, (wq0 + 31) / 32 + 1) : nh_all;

  // S^T = K Q^T of the half tile in a K stage (one accumulator, KS dependent matrix instructions).
  auto scores = [&](const char* __restrict__ kstage, floatx16& st) {
    st = zero16();
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const u32x4 kv = *reinterpret_cast<const u32x4*>(kstage + kbase[s]);
      st = Elem<T>::mfma(__builtin_bit_cast(V8, kv), qf[s], st);
    }
  };

  // Bias and masks of half tile h (MASKED steps: those on the causal diagonal or past the last key).
  // st[i] <-> key 32 h + 8 (i/4) + 4 g + i%4.  Scores stay unscaled; the scale is folded into the
  // exponent.  bv: the staged bias of the half tile (BIAS == 2).
  auto bias_and_mask = [&](auto MASKED, floatx16& st, int h, const u32x2 (&bv)[4]) {
    const int k0 = 32 * h;
    if constexpr (BIAS == 2) {
#pragma unroll
      for (int i = 0; i < 16; ++i) st[i] += bias_value(bv[i / 4], i % 4) * inv_scale;
    }
    if constexpr (BIAS == 1) {
      if (qrow < F) {
        const T* bp = reinterpret_cast<const T*>(p.bias) + ((int64_t)unit * F + qrow) * Tk;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = k0 + 8 * (i / 4) + 4 * g + (i % 4);
          if (key < Tk) st[i] += (float)bp[key] * inv_scale;
        }
      }
    }
    if constexpr (decltype(MASKED)::value) {
      // Most masked steps of a wave have nothing to mask (the half tile lies below the wave's rows and inside
      // the keys): a wave-uniform test skips those.  Otherwise both limits fold into one threshold per lane
      // and an element costs a compare with a constant and a select.
      if ((CAUSAL && k0 + 31 > wq0) || k0 + 32 > Tk) {
        const int thr = min(CAUSAL ? qrow : 0x7fffffff, Tk - 1) - k0 - 4 * g;  // key offsets above it are masked
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (8 * (i / 4) + (i % 4) > thr) st[i] = -INFINITY;
      }
    }
  };

  // The running reference max m_run only moves when some row's max exceeds it by more than 2^8, so
  // that P stays below 256 and O needs a rescale in few steps.  The test is wave-uniform and the
  // common case (nothing moves) costs an exchange with lane l ^ 32 (which holds the row's other 16
  // keys of the half tile), a max and a compare against thr_run = (m_run + 8) / scale2, the
  // threshold in score units; the move itself sits behind a branch.  mx: the maximum of the lane's
  // 16 scores of the half tile.
  float thr_run = -INFINITY;
  const float inv_scale2 = 1.0f / p.scale2;
  auto row_max_exceeds = [&](float& mx) -> bool {
    // v_permlane32_swap exchanges the upper 32 lanes of its first operand with the lower 32 of its second:
    // started from two copies of mx, the first ends as the lower half's values in both halves and the
    // second as the upper half's.  Written out because BOTH results are needed and this compiler's
    // __builtin_amdgcn_permlane32_swap hands back the first one twice (the max of the two then folds
    // away and the row max would cover the lower lanes' 16 keys only).  The s_nop covers the two wait
    // states the instruction needs after a vector write of its operands, which the hazard recogniser
    // cannot insert inside an asm statement.
    float other = mx;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(mx), "+v"(other));
    mx = __builtin_elementwise_maximum(mx, other);
    return __any(mx > thr_run);
  };
  // The move: returns the new exponent reference; `alpha` is the factor l and O still have to be
  // multiplied by.
  auto move_reference = [&](float mx, float& alpha) -> float {
    const float m_new = fmaxf(m_run, mx * p.scale2);
    alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // first step: exp2(-inf) = 0
    m_run = m_new;
    thr_run = (m_new + 8.0f) * inv_scale2;
    // A row that has seen no visible key keeps m_run = -inf; use 0 as its reference so that
    // its masked (-inf) scores give exp2(-inf) = 0 and not NaN.
    return m_new == -INFINITY ? 0.0f : m_new;
  };
  // Maximum of an accumulator's 16 elements (v_maximum3_f32: no canonicalising copies of the inputs).
  auto max16 = [](const floatx16& x) -> float {
    float mx = __builtin_elementwise_maximum(x[0], x[1]);
#pragma unroll
    for (int i = 2; i < 16; i += 2) mx = __builtin_elementwise_maximum(__builtin_elementwise_maximum(mx, x[i]), x[i + 1]);
    return mx;
  };

  // O^T += V^T P^T for the 16 keys of group ug (0, 1) of the half tile in a V stage.
  auto accumulate = [&](const char* __restrict__ vtile, int ug, const V8& pf) {
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) {
      typedef short4v __attribute__((address_space(3))) * lds_ptr;
      const char* vt = vtile + ug * 16 * ROWB;
      const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(vt + vbase[ht][0]));
      const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(vt + vbase[ht][1]));
      u32x4 vv;
      vv[0] = __builtin_bit_cast(u32x2, lo)[0];
      vv[1] = __builtin_bit_cast(u32x2, lo)[1];
      vv[2] = __builtin_bit_cast(u32x2, hi)[0];
      vv[3] = __builtin_bit_cast(u32x2, hi)[1];
      ot[ht] = Elem<T>::mfma(__builtin_bit_cast(V8, vv), pf, ot[ht]);
    }
  };

  // LDS: K half tile h in K stage h % 4, V half tile h in V stage h % 4.
  char* const kst0 = lds;
  char* const vst0 = lds + NST * HALF;
  char* const btile = lds + 2 * NST * HALF + wave * BTILE;  // this wave's bias tile (BIAS == 2)
  const int nhalf = 2 * nblk;  // half tiles staged (the last may lie past T: it loads zeros)

  floatx16 sa, sb;     // S of even / odd half tiles
  V8 pa[2], pb[2];     // P of even / odd half tiles
  u32x2 b0[4], b1[4];  // staged bias of the even / odd half tile of the current tile

  // Reads the staged bias tile of key tile j (it landed during the previous steps) and sends
  // the next tile's into the same 4 KiB.
  auto take_bias = [&](int j) {
    if constexpr (BIAS == 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        b0[r] = *reinterpret_cast<const u32x2*>(btile + bread[r]);
        b1[r] = *reinterpret_cast<const u32x2*>(btile + bread[4 + r]);
      }
      if (j + 1 < nblk) issue_bias((j + 1) * BC, btile);
    }
  };

  // One pipeline step on half tile h (HS = h % 4, a compile-time constant so that the stage offsets
  // fold into the LDS instructions):
  //   - sends the loads of K half tile h+4 and V half tile h+2 into the stages that fell free at the
  //     last barrier (they are needed three steps from now);
  //   - matrix cores: S of half tile h+1, then P V of half tile h-1;
  //   - vector ALU: P_h = exp2(S_h - reference) with the reference found in the last step, then, once
  //     S_{h+1} is there, its bias, mask and row max, which give the next step's reference;
  //   - rescales O if the last step moved the reference (rare), i.e. after P V of half tile h-1 and
  //     before that of half tile h;
  //   - waits until the loads that the NEXT step reads have landed (those sent two steps ago: the
  //     loads of this and the last step may stay in flight) and meets the other waves.
  // MASKED steps: S_{h+1} may touch the causal diagonal or the end of the keys: the mask is applied where a
  // wave needs one, and a wave leaves out the work past its last half tile (nh).  Loads and waits are those
  // of the plain form: ranged loads, which may reach past the keys, and a counted wait.  A masked step
  // takes 1.1-1.4 us where a plain one takes 0.86 (per-wave timestamps, [8,32,2048,128]), mask or no
  // mask, so the plain form runs wherever no wave needs a mask.  PV / SC: whether there is a P V product
  // (not in step 0) and an S product (not in the last step) to run.
  float mref_c, alpha_c = 1.0f;  // exponent reference of S_h; factor O has to be multiplied by before P V of h
  bool moved_c = false;          // whether alpha_c differs from 1 for some row
  auto step = [&](auto MASKED, auto PV, auto SC, auto HSC, int h) {
    constexpr bool masked = decltype(MASKED)::value, pv = decltype(PV)::value, sco = decltype(SC)::value;
    constexpr int HS = decltype(HSC)::value;
    floatx16& sc = (HS & 1) ? sb : sa;
    floatx16& sn = (HS & 1) ? sa : sb;
    const V8(&pp)[2] = (HS & 1) ? pa : pb;
    V8(&pf)[2] = (HS & 1) ? pb : pa;
    // The four stages a step touches never overlap; as __restrict__ parameters they tell the compiler so,
    // and it does not make the fragment reads wait for the loads in flight.
    [&](const char* __restrict__ knext, const char* __restrict__ vprev, char* __restrict__ kfree,
        char* __restrict__ vfree) {
    // The step is written as a sequence of slots, one per matrix instruction, each closed by a
    // scheduling fence: slot i sends the LDS fragment reads of matrix instruction i + D, issues matrix
    // instruction i and runs its share of the vector work.  Empty asm statements pin every piece
    // of vector work (its inputs at the start, its results at the end) and every accumulator to the
    // slot, since arithmetic is otherwise free to drift across the fences.
    constexpr int NS = sco ? KS : 0, NP = pv ? 2 * HT : 0, NM = NS + NP, D = kAhead;
    constexpr int R0 = NS + 1, R1 = NS + 2;                   // slots of the row max of the new S
    constexpr int NSLOT = sco ? (NM > R1 + 1 ? NM : R1 + 1) : (NM > 8 ? NM : 8);
    const bool active = !masked || h - 1 < nh;
    u32x4 frag[D + 1];
    auto fetch = [&](auto I) {
      constexpr int i = decltype(I)::value;
      if constexpr (i < NS) {
        frag[i % (D + 1)] = *reinterpret_cast<const u32x4*>(knext + kbase[i]);
      } else if constexpr (i < NM) {
        constexpr int q = i - NS, u = q / HT, ht = q % HT;
        typedef short4v __attribute__((address_space(3))) * lds_ptr;
        const char* vt = vprev + u * 16 * ROWB;
        const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(vt + vbase[ht][0]));
        const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(vt + vbase[ht][1]));
        u32x4 vv;
        vv[0] = __builtin_bit_cast(u32x2, lo)[0];
        vv[1] = __builtin_bit_cast(u32x2, lo)[1];
        vv[2] = __builtin_bit_cast(u32x2, hi)[0];
        vv[3] = __builtin_bit_cast(u32x2, hi)[1];
        frag[i % (D + 1)] = vv;
      }
    };
    // The first fragment reads go out before the step's loads: sending the loads takes the wave about 170
    // cycles, under which the reads' latency passes.
    if (active) static_for<D>(fetch);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (sco) {  // (the last step has nothing left to send)
      issue_half(true_type{}, K, h + 4, kfree, koff, KV);
      issue_half(true_type{}, V, h + 2, vfree, &voff, 1);
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr ((HS & 1) == 1 && sco) take_bias((h + 1) / 2);
    if (active) {
      float alpha_n = 1.0f, mref_n = mref_c;
      bool moved_n = false;
      auto fire = [&](auto I) {
        constexpr int i = decltype(I)::value;
        if constexpr (i < NS) {
          if constexpr (i == 0) sn = Elem<T>::mfma(__builtin_bit_cast(V8, frag[i % (D + 1)]), qf[i], zero16());
          else sn = Elem<T>::mfma(__builtin_bit_cast(V8, frag[i % (D + 1)]), qf[i], sn);
          asm volatile("" : XMK_ACC(sn));
        } else if constexpr (i < NM) {
          constexpr int q = i - NS, u = q / HT, ht = q % HT;
          ot[ht] = Elem<T>::mfma(__builtin_bit_cast(V8, frag[i % (D + 1)]), pp[u], ot[ht]);
          asm volatile("" : XMK_ACC(ot[ht]));
        }
      };
      // Elements 2k, 2k+1 of S_h: exponentials, rounding to one packed word of P_h, row-sum share.  In two
      // halves one slot apart: a transcendental's result costs a wait state when the very next vector
      // instruction uses it, so the rounding of piece k runs behind the exponentials of piece k + 1.
      float e0[8], e1[8];
      auto epiece_exp = [&](auto KC) {
        constexpr int k = decltype(KC)::value;
        float x0 = sc[2 * k], x1 = sc[2 * k + 1];
        asm volatile("" : "+v"(x0), "+v"(x1));
        e0[k] = __builtin_amdgcn_exp2f(__builtin_fmaf(x0, p.scale2, -mref_c));
        e1[k] = __builtin_amdgcn_exp2f(__builtin_fmaf(x1, p.scale2, -mref_c));
        asm volatile("" : "+v"(e0[k]), "+v"(e1[k]));
      };
      auto epiece_round = [&](auto KC) {
        constexpr int k = decltype(KC)::value;
        const T r0 = (T)e0[k], r1 = (T)e1[k];
        l_run = Elem<T>::dot2_ones(r0, r1, l_run);
        pf[k / 4][2 * (k % 4)] = r0;
        pf[k / 4][2 * (k % 4) + 1] = r1;
        asm volatile("" : "+v"(l_run));
      };
      float mx = 0.0f;
      auto rpiece0 = [&]() {
        bias_and_mask(MASKED, sn, h + 1, (HS & 1) ? b0 : b1);
        mx = max16(sn);
        asm volatile("" : "+v"(mx));
      };
      auto rpiece1 = [&]() {
        moved_n = row_max_exceeds(mx);
        asm volatile("" : "+v"(mx));
      };
      static_for<NSLOT>([&](auto I) {
        constexpr int i = decltype(I)::value;
        fetch(std::integral_constant<int, i + D>{});
        fire(I);
        static_for<8>([&](auto KC) {
          constexpr int k = decltype(KC)::value;
          if constexpr ((k * NSLOT) / 8 == i) {
            epiece_exp(KC);
            if constexpr (k > 0) epiece_round(std::integral_constant<int, (k > 0 ? k - 1 : 0)>{});
          }
        });
        if constexpr (sco && i == R0) rpiece0();
        if constexpr (sco && i == R1) rpiece1();
        __builtin_amdgcn_sched_barrier(0);
      });
      epiece_round(std::integral_constant<int, 7>{});
      static_for<2>([&](auto U) {
        u32x4 w = __builtin_bit_cast(u32x4, pf[decltype(U)::value]);
        asm volatile("" : "+v"(w));
        pf[decltype(U)::value] = __builtin_bit_cast(V8, w);
      });
      // The rare move of the reference (wave-uniform).  l_run holds every term up to P_h under the
      // reference of S_h: it moves to the new reference here, O a step later.
      if (moved_n) {
        mref_n = move_reference(mx, alpha_n);
        l_run *= alpha_n;
      }
      // The rare rescale of O, after the P V product of half tile h-1 and before that of half tile h.
      if (moved_c) {
#pragma unroll
        for (int ht = 0; ht < HT; ++ht) scale_acc(ot[ht], alpha_c);
      }
      mref_c = mref_n;
      alpha_c = alpha_n;
      moved_c = moved_n;
    }
    }(kst0 + ((HS + 1) % NST) * HALF, vst0 + ((HS + 3) % NST) * HALF, kst0 + HS * HALF, vst0 + ((HS + 2) % NST) * HALF);
    // The loads of this step and of the one before may stay in flight; the last step sends none and ends
    // with all of them landed, since the output rows are staged where K and V were.
    if constexpr (!sco || BIAS == 2) __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
    else __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(4 * NL));
    __builtin_amdgcn_s_barrier();
  };
  typedef std::integral_constant<int, 0> hs0;
  typedef std::integral_constant<int, 1> hs1;
  typedef std::integral_constant<int, 2> hs2;
  typedef std::integral_constant<int, 3> hs3;

  // Prologue: the query rows, staged in the V ring (free until V half tile 0 is sent) and read back as row
  // fragments, wave w those of stage w; beside them the first two K half tiles, then the four half tiles the
  // pipeline keeps ahead.
  static_assert(NW <= NST, "one V stage per wave for the query rows");
#pragma unroll
  for (int i = 0; i < NW; ++i) issue_q(i, vst0 + i * HALF);
  if constexpr (BIAS == 2) issue_bias(0, btile);
  issue_half(false_type{}, K, 0, kst0, koff, KV);
  issue_half(false_type{}, K, 1, kst0 + HALF, koff, KV);
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(2 * NL + (BIAS == 2 ? 4 : 0)));  // the query rows have landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int s = 0; s < KS; ++s) qf[s] = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4*>(vst0 + wave * HALF + kbase[s]));
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(63));  // (lgkmcnt(0): the fragments are in registers)
  __builtin_amdgcn_s_barrier();                   // every wave has its own: the V ring may be filled
  issue_half(false_type{}, V, 0, vst0, &voff, 1);
  issue_half(true_type{}, K, 2, kst0 + 2 * HALF, koff, KV);  // (ranged: past the keys they touch no memory, and
  issue_half(true_type{}, K, 3, kst0 + 3 * HALF, koff, KV);  //  the count of loads in flight is the same for every T)
  issue_half(false_type{}, V, 1, vst0 + HALF, &voff, 1);
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(4 * NL));
  __builtin_amdgcn_s_barrier();
  take_bias(0);
  scores(kst0, sa);
  bias_and_mask(true_type{}, sa, 0, b0);
  {
    float a0, mx = max16(sa);
    row_max_exceeds(mx);
    mref_c = move_reference(mx, a0);  // O and l are still zero: nothing to rescale
  }
  // step 0 sends K half tile 4 into the stage this S product has just read
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(63));
  __builtin_amdgcn_s_barrier();
  step(true_type{}, false_type{}, true_type{}, hs0{}, 0);

  // Steps 1 .. nhalf-2.  A step's S product is that of half tile h + 1: it needs the masked form from the
  // first half tile on that touches the causal diagonal of the work-group's first row or holds keys past T;
  // before that every wave has all of its rows below the keys and the plain form (whose loads are ranged)
  // runs.  Plain steps go four to a trip (stage positions 1, 2, 3, 0); the causal diagonal starts in the
  // middle of such a group, hence the two extra plain steps and the two masked ones that follow them,
  // after which the masked steps go on from stage position 1 like the plain ones.  (One loop that picks a
  // step's copy by h % 4 was tried: it spilled registers in the step and ran at a third of the rate.)
  const int hmask = min(CAUSAL ? q0 / 32 : 0x7fffffff, Tk / 32);  // first half tile that needs a mask
  const int hend = nhalf - 1;                                     // the last step, which has no S product
  const int hplain = min(hend, hmask - 1);                        // steps below it may be plain
  int h = 1;
  for (; h + 3 < hplain; h += 4) {
    step(false_type{}, true_type{}, true_type{}, hs1{}, h);
    step(false_type{}, true_type{}, true_type{}, hs2{}, h + 1);
    step(false_type{}, true_type{}, true_type{}, hs3{}, h + 2);
    step(false_type{}, true_type{}, true_type{}, hs0{}, h + 3);
  }
  if (h + 1 < hplain) {
    step(false_type{}, true_type{}, true_type{}, hs1{}, h);
    step(false_type{}, true_type{}, true_type{}, hs2{}, h + 1);
    h += 2;
    if (h < hend) {  // (hend is odd, h is 3 mod 4: a further step is followed by another)
      step(true_type{}, true_type{}, true_type{}, hs3{}, h);
      step(true_type{}, true_type{}, true_type{}, hs0{}, h + 1);
      h += 2;
    }
  }
  for (; h < hend; h += 2) {
    step(true_type{}, true_type{}, true_type{}, hs1{}, h);
    step(true_type{}, true_type{}, true_type{}, hs2{}, h + 1);
    if (h + 2 < hend) {
      step(true_type{}, true_type{}, true_type{}, hs3{}, h + 2);
      step(true_type{}, true_type{}, true_type{}, hs0{}, h + 3);
      h += 2;
    }
  }
  // The last step (half tile nhalf-1, odd: no further S) and the P V product of that half tile.
  if (nblk & 1) step(true_type{}, true_type{}, false_type{}, hs1{}, nhalf - 1);
  else step(true_type{}, true_type{}, false_type{}, hs3{}, nhalf - 1);
  if (nhalf - 1 < nh) {
    const char* vlast = vst0 + ((nhalf - 1) % NST) * HALF;
    accumulate(vlast, 0, pb[0]);
    accumulate(vlast, 1, pb[1]);
  }

  // ---- finish: O = O^T / l; LSE = m ln2 + ln l.  The accumulator layout gives a lane 8 bytes in each of 16
  // places of its row, so the rounded rows go through LDS (one region of 32 rows per wave, 16-byte chunks XORed
  // with the row so that both passes spread over the banks) and leave with 16-byte stores that cover whole rows.
  // The regions start at the K stages, which no wave reads after the loop's last barrier; where they reach
  // into the V stages, every wave must be done with the last V tile first.
  if constexpr (NW * 32 * ROWB > NST * HALF) {
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
    __builtin_amdgcn_s_barrier();
  }
  constexpr int OCPR = HP / 8;  // 16-byte chunks per output row
  static_assert(NW * 32 * ROWB <= 2 * NST * HALF, "the output tiles are staged in the K / V stages");
  {
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv = 1.0f / l_tot;
    char* region = lds + wave * (32 * ROWB);
    static_for<HT>([&](auto HTI) {
      constexpr int ht = decltype(HTI)::value;
      const floatx16 o = ot[ht];
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        union { T e[4]; u32x2 w; } r;
        r.e[0] = (T)(o[4 * qd + 0] * inv);
        r.e[1] = (T)(o[4 * qd + 1] * inv);
        r.e[2] = (T)(o[4 * qd + 2] * inv);
        r.e[3] = (T)(o[4 * qd + 3] * inv);
        const int chunk = (4 * ht + qd) ^ (l32 & (OCPR - 1));
        *reinterpret_cast<u32x2*>(region + l32 * ROWB + (chunk << 4) + g * 8) = r.w;
      }
    });
    if (qrow < F && p.lse && g == 0) p.lse[(int64_t)unit * F + qrow] = m_run * 0.6931471805599453f + logf(l_tot);
    // this wave's own region: its LDS writes are complete for its own reads once lgkmcnt is zero
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(63));
    constexpr int RPI = 64 / OCPR;  // rows per store instruction
    const int c = lane % OCPR;
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
      const int row = it * RPI + lane / OCPR;
      const u32x4 v = *reinterpret_cast<const u32x4*>(region + row * ROWB + ((c ^ (row & (OCPR - 1))) << 4));
      const int qr = wq0 + row;
      if (qr < F && c * 8 < H)  // H % 8 == 0: a chunk lies inside the row or outside as a whole
        *reinterpret_cast<u32x4*>(reinterpret_cast<T*>(p.out) + ((int64_t)unit * F + qr) * H + c * 8) = v;
    }
  }
}

template <typename T, int HP, int NW, int WPS>
void launch_cfg(FmhaParams p, uint64_t units, uint32_t F, bool causal, int bias, hipStream_t st) {
  p.nqb = (int)((F + NW * 32 - 1) / (NW * 32));
  p.total = (int)(units * p.nqb);
  p.per_xcd = (p.total + 7) / 8;
  // Four units at a time (measured on causal [8,32,2048,128]: 1: 697, 2: 730, 4: 756, 8: 751, 16: 733, 32: 699
  // TFLOP/s), more when a unit has so few query blocks that four units do not fill an XCD's 64 slots.
  p.ug = std::max(4, (64 + p.nqb - 1) / p.nqb);
  const dim3 grid((unsigned)(p.per_xcd * 8)), block(NW * 64);
  // bias: 0 none, 1 element-wise from global memory, 2 staged through LDS
  if (causal) {
    if (bias == 2) hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, NW, WPS, true, 2>), grid, block, 0, st, p);
    else if (bias == 1) hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, NW, WPS, true, 1>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, NW, WPS, true, 0>), grid, block, 0, st, p);
  } else {
    if (bias == 2) hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, NW, WPS, false, 2>), grid, block, 0, st, p);
    else if (bias == 1) hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, NW, WPS, false, 1>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, NW, WPS, false, 0>), grid, block, 0, st, p);
  }
}

// Head size above 128 (the accumulators of that class need both halves of the register file);
// defined in fmha_fwd_h256.hip.
void launch_h256(const FmhaParams& p, int32_t dtype, uint64_t units, uint32_t F, bool causal, int bias,
                 hipStream_t st);

}  // namespace fmha_fwd_impl
