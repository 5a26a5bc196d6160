// Fused multi-head attention backward for bf16 / fp16 without a score-sized intermediate
// (the role of fmha_backward_kernel_{fp16,bf16}, xetla/sdp/sdp_backward.h:22-36).
//
// One kernel template, run with the roles of queries and keys exchanged:
//   owner = keys    : a work-group owns 128 keys (4 waves x 32) and walks the queries in blocks of 64;
//                     it accumulates dK = scale dS^T Q or dV = P^T dO for its keys (one launch each).
//   owner = queries : a work-group owns 128 queries and walks the keys; it accumulates dQ = scale dS K.
// with  P = exp(scale S - LSE),  dS = P o (dP - D),  S = Q K^T,  dP = dO V^T,  D = rowsum(dO o O).
// S (and dP) are recomputed in every pass (8 matrix products instead of 5) so that no gradient needs
// atomics or a second pass over partial sums: every output element is written once, in a fixed order.
//
// As in the forward kernel, every product is issued so that a lane owns ONE owner row:
//   scores  = Stream_tile . Owner^T : A operand = fragment of the streamed tile (LDS), B operand =
//             owner fragment (registers).  The 32x32 accumulator layout puts owner row l%32 in
//             lane l and the streamed rows in the lane's registers.
//   acc^T  += Stream_tile^T . dS    : the accumulator registers, converted, ARE the B operand (the
//             contraction runs over the streamed rows); the streamed tile is read with the LDS
//             transpose loads.
// The streamed tiles go from global memory straight into LDS, two stages.
#include <algorithm>
#include <utility>

#include "common.h"
#include "fmha_bwd_fused.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* lds_void_ptr;

constexpr int BS = 64;   // streamed rows per block
constexpr int BO = 128;  // owner rows per work-group
constexpr uint32_t kOob = 0x80000000u;
constexpr float kLog2e = 1.4426950408889634f;

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
};
template <> struct Elem<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ floatx16 mfma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

__device__ __forceinline__ floatx16 zero16() {
  return floatx16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load(__amdgpu_buffer_rsrc_t r, uint32_t voff) {
  return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
}
// s_waitcnt immediate (gfx9 encoding): vmcnt(n), lgkmcnt(0), expcnt untouched.
__host__ __device__ constexpr int wait_vm_lgkm0(int n) { return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4); }

struct KParams {
  const void* own1;   // owner operand of the score product:   K (owner = keys) or Q
  const void* own2;   // owner operand of the dP product:      V (owner = keys) or dO
  const void* strm1;  // streamed operand of the score product: Q (owner = keys) or K
  const void* strm2;  // streamed operand of the dP product:    dO (owner = keys) or V
  const void* bias;   // [units, F, T] additive bias of the scores, or null
  int bias_vec;       // queries-own pass: the bias may be read 4 keys (8 bytes) at a time
  float* lse;         // [units, F] LSE of the forward pass times log2(e)    } the queries-own launch writes them,
  float* dsum;        // [units, F] D = rowsum(dO o O)                       } the keys-own launches read them
  const void* o;      // [units, F, H] forward output and
  const float* lse_fwd;  // [units, F] its LSE (queries-own launch)
  void* out1;         // scale * dS^T Q (dK)  or  scale * dS K (dQ)
  void* out2;         // P^T dO (dV), owner = keys only
  int H, F, T;
  int nob;            // owner blocks per unit
  int total, per_xcd, ug;
  float scale;
};

// T: element type; HP: head size padded to 64, 128 or 256 (one wave per SIMD at 256); OWNER_K: the work-group owns keys (else queries).
// DS: accumulate out1 from dS (dK or dQ); PV: accumulate out2 from P (dV, owner = keys).  The
// keys-own work is run as two launches, one per output: with both accumulator sets and both owner
// operands a wave needs more than half the register file, and one wave per SIMD cannot overlap its
// matrix and vector work; recomputing S in a second launch at two waves per SIMD is faster.
// BIAS: S + bias enters the softmax; the bias is read from global memory at the start of each block
// (keys-own pass: 2-byte loads that are contiguous across the lanes of a wave; queries-own pass: each
// lane reads its own row, 8 bytes at a time where the alignment allows).
template <typename T, int HP, bool OWNER_K, bool CAUSAL, bool DS, bool PV, bool BIAS>
__global__ __launch_bounds__(256, (HP <= 128 && !BIAS && !(DS && PV && HP > 64)) ? 2 : 1) void fmha_bwd_kernel(KParams p) {
  static_assert(DS || PV, "nothing to compute");
  static_assert(!PV || OWNER_K, "P^T dO belongs to the keys-own pass");
  typedef typename Elem<T>::vec8 V8;
  constexpr int NW = 4;
  constexpr int ROWB = HP * 2;               // bytes of one tile row in LDS
  constexpr int CPR = ROWB / 16;             // 16-byte chunks per row
  constexpr int KMASK = 15;                  // the swizzle repeats every KMASK + 1 rows
  constexpr int TILE = BS * ROWB;
  constexpr int RPL = 1024 / ROWB;           // tile rows per 1 KiB load
  constexpr int NL = TILE / 1024 / NW;       // loads per wave per tile
  constexpr int LROWS = NW * RPL;            // tile rows between consecutive loads of a wave
  constexpr int KV = (LROWS % (KMASK + 1) == 0) ? 1 : 2;  // distinct swizzles among a wave's loads
  constexpr int KS = HP / 16;                // k-steps of the score products
  constexpr int HT = HP / 32;                // 32-wide h tiles of the gradients
  constexpr int STATS = 2 * BS * 4;          // LSE and D of one block's 64 query rows (owner = keys)
  static_assert(NL >= 1 && LROWS % 8 == 0 && (2 * LROWS) % (KMASK + 1) == 0, "tile / wave split");
  __shared__ __attribute__((aligned(1024))) char lds[4 * TILE + 2 * STATS];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5, l32 = lane & 31;
  // A tile row stores its 16-byte chunk c at position c ^ swz(row).  One tile serves two kinds of reads: row
  // fragments (16 lanes = 16 consecutive rows, one chunk column: swz must differ among 16 consecutive rows)
  // and transposed fragments (32 lanes = 4 consecutive rows x 4 adjacent chunks: bits 2-3 of swz must differ
  // among 4 consecutive rows, or the four rows land on the same banks).  Rows of 256 bytes and more: the two
  // bit pairs of row & 15, exchanged.  Rows of 128 bytes (8 chunks, two rows per 256 bytes of banks): the row's
  // parity already separates neighbours, and bits 1..3 of the row are dealt so that rows r and r + 2 differ in
  // bit 2 of swz and rows r and r + 8 in bit 1.
  auto swz = [](int row) {
    return CPR >= 16 ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
  };
  // Each XCD (own L2) gets a contiguous range of (unit, owner block) pairs: the owner blocks of a
  // unit stream the same tiles.
  const int wg = (int)(blockIdx.x % 8) * p.per_xcd + (int)(blockIdx.x / 8);
  if (wg >= p.total) return;
  // Inside the range, units go four at a time, owner blocks outermost and (causal) heaviest first, so that an
  // XCD's slots run dry at about the same time.
  const int UG = p.ug;
  const int ublk = wg / (UG * p.nob), r = wg % (UG * p.nob);
  const int gb = min(UG, p.total / p.nob - ublk * UG);  // units in this group (the last may hold fewer)
  const int unit = ublk * UG + r % gb;
  const int ob = OWNER_K ? r / gb : p.nob - 1 - r / gb;
  const int o0 = ob * BO;
  const int H = p.H;
  const int n_own = OWNER_K ? p.T : p.F;   // owner rows of the unit
  const int n_str = OWNER_K ? p.F : p.T;   // streamed rows of the unit

  const T* Own1 = reinterpret_cast<const T*>(p.own1) + (int64_t)unit * n_own * H;
  const T* Own2 = reinterpret_cast<const T*>(p.own2) + (int64_t)unit * n_own * H;
  const T* Str1 = reinterpret_cast<const T*>(p.strm1) + (int64_t)unit * n_str * H;
  const T* Str2 = reinterpret_cast<const T*>(p.strm2) + (int64_t)unit * n_str * H;
  float* lse = p.lse + (int64_t)unit * p.F;
  float* dsum = p.dsum + (int64_t)unit * p.F;

  // ---- owner fragments (B operands): this wave holds owner rows wo0 + l%32, fragment s covers
  // h = 16 s + 8 g .. +7.
  const int wo0 = o0 + wave * 32;
  const int orow = wo0 + l32;
  // They come in through LDS like the streamed tiles (below, once the tile loader is set up): read from global
  // memory in this layout, neighbouring lanes hold different rows, every lane is a cache access of its own, and
  // eight such loads per wave and operand cost the launch 18 us of load-path time at [8,32,2048,128].
  V8 of1[KS], of2[KS];
  // ---- streamed tile loads, global -> LDS, as in the forward kernel: load j = i * NW + wave fills
  // LDS bytes [1024 j, +1024) of the tile; lane l lands at row j * RPL + l / CPR, chunk l % CPR, and
  // fetches the global chunk that belongs there under the swizzle (swz below).
  const int lrow = wave * RPL + lane / CPR;
  uint32_t koff[KV];
#pragma unroll
  for (int v = 0; v < KV; ++v) {
    const int row = lrow + v * LROWS;
    const int chunk = (lane % CPR) ^ swz(row);
    koff[v] = chunk * 8 < H ? (uint32_t)((lrow * H + chunk * 8) * 2) : kOob;
  }
  const uint32_t lstride = (uint32_t)(LROWS * H * 2);
  auto issue_rows = [&](const T* base, int t0, char* __restrict__ tile, int n_rows) {
    const int rows_left = n_rows - t0;  // (<= 0: the whole tile is zeros)
    const __amdgpu_buffer_rsrc_t r = make_rsrc(base + (int64_t)t0 * H, 0x7fffffffu);
    const bool full = rows_left >= BS;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const uint32_t off = (full || lrow + i * LROWS < rows_left) ? koff[i % KV] : kOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void_ptr)(tile + (i * NW + wave) * 1024), 16, off,
                                               i * lstride, 0, 0);
    }
  };
  auto issue_tile = [&](const T* base, int t0, char* __restrict__ tile) { issue_rows(base, t0, tile, n_str); };
  // LSE (waves 0, 2) and D (waves 1, 3) of the block's 64 query rows, one float per lane; rows past
  // F load zeros.  Every wave issues one load so that the load counts stay uniform.
  auto issue_stats = [&](int t0, char* __restrict__ st) {
    const float* src = (wave & 1) ? dsum : lse;
    const __amdgpu_buffer_rsrc_t r = make_rsrc(src, (uint32_t)p.F * 4);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void_ptr)(st + (wave & 1) * (BS * 4)), 4,
                                             (uint32_t)((t0 + lane) * 4), 0, 0, 0);
  };

  // ---- per-lane LDS offsets of the fragments
  // Row fragment (kt, s): tile row 32 kt + l%32, logical chunk 2 s + g.
  int kbase[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) kbase[s] = l32 * ROWB + (((2 * s + g) ^ swz(l32)) << 4);
  // Transposed fragment (group u, h tile ht): two transpose reads; within a 16-lane block lane pl
  // addresses tile row 16 u + 4 g + pl/4 (+8 for the second read), h = cb + 4 (pl%4) .. +3.
  int tbase[HT][2];
  {
    const int pl = lane & 15;
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) {
      const int col = 32 * ht + ((lane >> 4) & 1) * 16 + 4 * (pl & 3);
      const int chunk = col >> 3, within = (col & 7) * 2;
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const int row = 4 * g + (pl >> 2) + 8 * h2;  // + 16 u: does not change swz(row)
        tbase[ht][h2] = row * ROWB + ((chunk ^ swz(row)) << 4) + within;
      }
    }
  }

  floatx16 acc1[DS ? HT : 1], acc2[PV ? HT : 1];
#pragma unroll
  for (int i = 0; i < (DS ? HT : 1); ++i) acc1[i] = zero16();
#pragma unroll
  for (int i = 0; i < (PV ? HT : 1); ++i) acc2[i] = zero16();
  const float scale2 = p.scale * kLog2e;
  auto to_f32 = [](uint16_t b) -> float {
    if constexpr (sizeof(T) == 2 && __is_same(T, __bf16)) return __builtin_bit_cast(float, (uint32_t)b << 16);
    else return (float)__builtin_bit_cast(_Float16, b);
  };
  // Bias of one block in the layout of the scores: bs[kt][i] <-> streamed row t0 + 32 kt + 8 (i/4) + 4 g + i%4.
  auto load_bias = [&](int t0, float (&bs)[2][16]) {
    const T* bb = reinterpret_cast<const T*>(p.bias) + (int64_t)unit * p.F * p.T;
    const __amdgpu_buffer_rsrc_t r = make_rsrc(bb, (uint32_t)((int64_t)p.F * p.T * 2));
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int s0 = t0 + 32 * kt + 8 * qd + 4 * g;  // first of 4 streamed rows
        if constexpr (OWNER_K) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int q = s0 + e;
            const uint32_t off = (q < p.F && orow < p.T) ? (uint32_t)(((int64_t)q * p.T + orow) * 2) : kOob;
            bs[kt][4 * qd + e] = to_f32((uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0));
          }
        } else {
          if (p.bias_vec) {  // T % 4 == 0: the 4 keys are inside the row or outside as a whole
            const uint32_t off = (orow < p.F && s0 < p.T) ? (uint32_t)(((int64_t)orow * p.T + s0) * 2) : kOob;
            const u32x2 w = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0));
#pragma unroll
            for (int e = 0; e < 4; ++e) bs[kt][4 * qd + e] = to_f32((uint16_t)(w[e >> 1] >> (16 * (e & 1))));
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const uint32_t off = (orow < p.F && s0 + e < p.T) ? (uint32_t)(((int64_t)orow * p.T + s0 + e) * 2) : kOob;
              bs[kt][4 * qd + e] = to_f32((uint16_t)__builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0));
            }
          }
        }
      }
  };

  // Blocks of streamed rows this work-group needs.
  //   owner = queries, causal: keys up to its last query.   owner = keys, causal: queries from its first key on.
  const int b0 = (OWNER_K && CAUSAL) ? o0 / BS : 0;
  const int b1 = (!OWNER_K && CAUSAL) ? (min(n_str, o0 + BO) + BS - 1) / BS : (n_str + BS - 1) / BS;

  // D[streamed row][owner row] = Stream_tile . Owner^T for the 64 streamed rows of a block.
  auto scores = [&](const char* __restrict__ tile, const V8 (&of)[KS], floatx16 (&st)[2]) {
    st[0] = zero16();
    st[1] = zero16();
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        const u32x4 kv = *reinterpret_cast<const u32x4*>(tile + kbase[s] + kt * 32 * ROWB);
        st[kt] = Elem<T>::mfma(__builtin_bit_cast(V8, kv), of[s], st[kt]);
      }
  };
  // The same for the 32 streamed rows of half kt alone.
  auto scores_half = [&](const char* __restrict__ tile, const V8 (&of)[KS], int kt, floatx16& st) {
    st = zero16();
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const u32x4 kv = *reinterpret_cast<const u32x4*>(tile + kbase[s] + kt * 32 * ROWB);
      st = Elem<T>::mfma(__builtin_bit_cast(V8, kv), of[s], st);
    }
  };
  // acc^T += Stream_tile^T . F, with F given as four B-operand fragments (group u contracts the
  // streamed rows 16 u + {0..3, 8..11} + 4 g).
  auto accumulate = [&](const char* __restrict__ tile, const V8 (&fr)[4], floatx16 (&acc)[HT]) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int ht = 0; ht < HT; ++ht) {
        typedef short4v __attribute__((address_space(3))) * lds_ptr;
        const char* vt = tile + u * 16 * ROWB;
        const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(vt + tbase[ht][0]));
        const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(vt + tbase[ht][1]));
        u32x4 vv;
        vv[0] = __builtin_bit_cast(u32x2, lo)[0];
        vv[1] = __builtin_bit_cast(u32x2, lo)[1];
        vv[2] = __builtin_bit_cast(u32x2, hi)[0];
        vv[3] = __builtin_bit_cast(u32x2, hi)[1];
        acc[ht] = Elem<T>::mfma(__builtin_bit_cast(V8, vv), fr[u], acc[ht]);
      }
  };

  char* const s1 = lds;              // streamed tiles of the score product, two stages
  char* const s2 = lds + 2 * TILE;   // streamed tiles of the dP product, two stages
  char* const sst = lds + 4 * TILE;  // statistics, two stages

  // ---- owner fragments: the block's BO = 2 BS owner rows of each operand fill the two stages of s1 / s2; wave w
  // picks its 32 rows' fragments up as row fragments of tile w / 2, half w % 2.
  static_assert(BO == 2 * BS, "an owner block fills both stages");
  const char* const own_at = lds + (wave >> 1) * TILE + (wave & 1) * 32 * ROWB;
  issue_rows(Own1, o0, s1, n_own);
  issue_rows(Own1, o0 + BS, s1 + TILE, n_own);
  if constexpr (DS) {
    issue_rows(Own2, o0, s2, n_own);
    issue_rows(Own2, o0 + BS, s2 + TILE, n_own);
  }
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    of1[s] = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4*>(own_at + kbase[s]));
    if constexpr (DS) of2[s] = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4*>(own_at + 2 * TILE + kbase[s]));
  }
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
  __builtin_amdgcn_s_barrier();  // every wave has its fragments: the stages may be overwritten
  // Softmax statistics of the lane's own query row (owner = queries): LSE log2(e) (one multiplication per row here
  // instead of one per score) and D = sum_h O[row][h] dO[row][h] (fmha_backward.h:48), formed from the dO fragments
  // the wave holds anyway and the same pieces of O, and written out for the keys-own launches that follow: a
  // separate pass over O and dO for them was 45 us at [8,32,2048,128].
  float own_lse2 = 0.f, own_d = 0.f;
  if constexpr (!OWNER_K) {
    static_assert(DS, "the queries-own launch holds dO");
    const T* Oo = reinterpret_cast<const T*>(p.o) + (int64_t)unit * n_own * H;
    issue_rows(Oo, o0, s1, n_own);
    issue_rows(Oo, o0 + BS, s1 + TILE, n_own);
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
    __builtin_amdgcn_s_barrier();
    float part = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const u32x4 ow = *reinterpret_cast<const u32x4*>(own_at + kbase[s]);
      const T* oe = reinterpret_cast<const T*>(&ow);
      const T* de = reinterpret_cast<const T*>(&of2[s]);
#pragma unroll
      for (int e = 0; e < 8; ++e) part += (float)oe[e] * (float)de[e];
    }
    own_d = part + __shfl_xor(part, 32);  // the row's other eight-element pieces are in lane l ^ 32
    if (orow < p.F) {
      own_lse2 = p.lse_fwd[(int64_t)unit * p.F + orow] * 1.4426950408889634f;
      if (g == 0) {
        lse[orow] = own_lse2;
        dsum[orow] = own_d;
      }
    }
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
    __builtin_amdgcn_s_barrier();
  }


  // One block: its tiles are in `c1`, `c2`, `cst`; the next block's go to `n1`, `n2`, `nst`.
  auto block = [&](int it, const char* __restrict__ c1, const char* __restrict__ c2, const char* __restrict__ cst,
                   char* __restrict__ n1, char* __restrict__ n2, char* __restrict__ nst) {
    const int t0 = it * BS;
    if (it + 1 < b1) {
      issue_tile(Str1, t0 + BS, n1);
      issue_tile(Str2, t0 + BS, n2);
      if constexpr (OWNER_K) issue_stats(t0 + BS, nst);
    }
    float bs[BIAS ? 2 : 1][16];
    if constexpr (BIAS) load_bias(t0, bs);
    // The dK launch of the larger head sizes holds both owner operands, the accumulators and the scores of
    // a whole block only with spills (30 registers): it goes through the block's two halves one after the
    // other, so that one half's scores are dead before the other's are made.
    constexpr bool BY_HALF = DS && ((OWNER_K && HP >= 128) || HP > 128);
    floatx16 sc[2], dp[2];
    if constexpr (!BY_HALF) {
      scores(c1, of1, sc);
      if constexpr (DS) scores(c2, of2, dp);
    }
    // sc[kt][i], dp[kt][i] <-> streamed row t0 + 32 kt + 8 (i/4) + 4 g + i%4, owner row `orow`.
    V8 pf[4], df[4];
    // Blocks that end inside the streamed range and (causal) lie wholly on the visible side of the
    // diagonal for every row of this wave need no mask (wave-uniform test).
    const bool masked = t0 + BS > n_str || (CAUSAL && (OWNER_K ? wo0 + 31 > t0 : t0 + BS - 1 > wo0));
    auto elementwise = [&](auto MASKED_T, auto KT_LO, auto KT_HI) {
      constexpr bool MASKED = decltype(MASKED_T)::value;
#pragma unroll
      for (int kt = decltype(KT_LO)::value; kt < decltype(KT_HI)::value; ++kt)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          floatx4 l2, dd;
          if constexpr (OWNER_K) {
            l2 = *reinterpret_cast<const floatx4*>(cst + (32 * kt + 8 * qd + 4 * g) * 4);
            dd = *reinterpret_cast<const floatx4*>(cst + BS * 4 + (32 * kt + 8 * qd + 4 * g) * 4);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int i = 4 * qd + e;
            const float lse2 = OWNER_K ? l2[e] : own_lse2;
            const float dq = OWNER_K ? dd[e] : own_d;
            float arg;
            if constexpr (BIAS) arg = __builtin_fmaf(sc[kt][i], scale2, __builtin_fmaf(bs[kt][i], kLog2e, -lse2));
            else arg = __builtin_fmaf(sc[kt][i], scale2, -lse2);
            if constexpr (MASKED) {
              // The mask goes into the exponent (a select on a ready value, exp2(-inf) = 0): with `pr = 0` after
              // the exponential the compiler branches around every single exponential instead.
              const int srow = t0 + 32 * kt + 8 * qd + 4 * g + e;
              const int q = OWNER_K ? srow : orow;
              const int key = OWNER_K ? orow : srow;
              arg = (srow >= n_str || (CAUSAL && key > q)) ? -INFINITY : arg;
            }
            const float pr = __builtin_amdgcn_exp2f(arg);
            // fragment u = 2 kt + (qd >> 1) holds registers 8 (u & 1) .. +7 of tile kt
            if constexpr (PV) pf[2 * kt + (qd >> 1)][4 * (qd & 1) + e] = (T)pr;
            if constexpr (DS) df[2 * kt + (qd >> 1)][4 * (qd & 1) + e] = (T)(pr * (dp[kt][i] - dq));
          }
        }
    };
    typedef std::integral_constant<int, 0> i0;
    typedef std::integral_constant<int, 1> i1;
    typedef std::integral_constant<int, 2> i2;
    if constexpr (BY_HALF) {
      scores_half(c1, of1, 0, sc[0]);
      scores_half(c2, of2, 0, dp[0]);
      if (masked) elementwise(std::true_type{}, i0{}, i1{});
      else elementwise(std::false_type{}, i0{}, i1{});
      scores_half(c1, of1, 1, sc[1]);
      scores_half(c2, of2, 1, dp[1]);
      if (masked) elementwise(std::true_type{}, i1{}, i2{});
      else elementwise(std::false_type{}, i1{}, i2{});
    } else {
      if (masked) elementwise(std::true_type{}, i0{}, i2{});
      else elementwise(std::false_type{}, i0{}, i2{});
    }
    if constexpr (DS) accumulate(c1, df, acc1);
    if constexpr (PV) accumulate(c2, pf, acc2);
    // The next block's tiles have landed (this wave's loads; every wave's after the barrier), and
    // this wave is done reading the tiles that the loads after the next block overwrite.
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
    __builtin_amdgcn_s_barrier();
  };

  if (b0 < b1) {
    issue_tile(Str1, b0 * BS, s1 + (b0 & 1) * TILE);
    issue_tile(Str2, b0 * BS, s2 + (b0 & 1) * TILE);
    if constexpr (OWNER_K) issue_stats(b0 * BS, sst + (b0 & 1) * STATS);
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
    __builtin_amdgcn_s_barrier();
    for (int it = b0; it < b1; ++it) {
      if (it & 1) block(it, s1 + TILE, s2 + TILE, sst + STATS, s1, s2, sst);
      else block(it, s1, s2, sst, s1 + TILE, s2 + TILE, sst + STATS);
    }
  }

  // ---- store: acc^T[h][owner row] -> out[owner row][h].  A lane holds 8 bytes in each of 16 places of its
  // row; the rounded rows go through this wave's own LDS region (the stages are free after the last block's
  // barrier), 16-byte chunks XORed with the row, and leave with 16-byte stores that cover whole rows.
  {
    constexpr int OCPR = HP / 8;  // 16-byte chunks per output row
    static_assert(4 * 32 * ROWB <= 4 * TILE, "the output rows are staged in the tile stages");
    char* region = lds + wave * (32 * ROWB);
    auto store = [&](void* out, const floatx16 (&acc)[HT], float mul) {
      static_for<HT>([&](auto HTI) {
        constexpr int ht = decltype(HTI)::value;
        const floatx16 o = acc[ht];
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          union { T e[4]; u32x2 w; } r;
          r.e[0] = (T)(o[4 * qd + 0] * mul);
          r.e[1] = (T)(o[4 * qd + 1] * mul);
          r.e[2] = (T)(o[4 * qd + 2] * mul);
          r.e[3] = (T)(o[4 * qd + 3] * mul);
          const int chunk = (4 * ht + qd) ^ (l32 & (OCPR - 1));
          *reinterpret_cast<u32x2*>(region + l32 * ROWB + (chunk << 4) + g * 8) = r.w;
        }
      });
      constexpr int RPI = 64 / OCPR;  // rows per store instruction
      const int c = lane % OCPR;
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int row = it * RPI + lane / OCPR;
        const u32x4 v = *reinterpret_cast<const u32x4*>(region + row * ROWB + ((c ^ (row & (OCPR - 1))) << 4));
        if (wo0 + row < n_own && c * 8 < H)  // H % 8 == 0: a chunk lies inside the row or outside as a whole
          *reinterpret_cast<u32x4*>(reinterpret_cast<T*>(out) + ((int64_t)unit * n_own + wo0 + row) * H + c * 8) = v;
      }
    };
    if constexpr (DS) store(p.out1, acc1, p.scale);
    if constexpr (PV) store(p.out2, acc2, 1.0f);
  }
}

template <typename T, int HP, bool OWNER_K, bool DS, bool PV>
void launch_pass(KParams p, uint64_t units, bool causal, hipStream_t st) {
  const int n_own = OWNER_K ? p.T : p.F;
  p.nob = (n_own + BO - 1) / BO;
  p.total = (int)(units * p.nob);
  p.per_xcd = (p.total + 7) / 8;
  p.ug = std::max(4, (64 + p.nob - 1) / p.nob);  // enough units to fill an XCD's slots with one round
  const dim3 grid((unsigned)(p.per_xcd * 8)), block(256);
  if (p.bias) {
    if (causal) hipLaunchKernelGGL((fmha_bwd_kernel<T, HP, OWNER_K, true, DS, PV, true>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((fmha_bwd_kernel<T, HP, OWNER_K, false, DS, PV, true>), grid, block, 0, st, p);
  } else {
    if (causal) hipLaunchKernelGGL((fmha_bwd_kernel<T, HP, OWNER_K, true, DS, PV, false>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((fmha_bwd_kernel<T, HP, OWNER_K, false, DS, PV, false>), grid, block, 0, st, p);
  }
}

template <typename T, int HP>
void launch_both(const fmha_bwd_fused::Args& a, uint64_t units, hipStream_t st) {
  KParams p;
  p.lse = a.lse; p.dsum = a.dsum; p.o = a.o; p.lse_fwd = a.lse_fwd; p.H = a.H; p.F = a.F; p.T = a.T; p.scale = a.scale;
  p.bias = a.bias;
  p.bias_vec = a.bias && a.T % 4 == 0 && xmk::aligned(a.bias, 8);
  p.nob = p.total = p.per_xcd = 0;
  // owner = queries first: dQ, and the per-row statistics the other launches read
  p.own1 = a.q; p.own2 = a.d_o; p.strm1 = a.k; p.strm2 = a.v; p.out1 = a.dq; p.out2 = nullptr;
  launch_pass<T, HP, false, true, false>(p, units, a.causal, st);
  // owner = keys: dK, then dV
  p.own1 = a.k; p.own2 = a.v; p.strm1 = a.q; p.strm2 = a.d_o; p.out1 = a.dk; p.out2 = a.dv;
  // One pass for both where the two accumulators fit beside everything else (S is then computed once for the
  // two): head size <= 64 (S = 4096, H = 64 causal: 0.69 -> 0.57 ms), and head size <= 128 with a bias, whose
  // kernels run one wave per SIMD anyway (6.2 -> 5.3 ms).  Without a bias the merged H = 128 pass would have to
  // give up the second wave per SIMD and comes out 2-4 % slower; at H = 256 it spills.
  if (HP <= 64 || (HP <= 128 && a.bias)) {
    launch_pass<T, HP, true, true, true>(p, units, a.causal, st);
  } else {
    launch_pass<T, HP, true, true, false>(p, units, a.causal, st);
    launch_pass<T, HP, true, false, true>(p, units, a.causal, st);
  }
}

}  // namespace

namespace fmha_bwd_fused {

bool eligible(const Args& a, uint64_t units) {
  return a.H <= 256 && a.H % 8 == 0 && units * ((uint64_t)((a.F > a.T ? a.F : a.T) + BO - 1) / BO) < 0x7fffffffull &&
         (uint64_t)a.F * a.H * 2 < kOob && (uint64_t)a.T * a.H * 2 < kOob &&
         (!a.bias || (uint64_t)a.F * a.T * 2 < kOob);
}

void launch(const Args& a, uint64_t units, bool bf16, hipStream_t st) {
  if (bf16) {
    if (a.H <= 64) launch_both<__bf16, 64>(a, units, st);
    else if (a.H <= 128) launch_both<__bf16, 128>(a, units, st);
    else launch_both<__bf16, 256>(a, units, st);
  } else {
    if (a.H <= 64) launch_both<_Float16, 64>(a, units, st);
    else if (a.H <= 128) launch_both<_Float16, 128>(a, units, st);
    else launch_both<_Float16, 256>(a, units, st);
  }
}

}  // namespace fmha_bwd_fused
