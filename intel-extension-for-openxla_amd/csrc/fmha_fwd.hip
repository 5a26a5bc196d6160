// Fused multi-head attention forward (flash attention) for bf16 / fp16:
//     O = softmax(scale * Q K^T + bias + mask) V,   optional LSE = m + log l.
//
// One work-group = NW waves, each owning QT tiles of 32 query rows of one (batch, head)
// unit; keys are walked in blocks of 64.  Both products are issued transposed so that a
// lane owns ONE query row per tile for the whole kernel:
//   S^T = K Q^T : A operand = K fragment (rows = keys) read from LDS, B operand = Q fragment
//                 kept in registers; the 32x32 accumulator layout puts query l%32 in lane l
//                 and keys in the lane's registers, so the row max is a register reduction
//                 plus one exchange with lane l^32 (which holds the other keys).  A K fragment
//                 read once from LDS feeds the MFMAs of all QT query tiles.
//   O^T += V^T P^T : P stays in registers (the accumulator registers, converted, ARE the B
//                 operand); V is staged untransposed [key][h] and read with the LDS transpose
//                 loads, which deliver four consecutive keys of one h.  The row sum of P comes
//                 from one more MFMA against a fragment of ones.
// K and V tiles go from global memory straight into LDS (buffer_load ... lds), two stages,
// the loads of block j+1 in flight while block j is computed.
// Online softmax in the exp2 domain: the scale is folded into the exponent (one FMA per
// element), the running reference max only moves when a block max exceeds it by more than
// 2^8 (so O is rescaled in few blocks), and O is divided by l once at the end.  Causal: key >
// query masked (top-left aligned), key blocks past the diagonal are never visited, work-groups
// are issued heaviest first.
#include <algorithm>
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
typedef __attribute__((address_space(3))) void* lds_void_ptr;

constexpr int BC = 64;  // keys per step
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

// x *= alpha for an MFMA accumulator that stays in the accumulator registers.  Written out so
// that the register allocator keeps the accumulators in one register file through the rare
// rescale path instead of moving all of them between files in every iteration.  The leading
// and trailing waits cover the MFMA -> VALU and VALU -> MFMA hazards, which the compiler
// cannot see through the asm text.
__device__ __forceinline__ void scale_acc(floatx16& x, float alpha) {
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
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load(__amdgpu_buffer_rsrc_t r, uint32_t voff) {
  return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
}
// s_waitcnt immediate (gfx9 encoding): vmcnt(n), lgkmcnt(0), expcnt untouched.
__host__ __device__ constexpr int wait_vm_lgkm0(int n) { return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4); }

// T: element type; HP: head size padded to 64 / 128 / 256; QT: 32-row query tiles per wave;
// NW: waves per work-group; WPS: waves per SIMD the register budget is set for.
// BIAS: 0 none; 1 read from global memory element by element (any shape and alignment); 2 staged
// through LDS one [rows x 64 keys] tile per key block (T % 8 == 0, 16-byte aligned bias).
template <typename T, int HP, int QT, int NW, int WPS, bool CAUSAL, int BIAS>
__global__ __launch_bounds__(NW * 64, WPS) void fmha_fwd_kernel(FmhaParams p) {
  typedef typename Elem<T>::vec8 V8;
  constexpr int BR = NW * QT * 32;           // query rows per work-group
  constexpr int ROWB = HP * 2;               // bytes of one K / V row in LDS
  constexpr int CPR = ROWB / 16;             // 16-byte chunks per row
  constexpr int KMASK = CPR >= 16 ? 15 : 7;  // K rows: chunk ^= key & KMASK (16 lanes -> 16 bank groups)
  constexpr int TILE = BC * ROWB;            // one K or V tile
  constexpr int RPL = 1024 / ROWB;           // tile rows per 1 KiB load
  constexpr int NL = TILE / 1024 / NW;       // loads per wave per tile
  constexpr int LROWS = NW * RPL;            // tile rows between consecutive loads of a wave
  constexpr int KV = (LROWS % (KMASK + 1) == 0) ? 1 : 2;  // distinct K swizzles among a wave's loads
  constexpr int KS = HP / 16;                // k-steps of the S product
  constexpr int HT = HP / 32;                // 32-wide h tiles of O
  static_assert(NL >= 1 && LROWS % 8 == 0 && (2 * LROWS) % (KMASK + 1) == 0, "tile / wave split");
  constexpr int BTILE = 32 * BC * 2;         // one wave's bias tile: its 32 query rows x 64 keys
  static_assert(BIAS != 2 || (QT == 1 && BC == 64), "bias staging is laid out for one 32 x 64 tile per wave");
  __shared__ __attribute__((aligned(1024))) char lds[4 * TILE + (BIAS == 2 ? NW * BTILE : 0)];

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

  const T* Q = reinterpret_cast<const T*>(p.q) + (int64_t)unit * F * H;
  const T* K = reinterpret_cast<const T*>(p.k) + (int64_t)unit * Tk * H;
  const T* V = reinterpret_cast<const T*>(p.v) + (int64_t)unit * Tk * H;

  // ---- Q fragments (B operand of S^T): tile t of this wave holds query rows wq0 + 32 t + l%32,
  // fragment s covers h = 16 s + 8 g .. +7.
  const int wq0 = q0 + wave * (QT * 32);
  V8 qf[QT][KS];
  {
    const int rows_left = F - q0;  // > 0
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(Q + (int64_t)q0 * H, (uint32_t)rows_left * H * 2);
#pragma unroll
    for (int t = 0; t < QT; ++t)
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int h = 16 * s + 8 * g;
        const int r = wave * (QT * 32) + 32 * t + l32;
        const uint32_t off = h < H ? (uint32_t)((r * H + h) * 2) : kOob;  // rows past F are out of range
        qf[t][s] = __builtin_bit_cast(V8, buf_load(rq, off));
      }
  }

  // ---- K / V tile loads, global -> LDS.  Load j = i * NW + wave fills LDS bytes [1024 j, +1024)
  // of the tile, i.e. tile rows j * RPL ..; lane l lands at row j * RPL + l / CPR, chunk l % CPR,
  // and fetches the global chunk that belongs there under the tile's swizzle.
  const int lrow = wave * RPL + lane / CPR;  // tile row of this lane in load 0; load i: + i * LROWS
  uint32_t koff[KV];
#pragma unroll
  for (int v = 0; v < KV; ++v) {
    const int row = lrow + v * LROWS;
    const int chunk = (lane % CPR) ^ (row & KMASK);
    koff[v] = chunk * 8 < H ? (uint32_t)((lrow * H + chunk * 8) * 2) : kOob;
  }
  // V rows: chunk ^= vswz(key).  A transpose read touches 4 chunks of each of 4 consecutive keys;
  // the XOR moves each key's group of 4 chunks to its own banks.
  auto vswz = [](int key) { return CPR >= 16 ? (key & 3) << 2 : (key & 2) << 1; };
  const int vchunk = (lane % CPR) ^ vswz(lrow);
  const uint32_t voff = vchunk * 8 < H ? (uint32_t)((lrow * H + vchunk * 8) * 2) : kOob;
  const uint32_t lstride = (uint32_t)(LROWS * H * 2);  // global bytes between a wave's loads
  // One tile (64 rows from row t0 of K or V) into `tile`.  The per-load scalar offset is not
  // range-checked by the hardware, so in the one ragged block rows past T are turned into
  // out-of-range lane offsets, which load zeros.
  auto issue_tile = [&](const T* base, int t0, char* __restrict__ tile, const uint32_t* offs, int noffs) {
    const int rows_left = Tk - t0;  // > 0
    const __amdgpu_buffer_rsrc_t r = make_rsrc(base + (int64_t)t0 * H, 0x7fffffffu);
    const bool full = rows_left >= BC;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const uint32_t off = (full || lrow + i * LROWS < rows_left) ? offs[i % noffs] : kOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void_ptr)(tile + (i * NW + wave) * 1024), 16, off,
                                               i * lstride, 0, 0);
    }
  };

  // ---- per-lane LDS offsets of the fragments
  // K fragment (kt, s): key row 32 kt + l%32, logical chunk 2 s + g.
  int kbase[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) kbase[s] = l32 * ROWB + (((2 * s + g) ^ (l32 & KMASK)) << 4);
  // V^T fragment (group u, h tile ht): two transpose reads; within a 16-lane block lane pl
  // addresses key row 16 u + 4 g + pl/4 (+8 for the second read), h = cb + 4 (pl%4) .. +3.
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
  // its own 4 KiB of LDS, loaded with four 1 KiB direct loads (8 rows of 128 bytes each) one block
  // ahead.  Row r stores its 16-byte chunk c at position c ^ ((r >> 1) & 7), so that the 8-byte reads
  // of 32 lanes (32 rows, one chunk column) spread over the banks.
  uint32_t boff[4];  // global byte offset of this lane's chunk in load i, from bias row q0, key 0
  int bkey[4];       // first key (within the block) of that chunk
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
  // Loads the bias tile of the key block that starts at t0.  T % 8 == 0, so a chunk lies inside
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

  floatx16 ot[QT][HT];
  float m_run[QT], l_run[QT];  // l_run: this lane's share (its 32 keys of every block) of the row sum
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    m_run[t] = -INFINITY;
    l_run[t] = 0.0f;
#pragma unroll
    for (int i = 0; i < HT; ++i) ot[t][i] = zero16();
  }
  const float inv_scale = kLog2e / p.scale2;  // bias is added in score units: (s + b / scale) * scale

  const int kend = CAUSAL ? min(Tk, q0 + BR) : Tk;  // keys this work-group can see
  const int nblk = (kend + BC - 1) / BC;

  // S^T = K Q^T of one key block for all query tiles; each K fragment is read once.
  auto scores = [&](const char* __restrict__ ktile, floatx16 (&st)[QT][2]) {
#pragma unroll
    for (int t = 0; t < QT; ++t) { st[t][0] = zero16(); st[t][1] = zero16(); }
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        const u32x4 kv = *reinterpret_cast<const u32x4*>(ktile + kbase[s] + kt * 32 * ROWB);
#pragma unroll
        for (int t = 0; t < QT; ++t) st[t][kt] = Elem<T>::mfma(__builtin_bit_cast(V8, kv), qf[t][s], st[t][kt]);
      }
  };

  // Bias, masks, block max and (rarely) the rescale of tile t; returns the exponent reference.
  // st[kt][i] <-> key t0 + 32 kt + 8 (i/4) + 4 g + i%4.  Scores stay unscaled; the scale is
  // folded into the exponent.
  auto prepare = [&](auto TI, floatx16 (&st)[2], int t0, const u32x2 (&bv)[8]) -> float {
    constexpr int t = decltype(TI)::value;
    const int qrow = wq0 + 32 * t + l32;
    if constexpr (BIAS == 2) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) st[kt][i] += bias_value(bv[4 * kt + i / 4], i % 4) * inv_scale;
    }
    if constexpr (BIAS == 1) {
      if (qrow < F) {
        const T* bp = reinterpret_cast<const T*>(p.bias) + ((int64_t)unit * F + qrow) * Tk;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key = t0 + 32 * kt + 8 * (i / 4) + 4 * g + (i % 4);
            if (key < Tk) st[kt][i] += (float)bp[key] * inv_scale;
          }
      }
    }
    const bool diag = CAUSAL && (t0 + BC - 1 > wq0 + 32 * t);
    const bool tail = t0 + BC > Tk;
    if (diag || tail) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = t0 + 32 * kt + 8 * (i / 4) + 4 * g + (i % 4);
          if ((CAUSAL && key > qrow) || key >= Tk) st[kt][i] = -INFINITY;
        }
    }
    // The reference max m_run only moves when some row's block max exceeds it by more than 2^8
    // (wave-uniform test): P then stays below 256, and O is rescaled in few blocks instead of all.
    float mx = fmaxf(st[0][0], st[0][1]);
#pragma unroll
    for (int i = 2; i < 16; i += 2) mx = fmaxf(fmaxf(mx, st[0][i]), st[0][i + 1]);  // v_max3_f32
#pragma unroll
    for (int i = 0; i < 16; i += 2) mx = fmaxf(fmaxf(mx, st[1][i]), st[1][i + 1]);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float mx2 = mx * p.scale2;
    if (__any(mx2 > m_run[t] + 8.0f)) {
      const float m_new = fmaxf(m_run[t], mx2);
      const float alpha = __builtin_amdgcn_exp2f(m_run[t] - m_new);  // first block: exp2(-inf) = 0
      m_run[t] = m_new;
      l_run[t] *= alpha;
#pragma unroll
      for (int ht = 0; ht < HT; ++ht) scale_acc(ot[t][ht], alpha);
    }
    // A row that has seen no visible key keeps m_run = -inf; use 0 as its reference so that
    // its masked (-inf) scores give exp2(-inf) = 0 and not NaN.
    return m_run[t] == -INFINITY ? 0.0f : m_run[t];
  };

  // P = exp2(s * scale2 - mref) of one tile as four B-operand fragments (group u contracts keys
  // 16 u + {0..3, 8..11} + 4 g), and the lane's row-sum share, summed from the rounded values
  // the P V product uses.
  auto probs = [&](const floatx16 (&st)[2], float mref, V8 (&pf)[4], float& lsum) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        pf[u][j] = (T)__builtin_amdgcn_exp2f(__builtin_fmaf(st[u >> 1][8 * (u & 1) + j], p.scale2, -mref));
#pragma unroll
      for (int j = 0; j < 8; j += 2) lsum = Elem<T>::dot2_ones(pf[u][j], pf[u][j + 1], lsum);
    }
  };

  // O^T += V^T P^T for tile t.
  auto accumulate = [&](auto TI, const char* __restrict__ vtile, const V8 (&pf)[4]) {
    constexpr int t = decltype(TI)::value;
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int ht = 0; ht < HT; ++ht) {
        typedef short4v __attribute__((address_space(3))) * lds_ptr;
        const char* vt = vtile + u * 16 * ROWB;
        const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(vt + vbase[ht][0]));
        const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(vt + vbase[ht][1]));
        u32x4 vv;
        vv[0] = __builtin_bit_cast(u32x2, lo)[0];
        vv[1] = __builtin_bit_cast(u32x2, lo)[1];
        vv[2] = __builtin_bit_cast(u32x2, hi)[0];
        vv[3] = __builtin_bit_cast(u32x2, hi)[1];
        ot[t][ht] = Elem<T>::mfma(__builtin_bit_cast(V8, vv), pf[u], ot[t][ht]);
      }
  };

  // LDS: K tiles of blocks j, j+1 in kst[j & 1], V tiles in vst[j & 1].
  char* const kst0 = lds;
  char* const vst0 = lds + 2 * TILE;

  // Prologue: K_0, then K_1 and V_0; S_0 is computed as soon as K_0 is there.
  issue_tile(K, 0, kst0, koff, KV);
  if (nblk > 1) issue_tile(K, BC, kst0 + TILE, koff, KV);
  issue_tile(V, 0, vst0, &voff, 1);
  char* const btile0 = lds + 4 * TILE + wave * BTILE;  // this wave's bias tile (BIAS == 2)
  constexpr int NB = BIAS == 2 ? 4 : 0;                // loads of one bias tile
  if constexpr (BIAS == 2) issue_bias(0, btile0);
  if (nblk > 1) __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(2 * NL + NB));
  else __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(NL + NB));
  __builtin_amdgcn_s_barrier();
  floatx16 st_a[QT][2], st_b[QT][2];
  scores(kst0, st_a);
  __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
  __builtin_amdgcn_s_barrier();

  // One key block j: `sc` holds S_j; K_{j+1} and V_j are in LDS.  Loads of K_{j+2} and V_{j+1}
  // are issued first and land during the block.  S_{j+1} (MFMA) is issued among the exponentials
  // of tile 0 (VALU), the P V product of tile 0 among those of tile 1.  The four tile pointers
  // never overlap (__restrict__), so the compiler does not make the fragment reads wait for the
  // loads in flight.
  // With a staged bias, the block first takes its bias tile out of LDS (it landed during the
  // previous block) and then sends the next block's tile into the same 4 KiB.
  auto block = [&](int it, floatx16 (&sc)[QT][2], floatx16 (&sn)[QT][2], const char* __restrict__ knext,
                   const char* __restrict__ vcur, char* __restrict__ kfree, char* __restrict__ vfree,
                   char* __restrict__ btile) {
    const int t0 = it * BC;
    u32x2 bv[8];
    if constexpr (BIAS == 2) {
#pragma unroll
      for (int r = 0; r < 8; ++r) bv[r] = *reinterpret_cast<const u32x2*>(btile + bread[r]);
    }
    if (it + 2 < nblk) issue_tile(K, t0 + 2 * BC, kfree, koff, KV);
    if (it + 1 < nblk) issue_tile(V, t0 + BC, vfree, &voff, 1);
    if constexpr (BIAS == 2) {
      if (it + 1 < nblk) issue_bias(t0 + BC, btile);
    }
    float mref[QT];
    static_for<QT>([&](auto TI) { mref[decltype(TI)::value] = prepare(TI, sc[decltype(TI)::value], t0, bv); });
    V8 pf[QT][4];
    // Past the last block this reads a stale tile: finite or not, S_{nblk} is never used.
    scores(knext, sn);
    probs(sc[0], mref[0], pf[0], l_run[0]);
    static_for<QT>([&](auto TI) {
      constexpr int t = decltype(TI)::value;
      accumulate(TI, vcur, pf[t]);
      if constexpr (t + 1 < QT) probs(sc[t + 1], mref[t + 1], pf[t + 1], l_run[t + 1]);
    });
    if constexpr (QT == 1) {
      // Issue order for the scheduler: LDS fragment reads run three MFMAs ahead of their use, the
      // exponentials are spread under the S MFMAs, and the copies of S_{j+1} out of the
      // accumulator registers under the P V MFMAs.
      constexpr int NS = 2 * KS, NP = 4 * HT, AHEAD = 3;  // MFMAs of S and of P V
      constexpr int VALU_S = (32 + 32 + 16 + 16 + NS - 1) / NS;
      __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
      static_for<NS>([&](auto I) {
        constexpr int i = decltype(I)::value;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, i + AHEAD < NS ? 1 : 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, VALU_S, 0);
      });
      static_for<NP>([&](auto I) {
        constexpr int i = decltype(I)::value;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if constexpr (i + AHEAD < NP) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, (32 + NP - 1) / NP, 0);
      });
    }
    // K_{j+2} and V_{j+1} have landed (this wave's loads; every wave's after the barrier), and
    // this wave is done reading the tiles the next block's loads overwrite.
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
    __builtin_amdgcn_s_barrier();
  };

  for (int it = 0; it < nblk; it += 2) {
    // K_{it+1} sits in K stage 1, V_it in V stage 0; K_{it+2} goes to K stage 0, V_{it+1} to V stage 1.
    block(it, st_a, st_b, kst0 + TILE, vst0, kst0, vst0 + TILE, btile0);
    if (it + 1 < nblk) block(it + 1, st_b, st_a, kst0, vst0 + TILE, kst0 + TILE, vst0, btile0);
  }

  // ---- finish: O = O^T / l; LSE = m ln2 + ln l.  The accumulator layout gives a lane 8 bytes in each of 16
  // places of its row, so the rounded rows go through LDS (free after the last block's barrier; one region of
  // 32 rows per wave and query tile, 16-byte chunks XORed with the row so that both passes spread over the
  // banks) and leave with 16-byte stores that cover whole rows.
  constexpr int OCPR = HP / 8;  // 16-byte chunks per output row
  static_assert(QT * NW * 32 * ROWB <= 4 * TILE, "the output tiles are staged in the K / V stages");
  static_for<QT>([&](auto TI) {
    constexpr int t = decltype(TI)::value;
    const int qrow = wq0 + 32 * t + l32;
    const float l_tot = l_run[t] + __shfl_xor(l_run[t], 32);
    const float inv = 1.0f / l_tot;
    char* region = lds + (wave * QT + t) * (32 * ROWB);
    static_for<HT>([&](auto HTI) {
      constexpr int ht = decltype(HTI)::value;
      const floatx16 o = ot[t][ht];
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
    if (qrow < F && p.lse && g == 0) p.lse[(int64_t)unit * F + qrow] = m_run[t] * 0.6931471805599453f + logf(l_tot);
    // this wave's own region: its LDS writes are complete for its own reads once lgkmcnt is zero
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(63));
    constexpr int RPI = 64 / OCPR;  // rows per store instruction
    const int c = lane % OCPR;
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
      const int row = it * RPI + lane / OCPR;
      const u32x4 v = *reinterpret_cast<const u32x4*>(region + row * ROWB + ((c ^ (row & (OCPR - 1))) << 4));
      const int qr = wq0 + 32 * t + row;
      if (qr < F && c * 8 < H)  // H % 8 == 0: a chunk lies inside the row or outside as a whole
        *reinterpret_cast<u32x4*>(reinterpret_cast<T*>(p.out) + ((int64_t)unit * F + qr) * H + c * 8) = v;
    }
  });
}

template <typename T, int HP, int QT, int NW, int WPS>
void launch_cfg(FmhaParams p, uint64_t units, uint32_t F, bool causal, int bias, hipStream_t st) {
  p.nqb = (int)((F + NW * QT * 32 - 1) / (NW * QT * 32));
  p.total = (int)(units * p.nqb);
  p.per_xcd = (p.total + 7) / 8;
  // Four units at a time (measured on causal [8,32,2048,128]: 1: 697, 2: 730, 4: 756, 8: 751, 16: 733, 32: 699
  // TFLOP/s), more when a unit has so few query blocks that four units do not fill an XCD's 64 slots.
  p.ug = std::max(4, (64 + p.nqb - 1) / p.nqb);
  const dim3 grid((unsigned)(p.per_xcd * 8)), block(NW * 64);
  // bias: 0 none, 1 element-wise from global memory, 2 staged through LDS
  if (causal) {
    if (bias == 2) hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, QT, NW, WPS, true, 2>), grid, block, 0, st, p);
    else if (bias == 1) hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, QT, NW, WPS, true, 1>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, QT, NW, WPS, true, 0>), grid, block, 0, st, p);
  } else {
    if (bias == 2) hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, QT, NW, WPS, false, 2>), grid, block, 0, st, p);
    else if (bias == 1) hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, QT, NW, WPS, false, 1>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, QT, NW, WPS, false, 0>), grid, block, 0, st, p);
  }
}

template <typename T>
void launch_t(const FmhaParams& p, uint64_t units, uint32_t F, bool causal, int bias, hipStream_t st) {
  // Head-size classes of the reference's policy choice (fmha_forward.h:622-646).  Two query tiles
  // per wave where the accumulators fit in the register file (head size <= 128).
  if (p.H <= 64) launch_cfg<T, 64, 1, 4, 2>(p, units, F, causal, bias, st);
  else if (p.H <= 128) launch_cfg<T, 128, 1, 4, 2>(p, units, F, causal, bias, st);
  else launch_cfg<T, 256, 1, 4, 1>(p, units, F, causal, bias, st);
}

}  // namespace

extern "C" int xmk_fmha_fwd(const void* query, const void* key, const void* value, const void* bias,
                            void* out, float* lse, int32_t dtype, uint32_t num_batches,
                            uint32_t num_heads, uint32_t head_size, uint32_t num_queries,
                            uint32_t num_keys, float head_scale, int32_t causal, void* stream) {
  if (!query || !key || !value || !out) return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: null pointer");
  if (dtype != XMK_F16 && dtype != XMK_BF16)
    return xmk::fail(XMK_INTERNAL, "Invalid MHA datatype");  // xetla_gpu_fused_mha_runner.cc:145
  if (num_batches == 0 || num_heads == 0 || head_size == 0 || num_queries == 0 || num_keys == 0)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: empty dimension");
  if (head_size > 256)
    return xmk::fail(XMK_UNIMPLEMENTED, "fmha_fwd: head_size %u > 256 (fmha_forward.h:642)", head_size);
  if (head_size % 8 != 0)
    return xmk::fail(XMK_UNIMPLEMENTED, "fmha_fwd: head_size %u is not a multiple of 8", head_size);
  if (!(head_scale > 0.0f) || head_scale > 3.0e38f)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: head_scale must be positive and finite");
  const uint64_t units = (uint64_t)num_batches * num_heads;
  if (units * ((num_queries + 31) / 32) > 0x7fffffffull || (uint64_t)num_keys * head_size * 2 >= kOob ||
      (uint64_t)num_queries * head_size * 2 >= kOob)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: shape too large");
  if (!xmk::aligned(query, 16) || !xmk::aligned(key, 16) || !xmk::aligned(value, 16) ||
      !xmk::aligned(out, 16))
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: tensors must be 16-byte aligned");
  FmhaParams p;
  p.q = query; p.k = key; p.v = value; p.bias = bias; p.out = out; p.lse = lse;
  p.H = (int)head_size; p.F = (int)num_queries; p.T = (int)num_keys;
  p.nqb = p.total = p.per_xcd = 0;
  p.scale2 = head_scale * kLog2e;
  xmk::trace("fmha_fwd B=%u N=%u F=%u T=%u H=%u causal=%d bias=%d lse=%d", num_batches, num_heads,
             num_queries, num_keys, head_size, causal, bias != nullptr, lse != nullptr);
  hipStream_t st = (hipStream_t)stream;
  // The staged bias path needs whole 16-byte chunks per row and offsets inside one query block
  // that fit the 31-bit buffer offset.
  const int bias_mode = !bias ? 0
                        : (num_keys % 8 == 0 && xmk::aligned(bias, 16) && (uint64_t)num_keys * 2 * 128 < kOob) ? 2
                                                                                                            : 1;
  if (dtype == XMK_BF16) launch_t<__bf16>(p, units, num_queries, causal != 0, bias_mode, st);
  else launch_t<_Float16>(p, units, num_queries, causal != 0, bias_mode, st);
  return xmk::check_launch("fmha_fwd");
}
