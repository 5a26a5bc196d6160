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
// where the second sum comes from one extra MFMA against a B operand of ones, and the offsets the
// unpack trick leaves on q are taken out by starting each group's accumulators at
// -sum_k a[m,k] offset_k (one more extra MFMA, against a constant fragment).  The kernel
// is bound by HBM only if the per-weight VALU work stays near one operation, so the
// nibbles are expanded with the fp16 "magic number" trick (5 operations per 8 weights).
#include <cstdlib>
#include <type_traits>

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

// (a & mask) | magic.  `magic_vgpr` must be a value the compiler cannot see through (it is
// laundered through an empty asm at the call site): with a known constant it emits separate
// v_and and v_or (VOP3 takes one scalar source and no literal), with an opaque VGPR it selects
// the single v_and_or_b32.  No instruction is written by hand here on purpose: the hazard
// recogniser cannot see inside inline asm, and these results feed MFMAs.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic_vgpr) {
  return (a & mask) | magic_vgpr;
}

// One packed word -> 8 fp16 values q + offset, in k-slot order (0,4,1,5,2,6,3,7):
// 0x6400 | q is 1024 + q (slots 0,1,4,5) and 0x5400 | (q << 4) is 64 + q (slots 2,3,6,7).
// The offsets are not subtracted here (that would cost as many VALU operations again);
// they are removed per quantisation group through -sum_k a_k * offset_k, which one extra
// MFMA against a constant fragment provides as the accumulators' start value.  5 VALU operations
// per 8 weights.
__device__ __forceinline__ half8 unpack_word(uint32_t w, uint32_t m1024, uint32_t m64) {
  const uint32_t w8 = w >> 8;
  Frag f;
  f.u[0] = and_or(w, 0x000f000fu, m1024);
  f.u[1] = and_or(w, 0x00f000f0u, m64);
  f.u[2] = and_or(w8, 0x000f000fu, m1024);
  f.u[3] = and_or(w8, 0x00f000f0u, m64);
  return f.h;
}

// 8 consecutive activations -> the same k-slot order (0,4,1,5,2,6,3,7).
// sel_lo = 0x05040100, sel_hi = 0x07060302 (passed in so that the caller can order these operations).
__device__ __forceinline__ half8 permute_act(u32x4 d, uint32_t sel_lo, uint32_t sel_hi) {
  Frag f;
  f.u[0] = __builtin_amdgcn_perm(d[2], d[0], sel_lo);  // (h0, h4)
  f.u[1] = __builtin_amdgcn_perm(d[2], d[0], sel_hi);  // (h1, h5)
  f.u[2] = __builtin_amdgcn_perm(d[3], d[1], sel_lo);  // (h2, h6)
  f.u[3] = __builtin_amdgcn_perm(d[3], d[1], sel_hi);  // (h3, h7)
  return f.h;
}

constexpr uint32_t kOob = 0x80000000u;
typedef __attribute__((address_space(3))) void* lds_void_ptr;
// s_waitcnt immediate: at most n vector-memory loads outstanding, the other counters not waited for.
constexpr int vmcnt_imm(int n) { return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4) | (0xf << 8); }
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

// 16 bytes per lane from byte offset voff + soff of a buffer straight into LDS: lane l's land at lds + 16 l
// (zeros where the offset is out of range).  (A function of its own: written into a kernel's body, the
// builtin makes the host pass drop the kernel's launch stub.)
__device__ __forceinline__ void load_to_lds(__amdgpu_buffer_rsrc_t r, char* lds, uint32_t voff, uint32_t soff) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void_ptr)lds, 16, voff, soff, 0, 0);
}

template <int NWORDS>
struct Words {
  uint32_t w[NWORDS];
};

// NWORDS consecutive dwords at byte offset voff + soff of a buffer.
template <int NWORDS>
__device__ __forceinline__ Words<NWORDS> load_words(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  Words<NWORDS> o;
  if constexpr (NWORDS == 4) {
    const u32x4 v = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
    o.w[0] = v[0]; o.w[1] = v[1]; o.w[2] = v[2]; o.w[3] = v[3];
  } else if constexpr (NWORDS == 2) {
    const auto v = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0);
    o.w[0] = v[0]; o.w[1] = v[1];
  } else {
    o.w[0] = __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0);
  }
  return o;
}
// W consecutive fp16 values at byte offset voff + soff, as packed dwords.
template <int W>
__device__ __forceinline__ Words<(W + 1) / 2> load_halves(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  if constexpr (W == 1) {
    Words<1> o;
    o.w[0] = __builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0);
    return o;
  } else {
    return load_words<W / 2>(r, voff, soff);
  }
}
template <int NWORDS>
__device__ __forceinline__ float half_at(const Words<NWORDS>& r, int c) {
  const uint16_t bits = (uint16_t)(r.w[c / 2] >> (16 * (c % 2)));
  return (float)__builtin_bit_cast(_Float16, bits);
}

// W    : words (output channels) per lane; a block covers 16*W output channels
// MT   : 16-row activation tiles (1 or 2)
// RI   : accumulator rows per lane that can be live (4, or fewer when M <= 4 so that the
//        per-group fix-up only touches rows that exist)
// SPG  : 32-channel k-steps a wave handles at a time (one load batch, one fix-up)
// SDIV : such batches per quantisation group (group = 32 * SPG * SDIV): groups of 256 channels run as two
//        batches of 128 that read the same scale and zero point -- s (d1 - z a1) + s (d2 - z a2) -- because
//        a batch of 256 does not fit the register file (it spilled over a hundred registers)
// NW   : waves per block; wave w takes groups w, w+NW, ... and the partial
//        sums meet in LDS in a fixed order (deterministic result)
// SPREAD: 2 to 4 rows (RI = 1) or 5 to 8 rows (RI = 2): activation row r is fed to the MFMA as row
//        (4 / RI) r, the rows between are zeros, so that the live rows come out in accumulator elements
//        0 (and 2) of every lane group and the per-group fix-up touches RI elements per lane instead of four
// SK   : K is also split over gridDim.y work-groups; slice y writes its fp32 partial sums
//        [32 rows][N] to partial + y * 32 * N and applies no epilogue (the consumer adds the
//        slices in a fixed order)
//
// One launch can carry two independent products of the same tile shape (e.g. the q/k/v and
// fc_in projections of a decoder block, which read the same activations): blocks
// [0, blocks0) work on p0, the rest on p1.
struct Int4Problem {
  const _Float16* act;
  const uint32_t* qw;
  const _Float16* scales;
  const _Float16* zeros;
  const _Float16* bias;
  _Float16* out;
  int m_base, M, K, N;
  xmk::Int4Epilogue ep;
  float* partial;
};

// f(integral_constant<I>), ..., f(integral_constant<N - 1>) in turn, stopping after the first that returns false.
template <int I, int N, class F>
__device__ __forceinline__ void static_steps(F&& f) {
  if constexpr (I < N) {
    if (f(std::integral_constant<int, I>{})) static_steps<I + 1, N>(f);
  }
}

// The first activation staging buffer of a work-group; the waves' partial sums take its place after the K loop.
template <int STAGE_BYTES, int SUMS>
union alignas(1024) StageOrSums {
  char stage[STAGE_BYTES];
  float sums[SUMS];
};

template <int W, int MT, int RI, int SPG, int NW, bool SK, bool SPREAD, int SDIV = 1>
__global__ __launch_bounds__(NW * 64) void int4_gemm_kernel(Int4Problem p0, Int4Problem p1, int blocks0, int mixed) {
  // Every argument the K loop needs is asked for here, so that the scalar loads of the argument block go out
  // together and the kernel starts after one round trip to it.  (Left to itself the compiler fetched them in
  // two or three dependent rounds in some instantiations: 0.25 us on a launch of 9.)
  if constexpr (NW != 16)  // (the sixteen-wave one-row form: 8.8 -> 9.15 us with it)
    asm volatile("" : : "s"(p0.act), "s"(p1.act), "s"(p0.qw), "s"(p1.qw), "s"(p0.scales), "s"(p1.scales), "s"(p0.zeros),
                 "s"(p1.zeros), "s"(p0.m_base), "s"(p1.m_base), "s"(p0.M), "s"(p1.M), "s"(p0.K), "s"(p1.K), "s"(p0.N),
                 "s"(p1.N), "s"(blocks0), "s"(mixed));
  // mixed (two K-split products of equal width): the products alternate from one block to the next, and
  // the alternation flips between the first and the second half of the K slices, so that work-groups
  // which are half a grid apart -- the ones that end up sharing a CU -- belong to different products
  // and every CU gets the same share of the longer reduction.
  const bool second = (SK && mixed) ? (((int)blockIdx.x + (int)(blockIdx.y >> 1)) & 1) != 0 : (int)blockIdx.x >= blocks0;
  const int bx = (SK && mixed) ? (int)blockIdx.x >> 1 : (int)blockIdx.x - (second ? blocks0 : 0);
  const _Float16* __restrict__ act = second ? p1.act : p0.act;
  const uint32_t* __restrict__ qw = second ? p1.qw : p0.qw;
  const _Float16* __restrict__ scales = second ? p1.scales : p0.scales;
  const _Float16* __restrict__ zeros = second ? p1.zeros : p0.zeros;
  const _Float16* __restrict__ bias = second ? p1.bias : p0.bias;
  _Float16* __restrict__ out = second ? p1.out : p0.out;
  const int m_base = second ? p1.m_base : p0.m_base, M = second ? p1.M : p0.M;
  const int K = second ? p1.K : p0.K, N = second ? p1.N : p0.N;
  const xmk::Int4Epilogue ep = second ? p1.ep : p0.ep;
  float* __restrict__ partial = second ? p1.partial : p0.partial;
  constexpr int NCOL = 16 * W;
  static_assert(!SPREAD || (MT == 1 && (RI == 1 || RI == 2)), "spread rows: one tile, one or two live elements per lane");
  constexpr int ROWS = SPREAD ? 4 * RI : (MT == 2 ? 32 : (RI == 4 ? 16 : RI));  // rows the block reduces
  constexpr int ESTEP = SPREAD ? 4 / RI : 1;  // live accumulator elements are 0, ESTEP, ...
  // kExact: work-groups that own their whole reduction, of eight waves, or four with several rows (see the
  // fetch below).
  // kStage: such work-groups with more than one row bring the activations in through LDS.  Read straight into
  // the matrix instruction's operand layout (lane -> row l % 16, 16 bytes of it), a load touches 64 separate
  // 64-byte pieces, one per lane group, because neighbouring lanes hold different rows: measured at 32 rows,
  // the CU's load path spent 64 cycles on every such load against 16 for a load of the packed weights, 20
  // thousand of the launch's 33 thousand cycles.  Instead each wave copies its group's ROWS x (64 SPG) bytes
  // global -> LDS with lanes along the rows (16 per 1 KiB load), into a region of its own, and picks the
  // operand fragments up with 16-byte LDS reads.  Chunk c of row r lives in slot c ^ sw(r) of the row, which
  // spreads the 16 rows a read phase touches over all banks.  No barrier: a wave reads what it loaded itself,
  // and the vector-memory counter orders the two.
  constexpr bool kExact = (NW == 8 || (NW == 4 && ROWS > 1)) && !SK;
  constexpr bool kStage = kExact && ROWS > 1 && !(SPG == 1 && SPREAD);  // (groups of 32, up to 8 rows: 4-5 % slower staged)
  constexpr int CPR = 4 * SPG;                              // 16-byte chunks per activation row and group
  constexpr int NI = kStage ? (ROWS * CPR + 63) / 64 : 0;   // 1 KiB loads per group and wave
  constexpr int REGION = NI * 1024;                         // bytes per wave and buffer
  // (the 256 bytes behind the waves' regions stay zero: the operand rows that carry no activation row read them)
  constexpr int STAGE_BYTES = kStage ? NW * REGION + 256 : 16;
  constexpr int kLoadsPerFetch = 2 + NI + SPG;  // scales, zero points, staging loads, weights: one instruction each
  static_assert(SPG + kLoadsPerFetch < 64, "the wait below counts up to 63 loads");
  __shared__ StageOrSums<STAGE_BYTES, NW * ROWS * NCOL> s0;  // two objects, so that the compiler can tell a read
  __shared__ alignas(1024) char s1[STAGE_BYTES];             // of one buffer from a load into the other
  float (*red)[ROWS][NCOL] = reinterpret_cast<float (*)[ROWS][NCOL]>(s0.sums);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col16 = lane & 15;
  const int kg = lane >> 4;
  const int n0 = bx * NCOL + col16 * W;
  const bool col_ok = n0 < N;
  const int ngroups = K / (32 * SPG);  // batches; ngroups / SDIV rows of scales and zero points

  // Buffer descriptors: hardware bounds checking zero-fills lanes that are out of range
  // (offset kOob), and the per-lane byte offsets below never change inside the K loop.
  const __amdgpu_buffer_rsrc_t r_none = make_rsrc(qw, 0);
  const __amdgpu_buffer_rsrc_t r_w_all = make_rsrc(qw, (uint32_t)((size_t)(K / 8) * N * 4));
  const __amdgpu_buffer_rsrc_t r_s_all = make_rsrc(scales, (uint32_t)((size_t)(ngroups / SDIV) * N * 2));
  const __amdgpu_buffer_rsrc_t r_z_all = make_rsrc(zeros, (uint32_t)((size_t)(ngroups / SDIV) * N * 2));
  // (the 32 rows of this launch only: the byte count must fit the descriptor's 32 bits for any M)
  const __amdgpu_buffer_rsrc_t r_a_all = make_rsrc(act + (size_t)m_base * K, (uint32_t)((size_t)min(M - m_base, 32) * K * 2));
  const uint32_t voff_w = col_ok ? (uint32_t)((kg * N + n0) * 4) : kOob;
  const uint32_t voff_sz = col_ok ? (uint32_t)(n0 * 2) : kOob;
  uint32_t voff_a[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = SPREAD ? col16 / ESTEP : mt * 16 + col16;
    const bool fed = !SPREAD || col16 % ESTEP == 0;  // MFMA rows ESTEP r carry activation row r, the others zeros
    voff_a[mt] = (fed && m_base + m < M) ? (uint32_t)((m * K + 8 * kg) * 2) : kOob;
  }

  uint32_t voff_st[kStage ? NI : 1];  // staging load i: this lane's chunk of the group's activations
  uint32_t rd_off[SPG];               // k-step s: where this lane's operand fragment of tile 0 sits in the wave's region
  if constexpr (kStage) {
    constexpr int RPS = 16 / CPR;  // rows per 256 bytes of LDS
    const int rows_here = min(M - m_base, ROWS);
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int l = i * 64 + lane, row = l / CPR, chunk = (l % CPR) ^ ((row / RPS) % CPR);
      voff_st[i] = row < rows_here ? (uint32_t)((row * K + chunk * 8) * 2) : kOob;
    }
    const int lr = SPREAD ? col16 / ESTEP : col16;
    const bool fed = !SPREAD || col16 % ESTEP == 0;
    const uint32_t at = fed ? (uint32_t)(wave * REGION + (lr * CPR + (kg ^ ((lr / RPS) % CPR))) * 16) : (uint32_t)(NW * REGION);
#pragma unroll
    for (int s = 0; s < SPG; ++s) rd_off[s] = at ^ (uint32_t)(s << 6);
    if (lane < 16) {
      *reinterpret_cast<u32x4*>(s0.stage + NW * REGION + lane * 16) = u32x4{0u, 0u, 0u, 0u};
      *reinterpret_cast<u32x4*>(s1 + NW * REGION + lane * 16) = u32x4{0u, 0u, 0u, 0u};
    }
  }

  floatx4 acc[MT][W];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int c = 0; c < W; ++c) acc[mt][c] = floatx4{0.f, 0.f, 0.f, 0.f};

  Frag ones, noffs;  // B operands that yield sum_k a_k and -sum_k a_k * offset_k
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ones.u[i] = 0x3c003c00u;
    noffs.u[i] = (i & 1) ? 0xd400d400u : 0xe400e400u;  // -64, -1024
  }
  uint32_t m1024 = 0x64006400u, m64 = 0x54005400u;
  asm volatile("" : "+v"(m1024), "+v"(m64));  // keep the magic constants in VGPRs

  // Everything a group needs (scales, zero points, activations, weights) is fetched one
  // group ahead, weights last: vector loads return in order, so computing group g waits only
  // for loads issued an iteration earlier, never for the prefetch of group g + NW.
  struct GroupData {
    Words<W> w[SPG];
    Words<(W + 1) / 2> sc, zp;
    u32x4 a[SPG][MT];
  };
  // kExact (work-groups that own their whole reduction: eight waves, or four with more than one row): a fetch
  // past the wave's last group is still issued, through descriptors of no bytes (no memory access, zeros
  // returned), and the groups run as straight-line code, so that the sequence of loads is the same on every
  // path and the counted waits the compiler places before a group's arithmetic leave the next group's loads
  // in flight.  The other shapes keep a loop with fetches behind branches, whose waits drain the prefetch at
  // every turn: measured on one device, the exact form is 9-12 % faster at 8 rows and 5 % at 32 (k 4096,
  // n 16384), 3-5 % slower on the sixteen-wave one-row kernel, and level on the K-split launches; on the
  // four-wave form it is 1.4 % slower over a decode step by itself and 1.5 % faster together with the staged
  // activations.
  auto fetch = [&](int g_asked, GroupData& d, bool live, auto which) {
    // (a fetch past the end uses group 0's scalar offsets, so that kOob plus the scalar offset cannot wrap
    //  around 32 bits whatever the unit that checks the range adds up)
    const int g = live ? g_asked : 0;
    // (wave-uniform; said explicitly, or the compiler wraps each of the two loads in a loop over lane values)
    const uint32_t so = __builtin_amdgcn_readfirstlane((uint32_t)((g / SDIV) * N * 2));
    // (a fetch past the end: descriptors of no bytes, four scalar selects instead of a vector select per load)
    const __amdgpu_buffer_rsrc_t r_s = live ? r_s_all : r_none, r_z = live ? r_z_all : r_none;
    const __amdgpu_buffer_rsrc_t r_a = live ? r_a_all : r_none, r_w = live ? r_w_all : r_none;
    const uint32_t vsz = voff_sz, vw = voff_w;
    constexpr bool kPinned = kExact;
    if constexpr (kPinned) __builtin_amdgcn_sched_barrier(0);  // the loads stay together and in this order
    d.sc = load_halves<W>(r_s, vsz, so);
    d.zp = load_halves<W>(r_z, vsz, so);
    if constexpr (kStage) {
      char* dst = (which == 0 ? s0.stage : s1) + wave * REGION;
#pragma unroll
      for (int i = 0; i < NI; ++i)
        load_to_lds(r_a, dst + i * 1024, voff_st[i], (uint32_t)(g * SPG * 64));
    } else {
#pragma unroll
      for (int s = 0; s < SPG; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          d.a[s][mt] = __builtin_bit_cast(
              u32x4, __builtin_amdgcn_raw_buffer_load_b128(r_a, voff_a[mt], (uint32_t)((g * SPG + s) * 64), 0));
    }
#pragma unroll
    for (int s = 0; s < SPG; ++s)
      d.w[s] = load_words<W>(r_w, vw, (uint32_t)((g * 4 * SPG + s * 4) * N * 4));
    // Every unpack reads these constants and every activation shuffle a selector derived from them, so
    // the arithmetic that follows in program order is also emitted after these loads (instruction
    // selection is free to order what has no side effects, and would otherwise wait for a group's
    // activations before the next fetch goes out).
    if constexpr (kPinned) {
      asm volatile("" : "+v"(m1024), "+v"(m64) : : "memory");
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto compute = [&](const GroupData& cur, auto which) {
    floatx4 d[MT][W], asum[MT], noff[MT];
    half8 a[SPG][MT];
    // (kExact: derived from the constant that the fetch has just laundered, see there)
    const uint32_t sel_lo = kExact ? m64 ^ (0x54005400u ^ 0x05040100u) : 0x05040100u;
    const uint32_t sel_hi = kExact ? m64 ^ (0x54005400u ^ 0x07060302u) : 0x07060302u;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      asum[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
      noff[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    // The staged activations of this group have landed once at most the loads issued after them are
    // outstanding: this group's weights and the whole next fetch (always issued in this form).  Said
    // explicitly: inside the loop that follows the straight-line groups the compiler left this wait out
    // before the reads of one of the two buffers.
    if constexpr (kStage) __builtin_amdgcn_s_waitcnt(vmcnt_imm(SPG + kLoadsPerFetch));
    // -sum_k a_k offset_k of the whole group first: it is the start value of every column's
    // accumulator chain, so that the chains end at sum_k a_k q_k with the unpack offsets gone.
#pragma unroll
    for (int s = 0; s < SPG; ++s)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        u32x4 raw;
        if constexpr (kStage)
          raw = *reinterpret_cast<const u32x4*>((which == 0 ? s0.stage : s1) + rd_off[s] + mt * (16 * CPR * 16));
        else
          raw = cur.a[s][mt];
        a[s][mt] = permute_act(raw, sel_lo, sel_hi);
        noff[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[s][mt], noffs.h, noff[mt], 0, 0, 0);
      }
#pragma unroll
    for (int s = 0; s < SPG; ++s) {
#pragma unroll
      for (int c = 0; c < W; ++c) {
        const half8 b = unpack_word(cur.w[s].w[c], m1024, m64);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          d[mt][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[s][mt], b, s == 0 ? noff[mt] : d[mt][c], 0, 0, 0);
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        asum[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[s][mt], ones.h, asum[mt], 0, 0, 0);
    }
    // acc += s * (sum a q - z sum a), only for rows that can exist
#pragma unroll
    for (int c = 0; c < W; ++c) {
      const float sc = half_at(cur.sc, c), z = half_at(cur.zp, c);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < RI; ++i) {
          const int e = i * ESTEP;
          acc[mt][c][e] = fmaf(sc, fmaf(-z, asum[mt][e], d[mt][c][e]), acc[mt][c][e]);
        }
    }
  };

  // Two register buffers, one group in flight while one is computed.  (Three were slower wherever they were
  // tried: 5-7 % at 2 to 16 rows on the eight-wave form, 1.747 against 1.704 ms over a decode step on the
  // four-wave one.)
  constexpr int DEPTH = 2;
  GroupData buf[DEPTH];
  // This work-group's share of the groups: all of them, or slice blockIdx.y of gridDim.y.
  const int gper = SK ? (ngroups + (int)gridDim.y - 1) / (int)gridDim.y : ngroups;
  const int gend = SK ? min(ngroups, ((int)blockIdx.y + 1) * gper) : ngroups;
  int g = (SK ? (int)blockIdx.y * gper : 0) + wave;  // groups g, g + NW, ... below gend are this wave's
  if constexpr (kExact) {
    // The first kStraight groups as straight-line code with forward exits only: no loop edge merges two
    // histories of outstanding loads.  (Around a loop with an exit in its middle the compiler's wait
    // accounting merges the path that leaves with the path that goes round.)  Compile-time buffer indices
    // throughout: a buffer indexed by a loop variable would live in scratch memory.
    const int mine = g < gend ? (gend - g + NW - 1) / NW : 0;
    constexpr int kStraight = DEPTH == 3 ? 9 : 8;
    static_steps<0, DEPTH - 1>([&](auto j) {
      fetch(g + j * NW, buf[j], j < mine, j);
      return true;
    });
    static_steps<0, kStraight>([&](auto i) {
      if (i >= mine) return false;
      fetch(g + (i + DEPTH - 1) * NW, buf[(i + DEPTH - 1) % DEPTH], i + DEPTH - 1 < mine,
            std::integral_constant<int, (decltype(i)::value + DEPTH - 1) % DEPTH>{});
      compute(buf[i % DEPTH], std::integral_constant<int, decltype(i)::value % DEPTH>{});
      return true;
    });
    // long reductions: the rest in a loop (buf[j] holds group kStraight + j; kStraight is a multiple of DEPTH)
    for (int i = kStraight; i < mine;) {
      static_steps<0, DEPTH>([&](auto j) {
        if (i >= mine) return false;
        fetch(g + (i + DEPTH - 1) * NW, buf[(j + DEPTH - 1) % DEPTH], i + DEPTH - 1 < mine,
              std::integral_constant<int, (decltype(j)::value + DEPTH - 1) % DEPTH>{});
        compute(buf[j], j);
        ++i;
        return true;
      });
    }
  } else {
    constexpr std::integral_constant<int, 0> b0{};
    constexpr std::integral_constant<int, 1> b1{};
    if (g < gend) fetch(g, buf[0], true, b0);
    while (g < gend) {
      if (g + NW < gend) fetch(g + NW, buf[1], true, b1);
      compute(buf[0], b0);
      g += NW;
      if (g >= gend) break;
      if (g + NW < gend) fetch(g + NW, buf[0], true, b0);
      compute(buf[1], b1);
      g += NW;
    }
  }
  if constexpr (kStage) {
    // The partial sums below reuse the staging memory: every load into it has landed (the fetches past the end
    // write zeros there) and every wave has read its last group.
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
  }

  // Lane holds rows 4*kg+i (+16 mt) of columns col16*W+c.
  // Q: columns per thread of the reduction below.  Where single values would take four rounds or more (32 rows
  // on eight waves, 16 on four: measured 1.9 us at 32 rows), a lane's four columns of a row go to LDS as one
  // 16-byte store and a thread of the reduction owns such a quad: one round of 16-byte reads.  With fewer
  // rounds the quads are slower (one row 8.8 -> 9.25 us, eight rows 9.0 -> 9.55, decode step +1.3 %).
  constexpr int Q = (W == 4 && ROWS * NCOL >= 4 * NW * 64) ? 4 : 1;
  auto put = [&](int row, int i, int mt) {
    if constexpr (Q == 4) {
      *reinterpret_cast<floatx4*>(&red[wave][row][col16 * 4]) = floatx4{acc[mt][0][i], acc[mt][1][i], acc[mt][2][i], acc[mt][3][i]};
    } else {
#pragma unroll
      for (int c = 0; c < W; ++c) red[wave][row][col16 * W + c] = acc[mt][c][i];
    }
  };
  if constexpr (SPREAD) {
#pragma unroll
    for (int j = 0; j < RI; ++j) put(kg * RI + j, j * ESTEP, 0);
  } else if (RI == 4 || kg == 0) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < RI; ++i) put(mt * 16 + (RI == 4 ? 4 * kg : 0) + i, i, mt);
  }
  __syncthreads();

  // Thread e of the reduction owns Q consecutive columns of one row: sums over the waves in wave order.
  const int rows = min(ROWS, M - m_base);
  auto wave_sums = [&](int row, int col, float (&sum)[Q]) {
    if constexpr (Q == 4) {
      floatx4 v = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < NW; ++w) v += *reinterpret_cast<const floatx4*>(&red[w][row][col]);
      sum[0] = v[0]; sum[1] = v[1]; sum[2] = v[2]; sum[3] = v[3];
    } else {
      sum[0] = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) sum[0] += red[w][row][col];
    }
  };
  if constexpr (SK) {
    // This work-group's partial sums, fp32, no epilogue: the consumer adds the slices up.
    float* mine = partial + (size_t)blockIdx.y * 32 * N;
    for (int e = threadIdx.x; e < rows * (NCOL / Q); e += NW * 64) {
      const int row = e / (NCOL / Q), col = e % (NCOL / Q) * Q;
      const int n = bx * NCOL + col;
      if (n >= N) continue;
      float sum[Q];
      wave_sums(row, col, sum);
      if constexpr (Q == 4) {  // (N is a multiple of 8 and the host checks the buffer's alignment)
        *reinterpret_cast<floatx4*>(mine + (size_t)row * N + n) = floatx4{sum[0], sum[1], sum[2], sum[3]};
      } else {
        mine[(size_t)row * N + n] = sum[0];
      }
    }
    return;
  }
  if (Q == 4 && ep.rope_d <= 0) {
    // plain epilogue, a quad per thread
    const bool out8 = (reinterpret_cast<uintptr_t>(out) & 7) == 0;  // the quad can go out as 8 bytes
    for (int e = threadIdx.x; e < rows * (NCOL / Q); e += NW * 64) {
      const int row = e / (NCOL / Q), col = e % (NCOL / Q) * Q;
      const int n = bx * NCOL + col;
      if (n >= N) continue;  // (N is a multiple of 8: a quad is inside or outside as a whole)
      float sum[Q];
      wave_sums(row, col, sum);
      const size_t o = (size_t)(m_base + row) * N + n;
      _Float16 res[Q];
#pragma unroll
      for (int c = 0; c < Q; ++c) {
        float v = sum[c];
        if (bias) v += (float)bias[n + c];
        if (ep.gelu) {  // gelu_new, see below
          const float u = 0.7978845608028654f * (v + 0.044715f * v * v * v);
          v = v / (1.0f + __expf(-2.0f * u));
        }
        if (ep.add0) v += (float)reinterpret_cast<const _Float16*>(ep.add0)[o + c];
        if (ep.add1) v += (float)reinterpret_cast<const _Float16*>(ep.add1)[o + c];
        res[c] = (_Float16)v;
      }
      if (out8) {
        typedef _Float16 half4 __attribute__((ext_vector_type(4)));
        *reinterpret_cast<half4*>(out + o) = half4{res[0], res[1], res[2], res[3]};
      } else {
#pragma unroll
        for (int c = 0; c < Q; ++c) out[o + c] = res[c];
      }
    }
    return;
  }
  for (int e = threadIdx.x; e < rows * NCOL; e += NW * 64) {
    const int row = e / NCOL, col = e % NCOL;
    const int n = bx * NCOL + col;
    if (n >= N) continue;
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) s += red[w][row][col];
    if (bias) s += (float)bias[n];
    if (ep.rope_d > 0) {
      const int d = ep.rope_d, which = n / d, hd = n % d;  // 0 q, 1 k, 2 v; element of the [heads, head_dim] row
      const int head = hd / ep.head_dim, i = hd % ep.head_dim;
      if (which < 2 && i < ep.rotary_dim) {
        // the other element of the rotary pair sits in the neighbouring column of this block
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) t += red[w][row][col ^ 1];
        if (bias) t += (float)bias[n ^ 1];
        const float inv_freq = powf(10000.0f, -(float)(i & ~1) / (float)ep.rotary_dim);
        float sn, cs;
        sincosf((float)ep.position * inv_freq, &sn, &cs);
        s = (i & 1) ? s * cs + t * sn : s * cs - t * sn;
      }
      const int m = m_base + row;
      if (which == 0) {
        reinterpret_cast<_Float16*>(ep.q_out)[(size_t)m * d + hd] = (_Float16)s;
      } else {
        _Float16* cache = reinterpret_cast<_Float16*>(which == 1 ? ep.k_cache : ep.v_cache);
        const int heads = d / ep.head_dim;
        cache[(((size_t)m * heads + head) * ep.capacity + ep.position) * ep.head_dim + i] = (_Float16)s;
      }
      continue;
    }
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

// One product as the host sees it, and the tile configuration chosen for it.
struct Config {
  int w = 4, nw = 16, ksplit = 1;
  bool operator==(const Config& o) const { return w == o.w && nw == o.nw && ksplit == o.ksplit; }
};

template <int W, int MT, int RI, int SPG, int NW, bool SPREAD, int SDIV = 1>
void launch(const Int4Problem& a, const Int4Problem* b, int ksplit, hipStream_t st) {
  const int blocks0 = (int)xmk::ceil_div(a.N, 16 * W);
  const int blocks = blocks0 + (b ? (int)xmk::ceil_div(b->N, 16 * W) : 0);
  const Int4Problem& second = b ? *b : a;
  if (ksplit > 1) {
    if constexpr (W == 4 && MT == 1) {  // the only shape the split is planned for
      const int mixed = b && blocks == 2 * blocks0 && ksplit % 4 == 0 ? 1 : 0;
      hipLaunchKernelGGL((int4_gemm_kernel<W, MT, RI, SPG, NW, true, SPREAD, SDIV>), dim3(blocks, ksplit), dim3(NW * 64), 0, st, a,
                         second, blocks0, mixed);
      return;
    }
  }
  hipLaunchKernelGGL((int4_gemm_kernel<W, MT, RI, SPG, NW, false, SPREAD, SDIV>), dim3(blocks), dim3(NW * 64), 0, st, a, second,
                     blocks0, 0);
}

template <int W, int MT, int RI, int NW, bool SPREAD = false>
int launch_spg(int spg, const Int4Problem& a, const Int4Problem* b, int ksplit, hipStream_t st) {
  switch (spg) {
    case 1: launch<W, MT, RI, 1, NW, SPREAD>(a, b, ksplit, st); break;
    case 2: launch<W, MT, RI, 2, NW, SPREAD>(a, b, ksplit, st); break;
    case 4: launch<W, MT, RI, 4, NW, SPREAD>(a, b, ksplit, st); break;
    case 8: launch<W, MT, RI, 4, NW, SPREAD, 2>(a, b, ksplit, st); break;  // groups of 256: two batches of 128
    default: return xmk::fail(XMK_UNIMPLEMENTED, "int4_gemm: group must be 32, 64, 128 or 256");
  }
  return XMK_OK;
}

// Checks one product and picks its tile configuration.
int prepare(const xmk::Int4Call& c, int64_t m, int64_t group, Config* cfg) {
  if (!c.act || !c.qweight || !c.scales || !c.zeros || (!c.out && c.split.ksplit <= 1))
    return xmk::fail(XMK_INVALID_ARGUMENT, "int4_gemm: null pointer");
  const int64_t k = c.k, n = c.n;
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
  // The kernel addresses the packed weights, the scales and the zero points with 32-bit byte offsets.
  if ((uint64_t)(k / 8) * (uint64_t)n * 4 >= (1ull << 31))
    return xmk::fail(XMK_INVALID_ARGUMENT, "int4_gemm: packed weights of 2 GiB or more (k=%lld n=%lld)", (long long)k,
                     (long long)n);
  if (!xmk::aligned(c.act, 16) || !xmk::aligned(c.qweight, 16) || !xmk::aligned(c.scales, 8) ||
      !xmk::aligned(c.zeros, 8) || !xmk::aligned(c.out, 2))
    return xmk::fail(XMK_INVALID_ARGUMENT, "int4_gemm: act, qweight must be 16-byte and scales, zeros 8-byte aligned");
  // Words per lane: the widest load that still yields about one block per CU.
  cfg->w = 4;
  if (n / 64 < 192) cfg->w = 2;
  if (n / 32 < 192) cfg->w = 1;
  cfg->nw = 16;
  // XMK_INT4_TILE="<words per lane>,<waves per block>" overrides the choice (tuning aid).
  static const char* tile_env = getenv("XMK_INT4_TILE");
  if (tile_env) {
    int ew = 0, enw = 0;
    if (sscanf(tile_env, "%d,%d", &ew, &enw) == 2 && (ew == 1 || ew == 2 || ew == 4) && (enw == 4 || enw == 8 || enw == 16)) {
      cfg->w = ew;
      cfg->nw = enw;
    }
  }
  cfg->ksplit = 1;
  if (c.split.ksplit > 1) {
    if (m > 16 || !c.split.partial || !xmk::aligned(c.split.partial, 16) || c.split.ksplit > xmk::kInt4MaxSplit ||
        c.split.partial_bytes < (size_t)c.split.ksplit * 32 * n * sizeof(float))
      return xmk::fail(XMK_INTERNAL, "int4_gemm: bad K split request");
    cfg->w = 4;
    cfg->nw = 8;
    cfg->ksplit = c.split.ksplit;
  }
  return XMK_OK;
}

Int4Problem problem(const xmk::Int4Call& c, int m_base, int M) {
  Int4Problem p;
  p.act = (const _Float16*)c.act; p.qw = (const uint32_t*)c.qweight; p.scales = (const _Float16*)c.scales;
  p.zeros = (const _Float16*)c.zeros; p.bias = (const _Float16*)c.bias; p.out = (_Float16*)c.out;
  p.m_base = m_base; p.M = M; p.K = (int)c.k; p.N = (int)c.n;
  p.ep = c.ep;
  p.partial = c.split.ksplit > 1 ? c.split.partial : nullptr;
  return p;
}

// Launches `a` (and `b`, if given, in the same grid) for rows [m_base, m_base + 32).
int launch_cfg(const Config& cfg, int spg, const xmk::Int4Call& a, const xmk::Int4Call* b, int m_base, int M,
               hipStream_t st) {
  const Int4Problem pa = problem(a, m_base, M);
  Int4Problem pb_store;
  const Int4Problem* pb = nullptr;
  if (b) {
    pb_store = problem(*b, m_base, M);
    pb = &pb_store;
  }
  const int rows = M - m_base;
  int rc;
#define XMK_INT4_CASE(WW)                                                            \
  do {                                                                               \
    if (rows > 16) rc = launch_spg<WW, 2, 4, 8>(spg, pa, pb, cfg.ksplit, st);        \
    else if (rows > 1 && rows <= 4)                                                  \
      rc = cfg.nw == 4 ? launch_spg<WW, 1, 1, 4, true>(spg, pa, pb, cfg.ksplit, st)  \
                       : launch_spg<WW, 1, 1, 8, true>(spg, pa, pb, cfg.ksplit, st); \
    else if (rows > 4 && rows <= 8)                                                  \
      rc = cfg.nw == 4 ? launch_spg<WW, 1, 2, 4, true>(spg, pa, pb, cfg.ksplit, st)  \
                       : launch_spg<WW, 1, 2, 8, true>(spg, pa, pb, cfg.ksplit, st); \
    else if (rows > 1) rc = cfg.nw == 4 ? launch_spg<WW, 1, 4, 4>(spg, pa, pb, cfg.ksplit, st)   \
                                        : launch_spg<WW, 1, 4, 8>(spg, pa, pb, cfg.ksplit, st); \
    else rc = cfg.nw == 16 ? launch_spg<WW, 1, 1, 16>(spg, pa, pb, cfg.ksplit, st)   \
                           : launch_spg<WW, 1, 1, 8>(spg, pa, pb, cfg.ksplit, st);   \
  } while (0)
  if (cfg.w == 4) XMK_INT4_CASE(4);
  else if (cfg.w == 2) XMK_INT4_CASE(2);
  else XMK_INT4_CASE(1);
#undef XMK_INT4_CASE
  return rc;
}

}  // namespace

int xmk::int4_plan_split(int64_t m, int64_t k, int64_t n, int64_t group) {
  // Worth it when 64-column blocks alone cannot fill the device (256 CUs) and every wave of
  // every slice still gets at least one quantisation group.
  if (m > 16 || group <= 0 || k % group != 0) return 1;
  const int64_t blocks = xmk::ceil_div(n, 64);
  if (blocks >= 192) return 1;
  // XMK_INT4_SPLIT=<k splits> overrides the choice (tuning aid).
  static const char* split_env = getenv("XMK_INT4_SPLIT");
  if (split_env) {
    const int e = atoi(split_env);
    if (e >= 1 && e <= kInt4MaxSplit) return e;
  }
  int ks = (int)(256 / blocks);
  if (ks > kInt4MaxSplit) ks = kInt4MaxSplit;
  while (ks > 1 && (k / group) / ks < 8) ks /= 2;
  return ks < 1 ? 1 : ks;
}

int xmk::int4_gemm_launch2(const Int4Call& a, const Int4Call* b, int64_t m, int64_t group, hipStream_t st) {
  Config ca, cb;
  int rc = prepare(a, m, group, &ca);
  if (rc != XMK_OK) return rc;
  if (b && (rc = prepare(*b, m, group, &cb)) != XMK_OK) return rc;
  const int spg = (int)(group / 32);
  const int M = (int)m;
  // One grid for both when they take the same tile shape; else one after the other.
  const bool together = b && ca == cb;
  // 2 to 16 rows: a launch of more blocks than the 256 CUs runs four-wave work-groups, three of which
  // share a CU, so that the blocks beyond a multiple of 256 do not cost a whole extra round (measured:
  // 448 blocks 19.0 -> 17.7 us, 787 blocks 30.7 -> 28.1 us; 256 blocks or fewer are faster with eight waves).
  // One row: eight waves instead of sixteen under the same condition, two work-groups per CU (448 blocks
  // 16.7 -> 15.2 us, 787 blocks 27.8 -> 23.4 us).
  static const bool tile_forced = getenv("XMK_INT4_TILE") != nullptr;
  if (!tile_forced && M <= 16 && ca.ksplit == 1) {
    const int small = M == 1 ? 8 : 4;
    const int64_t blocks = xmk::ceil_div(a.n, 16 * ca.w) + (together ? xmk::ceil_div(b->n, 16 * cb.w) : 0);
    if (blocks > 256) ca.nw = small;
    if (b && !together && cb.ksplit == 1 && xmk::ceil_div(b->n, 16 * cb.w) > 256) cb.nw = small;
  }
  xmk::trace("int4_gemm m=%d k=%lld n=%lld group=%d words_per_lane=%d waves=%d ksplit=%d%s", M, (long long)a.k,
             (long long)a.n, (int)group, ca.w, ca.nw, ca.ksplit, together ? " (+ a second product in the same launch)" : "");
  for (int m_base = 0; m_base < M; m_base += 32) {
    if ((rc = launch_cfg(ca, spg, a, together ? b : nullptr, m_base, M, st)) != XMK_OK) return rc;
    if (b && !together && (rc = launch_cfg(cb, spg, *b, nullptr, m_base, M, st)) != XMK_OK) return rc;
  }
  return xmk::check_launch("int4_gemm");
}

int xmk::int4_gemm_launch(const void* act, const void* qweight, const void* scales,
                          const void* zeros, const void* bias, void* out, int64_t m, int64_t k,
                          int64_t n, int64_t group, const Int4Epilogue& ep, hipStream_t st,
                          const Int4SplitK& split) {
  Int4Call c;
  c.act = act; c.qweight = qweight; c.scales = scales; c.zeros = zeros; c.bias = bias; c.out = out;
  c.k = k; c.n = n; c.ep = ep; c.split = split;
  return int4_gemm_launch2(c, nullptr, m, group, st);
}

extern "C" int xmk_int4_gemm(const void* act, const void* qweight, const void* scales,
                             const void* zeros, const void* bias, void* out, int64_t m, int64_t k,
                             int64_t n, int64_t group, void* stream) {
  return xmk::int4_gemm_launch(act, qweight, scales, zeros, bias, out, m, k, n, group,
                               xmk::Int4Epilogue{}, (hipStream_t)stream);
}

// From this many rows on, writing the fp16 weight matrix out once and running the dense fp16 GEMM on it is
// faster than streaming the packed weights once per 32 rows (measured at 128 rows: 54 against 68 us for
// k 4096, n 16384; 82 against 131 us for k 16384, n 4096; at 96 rows the first shape is a tie).
constexpr int64_t kInt4DenseRows = 96;

extern "C" size_t xmk_int4_gemm_workspace_bytes(int64_t m, int64_t k, int64_t n) {
  if (m < kInt4DenseRows || k <= 0 || n <= 0 || k > (1 << 24) || n > (1 << 24)) return 0;
  return (size_t)k * (size_t)n * sizeof(_Float16);
}

extern "C" int xmk_int4_gemm_ws(const void* act, const void* qweight, const void* scales, const void* zeros,
                                const void* bias, void* out, int64_t m, int64_t k, int64_t n, int64_t group,
                                void* workspace, size_t workspace_bytes, void* stream) {
  const size_t need = xmk_int4_gemm_workspace_bytes(m, k, n);
  if (need == 0 || !workspace || workspace_bytes < need || !xmk::aligned(workspace, 16) || !act || !out ||
      !xmk::aligned(act, 16) || !xmk::aligned(out, 16) || k % 8 != 0)
    return xmk_int4_gemm(act, qweight, scales, zeros, bias, out, m, k, n, group, stream);
  if (group <= 0 || group % 32 != 0 || group > 256)  // the same contract whatever the path
    return xmk::fail(XMK_UNIMPLEMENTED, "int4_gemm: group must be 32, 64, 128 or 256");
  xmk::trace("int4_gemm m=%lld k=%lld n=%lld group=%d dense: dequantise + fp16 GEMM", (long long)m, (long long)k,
             (long long)n, (int)group);
  const int rc = xmk_int4_dequant(qweight, scales, zeros, workspace, k, n, group, stream);
  if (rc != XMK_OK) return rc;
  xmk_gemm_desc d{};
  d.lhs = xmk_matrix{const_cast<void*>(act), 0, m, k, 0, k};
  d.rhs = xmk_matrix{workspace, 0, k, n, 0, n};
  d.out = xmk_matrix{out, 0, m, n, 0, n};
  d.bias = bias;
  d.dtype_in = d.dtype_out = XMK_F16;
  d.batch_size = 1;
  d.alpha = 1.0f;
  d.epilogue = bias ? XMK_EPI_BIAS : XMK_EPI_DEFAULT;
  return xmk_gemm(&d, stream);
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
