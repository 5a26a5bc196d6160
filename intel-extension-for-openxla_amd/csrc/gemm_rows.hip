// 16-bit GEMM for one to eight rows against a [K, N] row-major matrix: the decode shapes that fill the
// reference's tile table (xla/service/gpu/xetla/gemm/gemm.cc:33-47,77-80,92-93: m in {1, 4} against
// n = 4096 ... 50400).  The product is bound by reading B once, so B is not staged anywhere: a lane
// owns eight consecutive output columns and loads 16 bytes of each reduction row straight into
// registers (a wave reads 1 KiB of a row per instruction), the eight waves of a work-group take the
// rows in turns of eight and meet in LDS at the end.  Arithmetic on the vector ALU: two rows of B are
// interleaved into (k, k+1) pairs per column with v_perm and multiplied with the matching pair of A,
// which lies that way in memory, by one v_dot2 per row of A (fp32 accumulation): 0.5 + M/2
// instructions per element of B, far below what the stream leaves time for up to eight rows.
// The matrix-core kernel pays LDS traffic and 16 or 32 MFMA rows for these shapes; here nothing but
// the loads and M/2 instructions per element draw power.
//
// B stored [N, K] (reduction index contiguous) has its own kernel, gemm_cols_kernel: an output column is
// one contiguous row of B, a work-group walks 64 of them one after the other, its eight waves each
// holding one eighth of the reduction range (a wave's load is 1 KiB of the row, the work-group's eight
// loads the next 8 KiB of memory), with the matching pieces of A in registers for the whole launch.
// Products need no pairing (both operands hold (k, k+1) pairs); the per-lane partial sums of 64 rows are
// added across the wave by pairwise folding (one lane exchange per row), across the waves in LDS once per
// 64 columns.
#include "gemm_rows.h"

#include "gemm_rows_common.h"

namespace gemm_impl {

// (defined in gemm_cols_bf16.hip / gemm_cols_f16.hip)
template <typename T>
void launch_gemm_cols(const GemmParams& p, bool out_f32, int batch, hipStream_t st);
template <>
void launch_gemm_cols<__bf16>(const GemmParams& p, bool out_f32, int batch, hipStream_t st);
template <>
void launch_gemm_cols<_Float16>(const GemmParams& p, bool out_f32, int batch, hipStream_t st);

namespace {
using namespace rows_detail;

// MT: rows of A the kernel carries (M <= MT; rows beyond M are read as zeros and not stored).
// LR: lanes per reduction row.  A work-group owns 8 LR output columns; the 64 / LR lane groups of a wave
//     take different blocks of eight reduction rows (a load instruction then covers 64 / LR rows, 16 LR
//     bytes of each) and are added up with lane exchanges before the waves meet in LDS.  Narrow blocks
//     make enough work-groups out of a narrow matrix without a second launch for a K split.
template <typename T, bool OutF32, int MT, int LR>
__global__ __launch_bounds__(kNW * 64) void gemm_rows_kernel(GemmParams p) {
  constexpr int G = 64 / LR;        // lane groups = blocks of eight rows per wave and batch
  constexpr int BN = LR * 8;        // columns per work-group
  __shared__ float red[kNW / 2][MT * 8][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lc = lane % LR, g = lane / LR;
  // Work-groups go to the eight XCDs in turn; XCD x takes the x-th eighth of the (column block, batch
  // member) list, so that its L2 sees neighbouring column blocks.  (With the plain order and a
  // power-of-two row length, the blocks of one XCD are a fixed distance apart in every row and use a
  // quarter of its L2 channels: 16384 columns streamed at 3.7 TB/s where 50400 reached 5.6.)
  const int blocks_n = (p.N + BN - 1) / BN;
  const int per_xcd = (int)gridDim.x / 8;
  const int item = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
  if (item >= blocks_n * p.tiles_m) return;  // tiles_m carries the batch count; the grid is rounded up to eight
  const int z = item / blocks_n;
  const int n0 = (item % blocks_n) * BN + lc * 8;
  const T* A = reinterpret_cast<const T*>(p.a) + (int64_t)z * p.sa;
  const T* B = reinterpret_cast<const T*>(p.b) + (int64_t)z * p.sb;
  // Hardware bounds checking zero-fills a lane whose offset is kOob; every offset in range stays
  // below 2^31 (the host checks the operand sizes).
  const __amdgpu_buffer_rsrc_t r_a = make_rsrc(A, (uint32_t)(((int64_t)(p.M - 1) * p.lda + p.K) * 2));
  const __amdgpu_buffer_rsrc_t r_b = make_rsrc(B, (uint32_t)(((int64_t)(p.K - 1) * p.ldb + p.N) * 2));
  // per lane: its block of eight rows inside a batch, its columns (N % 8 == 0: all in or all out)
  const uint32_t voff_b = n0 < p.N ? (uint32_t)(((int64_t)(8 * g) * p.ldb + n0) * 2) : kOob;
  const uint32_t voff_a = (uint32_t)(8 * g) * 2;

  float acc[MT][8];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[m][c] = 0.f;

  uint32_t sel_lo = 0x05040100u, sel_hi = 0x07060302u;  // (low halves), (high halves) of two registers
  asm volatile("" : "+v"(sel_lo), "+v"(sel_hi));

  struct Chunk {
    u32x4 a[MT];      // A[m, k .. k+7], k = 8 (G q + g)
    u32x4 b[kChunk];  // B[k + j, n0 .. n0+7]
  };
  // Batch q of a wave is reduction rows 8 G q .. 8 G (q + 1) - 1.  A fetch past the end still goes out,
  // out of range (no memory access, zeros back): the sequence of loads is then the same on every path, and
  // the counted wait before a batch's arithmetic leaves the next batch's loads in flight.
  const int batches = (p.K + 8 * G - 1) / (8 * G);
  auto fetch = [&](int q, Chunk& c) {
    const bool live = 8 * (G * q + g) < p.K;  // K % 8 == 0: a lane's eight rows are all in or all out
    const uint32_t vb = live ? voff_b : kOob;
    // (a batch wholly past the end uses batch 0's scalar offsets, so that kOob plus the scalar offset cannot
    //  wrap around 32 bits whatever the unit that checks the range adds up)
    const int64_t qs = 8 * G * q < p.K ? q : 0;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < MT; ++m)
      c.a[m] = __builtin_bit_cast(
          u32x4, __builtin_amdgcn_raw_buffer_load_b128(r_a, (live && m < p.M) ? voff_a : kOob,
                                                       (uint32_t)(((int64_t)m * p.lda + qs * 8 * G) * 2), 0));
#pragma unroll
    for (int j = 0; j < kChunk; ++j)
      c.b[j] = __builtin_bit_cast(
          u32x4, __builtin_amdgcn_raw_buffer_load_b128(r_b, vb, (uint32_t)((qs * 8 * G + j) * p.ldb * 2), 0));
    // Every pairing below reads these selectors, so the arithmetic that follows in program order is also
    // emitted after these loads (instruction selection is free to order what has no side effects).
    asm volatile("" : "+v"(sel_lo), "+v"(sel_hi) : : "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  auto compute = [&](const Chunk& c) {
#pragma unroll
    for (int jp = 0; jp < kChunk / 2; ++jp) {
      uint32_t pr[8];  // column c: (B[k + 2jp, n0 + c], B[k + 2jp + 1, n0 + c])
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        pr[2 * d] = __builtin_amdgcn_perm(c.b[2 * jp + 1][d], c.b[2 * jp][d], sel_lo);
        pr[2 * d + 1] = __builtin_amdgcn_perm(c.b[2 * jp + 1][d], c.b[2 * jp][d], sel_hi);
      }
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int col = 0; col < 8; ++col) acc[m][col] = Dot2<T>::f(c.a[m][jp], pr[col], acc[m][col]);
    }
  };

  // Wave w takes batches w, w + kNW, ...; two per turn of a loop whose only exit is at its end, so that both
  // edges into the loop carry the same outstanding loads (an odd count ends on a batch of zeros).
  const int mine = wave < batches ? (batches - wave + kNW - 1) / kNW : 0;
  Chunk buf_a, buf_b;
  int q = wave;
  fetch(q, buf_a);
  for (int pair = 0; pair < (mine + 1) / 2; ++pair) {
    fetch(q + kNW, buf_b);
    compute(buf_a);
    fetch(q + 2 * kNW, buf_a);
    compute(buf_b);
    q += 2 * kNW;
  }

  // Sum over the lane groups of a wave (every lane ends up with the total of its columns) ...
#pragma unroll
  for (int o = LR; o < 64; o <<= 1)
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int c = 0; c < 8; ++c) acc[m][c] += __shfl_xor(acc[m][c], o);
  // ... and over the waves: upper half into LDS, lower half adds, three times (a fixed order).
#pragma unroll
  for (int half = kNW / 2; half >= 1; half >>= 1) {
    if (wave >= half && wave < 2 * half) {
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int c = 0; c < 8; ++c) red[wave - half][m * 8 + c][lane] = acc[m][c];
    }
    __syncthreads();
    if (wave < half) {
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[m][c] += red[wave][m * 8 + c][lane];
    }
    __syncthreads();
  }
  if (wave != 0 || g != 0) return;
  const int64_t coff = (int64_t)z * p.sc;
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    store_quad<T, OutF32>(p, floatx4{acc[m][0], acc[m][1], acc[m][2], acc[m][3]}, m, n0, coff);
    store_quad<T, OutF32>(p, floatx4{acc[m][4], acc[m][5], acc[m][6], acc[m][7]}, m, n0 + 4, coff);
  }
}

template <typename T, bool OutF32, int LR>
void launch_rows_lr(const GemmParams& p0, int batch, hipStream_t st) {
  GemmParams p = p0;
  p.tiles_m = batch;
  const int64_t items = xmk::ceil_div(p.N, LR * 8) * batch;
  const dim3 grid((unsigned)(xmk::ceil_div(items, 8) * 8)), block(kNW * 64);
  if (p.M <= 1) hipLaunchKernelGGL((gemm_rows_kernel<T, OutF32, 1, LR>), grid, block, 0, st, p);
  else if (p.M <= 2) hipLaunchKernelGGL((gemm_rows_kernel<T, OutF32, 2, LR>), grid, block, 0, st, p);
  else if (p.M <= 4) hipLaunchKernelGGL((gemm_rows_kernel<T, OutF32, 4, LR>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((gemm_rows_kernel<T, OutF32, 8, LR>), grid, block, 0, st, p);
}

template <typename T, bool OutF32>
void launch_rows(const GemmParams& p, int batch, hipStream_t st) {
  switch (gemm_rows_lanes_per_row(p.N, batch)) {
    case 64: launch_rows_lr<T, OutF32, 64>(p, batch, st); break;
    case 32: launch_rows_lr<T, OutF32, 32>(p, batch, st); break;
    case 16: launch_rows_lr<T, OutF32, 16>(p, batch, st); break;
    default: launch_rows_lr<T, OutF32, 8>(p, batch, st); break;
  }
}

}  // namespace

int gemm_rows_lanes_per_row(int64_t n, int64_t batch) {
  // XMK_GEMM_ROWS_LANES=<8|16|32|64> overrides the choice (tuning aid, read at every call).
  if (const char* e = getenv("XMK_GEMM_ROWS_LANES")) {
    const int v = atoi(e);
    if (v == 8 || v == 16 || v == 32 || v == 64) return v;
  }
  // the widest column block that still makes about a work-group per CU and more
  for (int lr = 64; lr > 8; lr /= 2)
    if (xmk::ceil_div(n, (int64_t)lr * 8) * batch >= kRowsEnoughBlocks) return lr;
  return 8;
}

int gemm_rows_applicable(const GemmParams& p, bool a_mc, bool b_mc) {
  if (a_mc || p.M < 1 || p.M > kRowsMaxM || p.K % kChunk != 0) return kRowsNone;
  if (p.out_alt[0] || p.out_alt[1]) return kRowsNone;
  constexpr int64_t kLimit = int64_t{1} << 31;  // byte offsets below kOob
  if (((int64_t)(p.M - 1) * p.lda + p.K + 64) * 2 >= kLimit) return kRowsNone;
  if (b_mc) {
    // (a wave's batch is up to 64 rows, the last of which may lie past K)
    return (p.N % 8 == 0 && ((int64_t)(p.K + 63) * p.ldb + p.N) * 2 < kLimit) ? kRowsMC : kRowsNone;
  }
  // its pieces of A stay in registers: 4 per row of A and 4096 of K
  const int max_k = p.M > 4 ? kColsMaxK / 2 : kColsMaxK;
  return (p.K <= max_k && ((int64_t)(p.N - 1) * p.ldb + p.K) * 2 < kLimit) ? kRowsKC : kRowsNone;
}

void launch_gemm_rows(const GemmParams& p, bool b_mc, bool is_bf16, bool out_f32, int batch, hipStream_t st) {
  if (b_mc) {
    if (is_bf16) {
      if (out_f32) launch_rows<__bf16, true>(p, batch, st);
      else launch_rows<__bf16, false>(p, batch, st);
    } else {
      if (out_f32) launch_rows<_Float16, true>(p, batch, st);
      else launch_rows<_Float16, false>(p, batch, st);
    }
    return;
  }
  if (is_bf16) launch_gemm_cols<__bf16>(p, out_f32, batch, st);
  else launch_gemm_cols<_Float16>(p, out_f32, batch, st);
}

}  // namespace gemm_impl
