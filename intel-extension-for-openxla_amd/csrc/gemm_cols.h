// The streaming kernel for a few rows against B stored [N, K] (see gemm_rows.hip for the family); included by
// the gemm_cols_*.hip units, each of which instantiates one element type so that they compile in parallel.
#pragma once
#include "gemm_rows_common.h"

namespace gemm_impl {

// out = act(alpha * A B + beta * c + bias) with B stored [N, K], for `batch` batch members; defined for
// __bf16 and _Float16.
template <typename T>
void launch_gemm_cols(const GemmParams& p, bool out_f32, int batch, hipStream_t st);

namespace {
using namespace rows_detail;

// One output element: out[m, n] = act(alpha * v + beta * c[m, n] + bias[n]).
template <typename T, bool OutF32>
__device__ __forceinline__ void store_one(const GemmParams& p, float v, int m, int n, int64_t coff) {
  const int64_t off = coff + (int64_t)m * p.ldc + n;
  v *= p.alpha;
  if (p.c) {  // non-null only when beta != 0
    if constexpr (OutF32) v += p.beta * reinterpret_cast<const float*>(p.c)[off];
    else v += p.beta * Elem<T>::to_f32(reinterpret_cast<const T*>(p.c)[off]);
  }
  if (p.bias) v += Elem<T>::to_f32(reinterpret_cast<const T*>(p.bias)[n]);
  v = apply_act(v, p.act);
  if constexpr (OutF32) reinterpret_cast<float*>(p.out)[off] = v;
  else reinterpret_cast<uint16_t*>(p.out)[off] = Elem<T>::from_f32(v);
}

constexpr int kColsRB = 64;  // output columns (rows of B) a work-group folds at a time
constexpr int kColsD = 8;    // rows of B a wave keeps in flight

// B stored [N, K].  MT as above.  KL: 1 KiB loads per row and wave; wave w owns reduction indices
// [512 KL w, 512 KL (w + 1)), lane l the eight from 512 KL w + 512 j + 8 l for j < KL (K <= 4096 KL).
template <typename T, bool OutF32, int MT, int KL>
__global__ __launch_bounds__(kNW * 64) void gemm_cols_kernel(GemmParams p) {
  __shared__ float red[kNW][MT][kColsRB];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // A work-group owns p.tiles_n consecutive output columns (the host sizes that so that all work-groups are
  // resident at once and equally long) and walks them 64 at a time.  XCD x takes the x-th eighth of the
  // (column range, batch member) list (see gemm_rows_kernel); here that also makes an XCD's work-groups
  // walk one contiguous range of memory.
  const int blocks_n = (p.N + p.tiles_n - 1) / p.tiles_n;
  const int per_xcd = (int)gridDim.x / 8;
  const int item = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
  if (item >= blocks_n * p.tiles_m) return;  // tiles_m carries the batch count; the grid is rounded up to eight
  const int z = item / blocks_n;
  const int n_lo = (item % blocks_n) * p.tiles_n, n_hi = min(p.N, n_lo + p.tiles_n);
  int nb = n_lo;  // first column of the 64 being folded
  const T* A = reinterpret_cast<const T*>(p.a) + (int64_t)z * p.sa;
  const T* B = reinterpret_cast<const T*>(p.b) + (int64_t)z * p.sb;
  const __amdgpu_buffer_rsrc_t r_a = make_rsrc(A, (uint32_t)(((int64_t)(p.M - 1) * p.lda + p.K) * 2));
  const __amdgpu_buffer_rsrc_t r_b = make_rsrc(B, (uint32_t)(((int64_t)(p.N - 1) * p.ldb + p.K) * 2));

  // This lane's pieces of A, for the whole launch, and its byte offsets inside a row of B.
  u32x4 a[MT][KL];
  uint32_t voff[KL];
#pragma unroll
  for (int j = 0; j < KL; ++j) {
    const int k = 512 * (KL * wave + j) + 8 * lane;
    voff[j] = k < p.K ? (uint32_t)k * 2 : kOob;  // K % 8 == 0: a lane's eight are all in or all out
#pragma unroll
    for (int m = 0; m < MT; ++m)
      a[m][j] = __builtin_bit_cast(
          u32x4, __builtin_amdgcn_raw_buffer_load_b128(r_a, m < p.M ? voff[j] : kOob, (uint32_t)((int64_t)m * p.lda * 2), 0));
  }

  uint32_t launder = 0;  // an operand of every product below, re-defined after each fetch (see gemm_rows_kernel)
  asm volatile("" : "+v"(launder));
  struct Row {
    u32x4 b[KL];
  };
  // Row r is output column nb + r (r >= 64: a row of the next 64).  Past the work-group's range the fetch
  // still goes out, out of range.
  auto fetch = [&](int r, Row& row) {
    const bool live = nb + r < n_hi;
    const int64_t ns = live ? nb + r : 0;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < KL; ++j)
      row.b[j] = __builtin_bit_cast(
          u32x4, __builtin_amdgcn_raw_buffer_load_b128(r_b, live ? voff[j] : kOob, (uint32_t)(ns * p.ldb * 2), 0));
    asm volatile("" : "+v"(launder) : : "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  // The 64 per-lane partial sums of a row are not added up row by row (six dependent lane exchanges per
  // value): rows are folded pairwise like a binary counter.  Merging two registers that stand for 2^v rows
  // each, the lanes with bit v clear keep the earlier rows and receive their partner's share of them, the
  // lanes with bit v set the later rows: one exchange halves the data, 63 exchanges per 64 rows and row of
  // A instead of 384, and after row 63 lane l holds the whole sum of row l.
  int bperm_addr[6];
  bool hi[6];
#pragma unroll
  for (int v = 0; v < 6; ++v) {
    bperm_addr[v] = (lane ^ (1 << v)) << 2;
    hi[v] = ((lane >> v) & 1) != 0;
  }
  float pend[7][MT];
  auto compute = [&](auto R, const Row& row) {
    constexpr int r = decltype(R)::value;
    float cur[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      cur[m] = 0.f;
#pragma unroll
      for (int j = 0; j < KL; ++j)
#pragma unroll
        for (int d = 0; d < 4; ++d) cur[m] = Dot2<T>::f(a[m][j][d], row.b[j][d] | launder, cur[m]);
    }
    static_for<6>([&](auto V) {
      constexpr int v = decltype(V)::value;
      constexpr int ones = (2 << v) - 1;
      if constexpr ((r & ones) == ones) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const float send = hi[v] ? pend[v][m] : cur[m];
          const float keep = hi[v] ? cur[m] : pend[v][m];
          cur[m] = keep + __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(bperm_addr[v], __builtin_bit_cast(int, send)));
        }
      }
    });
    constexpr int level = __builtin_ctz(~(unsigned)r);  // trailing ones of r: the levels merged above
#pragma unroll
    for (int m = 0; m < MT; ++m) pend[level][m] = cur[m];
  };

  // A ring of kColsD rows in registers, kColsD - 1 in flight while one is worked on; the 64 rows as
  // straight-line code with compile-time ring positions and fold levels, fetches never behind a branch
  // (exact wait counts).
  static_assert(kColsRB % kColsD == 0, "the ring position of a row is the same in every 64");
  Row ring[kColsD];
  static_for<kColsD - 1>([&](auto i) { fetch(i, ring[i]); });
  do {  // (one exit, at the end: both edges into the loop carry the same kColsD - 1 rows in flight)
    static_for<kColsRB>([&](auto r) {
      fetch(r + kColsD - 1, ring[(r + kColsD - 1) % kColsD]);
      compute(r, ring[r % kColsD]);
    });
#pragma unroll
    for (int m = 0; m < MT; ++m) red[wave][m][lane] = pend[6][m];
    __syncthreads();
    // thread t: row m = t / 64 of A, column nb + t % 64
    for (int t = threadIdx.x; t < MT * kColsRB; t += kNW * 64) {
      const int m = t / kColsRB, r = t % kColsRB;
      if (m >= p.M || nb + r >= n_hi) continue;
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < kNW; ++w) v += red[w][m][r];
      store_one<T, OutF32>(p, v, m, nb + r, (int64_t)z * p.sc);
    }
    __syncthreads();  // red is written again at the end of the next 64
    nb += kColsRB;
  } while (nb < n_hi);
}

// Work-groups of `kernel` (512 threads) that fit one CU at a time.
template <typename K>
int resident_per_cu(K kernel) {
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, kNW * 64, 0) != hipSuccess || n < 1) n = 1;
  return n;
}

template <typename T, bool OutF32, int MT, int KL>
void launch_cols_mt(GemmParams p, int batch, hipStream_t st) {
  // Columns per work-group: 64 while that many work-groups are resident at once (no second round with a
  // part-filled device: 788 blocks of 64 on 512 places ran 50400 columns at 5.2 TB/s), else equal shares.
  static const int places = resident_per_cu(gemm_cols_kernel<T, OutF32, MT, KL>) * 256;
  const int64_t per_member = places / batch > 0 ? places / batch : 1;
  p.tiles_m = batch;
  p.tiles_n = xmk::ceil_div(p.N, kColsRB) <= per_member ? kColsRB : (int)xmk::ceil_div(p.N, per_member);
  const int64_t items = xmk::ceil_div(p.N, p.tiles_n) * batch;
  hipLaunchKernelGGL((gemm_cols_kernel<T, OutF32, MT, KL>), dim3((unsigned)(xmk::ceil_div(items, 8) * 8)), dim3(kNW * 64), 0,
                     st, p);
}

template <typename T, bool OutF32, int KL>
void launch_cols_kl(const GemmParams& p, int batch, hipStream_t st) {
  if (p.M <= 1) launch_cols_mt<T, OutF32, 1, KL>(p, batch, st);
  else if (p.M <= 2) launch_cols_mt<T, OutF32, 2, KL>(p, batch, st);
  else if (p.M <= 4) launch_cols_mt<T, OutF32, 4, KL>(p, batch, st);
  else if constexpr (KL <= 2) launch_cols_mt<T, OutF32, 8, KL>(p, batch, st);
  // (eight rows with four loads per row do not fit the register file: gemm_rows_applicable refuses them)
}

template <typename T, bool OutF32>
void launch_cols(const GemmParams& p, int batch, hipStream_t st) {
  if (p.K <= 4096) launch_cols_kl<T, OutF32, 1>(p, batch, st);
  else if (p.K <= 8192) launch_cols_kl<T, OutF32, 2>(p, batch, st);
  else launch_cols_kl<T, OutF32, 4>(p, batch, st);
}

}  // namespace
}  // namespace gemm_impl
