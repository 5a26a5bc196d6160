// Internal interface of the int4 weight-only GEMM: the public entry point plus the fused
// epilogue the decode step uses.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace xmk {

// out = fp16( gelu?(acc + bias) + add0 + add1 );  add0 / add1: optional fp16 [M, N] addends.
struct Int4Epilogue {
  int gelu = 0;
  const void* add0 = nullptr;
  const void* add1 = nullptr;
  // rope_d > 0: the product is a stacked q/k/v projection [rows, 3 * rope_d] of one decode step
  // (rope_d = heads * head_dim).  Instead of being stored to `out`, q and k get the GPT-J rotary
  // embedding (interleaved pairs of the first rotary_dim elements of each head, angle = position *
  // 10000^(-2i/rotary_dim)); q goes to q_out [rows, rope_d], k and v to row `position` of the caches
  // [rows, heads, capacity, head_dim].
  int rope_d = 0;
  int head_dim = 0, rotary_dim = 0, capacity = 0, position = 0;
  void* q_out = nullptr;
  void* k_cache = nullptr;
  void* v_cache = nullptr;
};

// Splitting K over work-groups, for shapes whose N alone gives too few of them.  With
// ksplit > 1 the launch writes fp32 partial sums [ksplit][32 rows][n] to `partial` and nothing
// else: no bias, no epilogue, `out` untouched.  The consumer adds the slices in index order.
struct Int4SplitK {
  int ksplit = 1;
  float* partial = nullptr;
  size_t partial_bytes = 0;
};
constexpr int kInt4MaxSplit = 8;
// Number of K slices worth using for this shape (1: do not split).
int int4_plan_split(int64_t m, int64_t k, int64_t n, int64_t group);

// One product out = epilogue(act [m, k] x dequant(qweight) [k, n] + bias), or its K-split partial sums.
struct Int4Call {
  const void* act = nullptr;
  const void* qweight = nullptr;
  const void* scales = nullptr;
  const void* zeros = nullptr;
  const void* bias = nullptr;
  void* out = nullptr;
  int64_t k = 0, n = 0;
  Int4Epilogue ep;
  Int4SplitK split;
};
// Launches `a` and, if non-null, the independent product `b` (same m and group size): in one
// grid when both take the same tile shape, else one after the other.
int int4_gemm_launch2(const Int4Call& a, const Int4Call* b, int64_t m, int64_t group, hipStream_t st);

int int4_gemm_launch(const void* act, const void* qweight, const void* scales, const void* zeros,
                     const void* bias, void* out, int64_t m, int64_t k, int64_t n, int64_t group,
                     const Int4Epilogue& ep, hipStream_t st, const Int4SplitK& split = Int4SplitK{});

}  // namespace xmk
