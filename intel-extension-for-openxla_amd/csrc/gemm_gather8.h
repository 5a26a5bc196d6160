// Gathering loader for 8-bit operands (int8, fp8), shared by gemm_s8.hip and fp8_gemm.hip: the LDS
// tile is [row][64 bytes] with XOR-swizzled 16-byte chunks whatever the operand's storage.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace gather8 {

typedef int intx4 __attribute__((ext_vector_type(4)));

constexpr int BKB = 64;  // k per K step = bytes of one LDS row
// How an operand is fetched: k-contiguous with one aligned 16-byte load per chunk, k-contiguous byte by
// byte, or from [K][rows] storage (16 rows of k apart).
enum : int { KC_VEC = 0, KC_SCALAR = 1, MC = 2 };

__device__ __forceinline__ int swz4(int row) { return (row >> 2) & 3; }

// Chunk i of this thread for one operand: LDS bytes [i * 4096 + tid * 16, +16) = row i * 64 + tid / 4,
// position tid % 4, which holds logical chunk (tid % 4) ^ swz4(row) = k 16 c .. 16 c + 15 of the K step.
// Branch-free: lanes outside the matrix load from `safe` (the operand's first element) and select zero.
template <int MODE>
__device__ __forceinline__ intx4 gather(const int8_t* base, const int8_t* safe, int64_t ld, int valid, int kleft, int i,
                                        int tid) {
  const int row = i * 64 + (tid >> 2);
  const int k = ((tid & 3) ^ swz4(row)) * 16;
  const bool in = row < valid;
  intx4 v;
  if constexpr (MODE == KC_VEC) {  // K % 16 == 0: the chunk is inside the row or outside as a whole
    const bool ok = in && k < kleft;
    v = *reinterpret_cast<const intx4*>(ok ? base + (int64_t)row * ld + k : safe);
    if (!ok) v = intx4{0, 0, 0, 0};
  } else {
    const int8_t* src = MODE == KC_SCALAR ? base + (int64_t)row * ld + k : base + (int64_t)k * ld + row;
    const int64_t step = MODE == KC_SCALAR ? 1 : ld;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      uint32_t word = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int j = 4 * w + b;
        const bool ok = in && k + j < kleft;
        const uint32_t x = (uint8_t) * (ok ? src + j * step : safe);
        word |= (ok ? x : 0u) << (8 * b);
      }
      v[w] = (int)word;
    }
  }
  return v;
}

}  // namespace gather8
