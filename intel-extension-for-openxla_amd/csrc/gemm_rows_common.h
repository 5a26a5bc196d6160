// Pieces shared by the streaming GEMM kernels for a few rows (gemm_rows.hip, gemm_cols.h).
#pragma once
#include "gemm_kernel.h"

namespace gemm_impl {
namespace rows_detail {

constexpr int kNW = 8;     // waves per work-group
constexpr int kChunk = 8;  // reduction rows per load batch (one 16-byte piece of every row of A)

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

template <typename T> struct Dot2;
template <> struct Dot2<__bf16> {
  static __device__ __forceinline__ float f(uint32_t a, uint32_t b, float acc) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), acc, false);
  }
};
template <> struct Dot2<_Float16> {
  static __device__ __forceinline__ float f(uint32_t a, uint32_t b, float acc) {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), acc, false);
  }
};

}  // namespace rows_detail
}  // namespace gemm_impl
