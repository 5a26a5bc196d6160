// fp32 GEMM on the matrix cores (gemm_f32.hip).
#pragma once
#include "gemm_kernel.h"

namespace gemm_impl {

// p as for the 16-bit kernel (leading dimensions and strides in elements); vec_a / vec_b >= 4 mean the
// operand's pointer is 16-byte aligned and its leading dimension, batch stride and row length are
// multiples of 4.  a_mc / b_mc: the operand's free index is contiguous ([K, M] / [K, N] storage).
void launch_gemm_f32(GemmParams& p, bool a_mc, bool b_mc, int batch, hipStream_t st);

}  // namespace gemm_impl
