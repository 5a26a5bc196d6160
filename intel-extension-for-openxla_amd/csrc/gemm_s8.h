// s8 x s8 -> s32 GEMM on the matrix cores (gemm_s8.hip).
#pragma once
#include "gemm_kernel.h"

namespace gemm_impl {

// p as for the 16-bit kernel (leading dimensions and strides in elements; alpha, beta, c, bias, act are
// not used); vec_a / vec_b >= 16 mean the operand's pointer is 16-byte aligned and its leading dimension,
// batch stride and row length are multiples of 16.  The output pointer must be 16-byte aligned.
void launch_gemm_s8(GemmParams& p, bool a_mc, bool b_mc, int batch, hipStream_t st);

}  // namespace gemm_impl
