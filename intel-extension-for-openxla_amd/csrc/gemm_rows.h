// 16-bit GEMM for a handful of rows (decode): the streaming kernel of gemm_rows.hip.
#pragma once
#include "gemm_kernel.h"

namespace gemm_impl {

// Lanes per reduction row (8, 16, 32 or 64; the work-group owns eight columns per lane) that the kernel
// uses for n columns and `batch` batch members.
int gemm_rows_lanes_per_row(int64_t n, int64_t batch);

// True when the streaming kernel can run the product p describes: A [M, K] row-major, B stored
// [K, N] (both with the 16-byte alignment the direct kernels need), at most kRowsMaxM rows, and
// operands short enough for 31-bit byte offsets.
bool gemm_rows_applicable(const GemmParams& p, bool a_mc, bool b_mc);

// out = act(alpha * A B + beta * c + bias) (or fp32 partial sums: whatever p says) for `batch` batch
// members with p's batch strides.
void launch_gemm_rows(const GemmParams& p, bool is_bf16, bool out_f32, int batch, hipStream_t st);

}  // namespace gemm_impl
