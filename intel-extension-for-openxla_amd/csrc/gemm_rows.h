// 16-bit GEMM for a handful of rows (decode): the streaming kernel of gemm_rows.hip.
#pragma once
#include "gemm_kernel.h"

namespace gemm_impl {

// Lanes per reduction row (8, 16, 32 or 64; the work-group owns eight columns per lane) that the kernel
// uses for n columns and `batch` batch members.
int gemm_rows_lanes_per_row(int64_t n, int64_t batch);

// Which streaming kernel can run the product p describes (A [M, K] row-major with the 16-byte alignment the
// direct kernels need, at most kRowsMaxM rows, operands short enough for 31-bit byte offsets):
// kRowsMC for B stored [K, N], kRowsKC for B stored [N, K] with K <= kColsMaxK, kRowsNone otherwise.
int gemm_rows_applicable(const GemmParams& p, bool a_mc, bool b_mc);

// out = act(alpha * A B + beta * c + bias) (or fp32 partial sums: whatever p says) for `batch` batch
// members with p's batch strides; b_mc: B stored [K, N].
void launch_gemm_rows(const GemmParams& p, bool b_mc, bool is_bf16, bool out_f32, int batch, hipStream_t st);

}  // namespace gemm_impl
