// Instantiates the [N, K] streaming kernel for one element type; see gemm_cols.h.
#include "gemm_cols.h"

namespace gemm_impl {
template <>
void launch_gemm_cols<__bf16>(const GemmParams& p, bool out_f32, int batch, hipStream_t st) {
  if (out_f32) launch_cols<__bf16, true>(p, batch, st);
  else launch_cols<__bf16, false>(p, batch, st);
}
}  // namespace gemm_impl
