// Instantiates the gathering MFMA GEMM for one (element type, output type) pair; see gemm_kernel.h.
#include "gemm_kernel.h"

namespace gemm_impl {
template <>
void launch_layout_gather<_Float16, false>(bool a_mc, bool b_mc, GemmParams& p, int batch, hipStream_t st) {
  launch_layout_gather_impl<_Float16, false>(a_mc, b_mc, p, batch, st);
}
}  // namespace gemm_impl
