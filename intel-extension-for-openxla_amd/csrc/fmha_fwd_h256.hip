// Fused multi-head attention forward, head sizes above 128 (up to 256): one wave per SIMD with
// the O accumulators in the AGPR half of the register file.
#define XMK_FMHA_AGPR 1
#include "fmha_fwd_kernel.h"

namespace fmha_fwd_impl {

void launch_h256(const FmhaParams& p, int32_t dtype, uint64_t units, uint32_t F, bool causal, int bias,
                 hipStream_t st) {
  if (dtype == XMK_BF16) launch_cfg<__bf16, 256, 4, 1>(p, units, F, causal, bias, st);
  else launch_cfg<_Float16, 256, 4, 1>(p, units, F, causal, bias, st);
}

}  // namespace fmha_fwd_impl
