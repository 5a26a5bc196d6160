// Host entry point of the fused multi-head attention forward and the head-size classes up to 128.
// This translation unit is compiled with the matrix instructions in their VGPR form
// (-mllvm -amdgpu-mfma-vgpr-form, set per file in build.py): the S accumulators are then read by the
// softmax's vector instructions where the matrix cores wrote them, with no copies between register
// files.  The class for head sizes above 128 needs both halves of the register file and lives in
// fmha_fwd_h256.hip.
#include "fmha_fwd_kernel.h"

namespace fmha_fwd_impl {
namespace {

template <typename T>
void launch_t(const FmhaParams& p, int32_t dtype, uint64_t units, uint32_t F, bool causal, int bias, hipStream_t st) {
  // Head-size classes of the reference's policy choice (fmha_forward.h:622-646).  Four waves of 32
  // query rows, two work-groups per CU.  Measured against it on [8,32,2048,128] with the current step:
  // eight waves per work-group (half the K / V loads per row) 1020 against 1032 TFLOP/s; a second
  // 32-row tile per wave (one wave per SIMD, O in AGPRs, every K / V fragment feeding two matrix
  // instructions) 1007 against 1033 without a mask and 789 against 872 with one, at a higher clock and
  // the same board power and energy per launch: the package power limit, not the schedule, sets the rate.
  if (p.H <= 64) launch_cfg<T, 64, 4, 2>(p, units, F, causal, bias, st);
  else if (p.H <= 128) launch_cfg<T, 128, 4, 2>(p, units, F, causal, bias, st);
  else launch_h256(p, dtype, units, F, causal, bias, st);
}

}  // namespace
}  // namespace fmha_fwd_impl

using namespace fmha_fwd_impl;

extern "C" int xmk_fmha_fwd(const void* query, const void* key, const void* value, const void* bias,
                            void* out, float* lse, int32_t dtype, uint32_t num_batches,
                            uint32_t num_heads, uint32_t head_size, uint32_t num_queries,
                            uint32_t num_keys, float head_scale, int32_t causal, void* stream) {
  if (!query || !key || !value || !out) return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: null pointer");
  if (dtype != XMK_F16 && dtype != XMK_BF16)
    return xmk::fail(XMK_INTERNAL, "Invalid MHA datatype");  // xetla_gpu_fused_mha_runner.cc:145
  if (num_batches == 0 || num_heads == 0 || head_size == 0 || num_queries == 0 || num_keys == 0)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: empty dimension");
  if (head_size > 256)
    return xmk::fail(XMK_UNIMPLEMENTED, "fmha_fwd: head_size %u > 256 (fmha_forward.h:642)", head_size);
  if (head_size % 8 != 0)
    return xmk::fail(XMK_UNIMPLEMENTED, "fmha_fwd: head_size %u is not a multiple of 8", head_size);
  if (!(head_scale > 0.0f) || head_scale > 3.0e38f)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: head_scale must be positive and finite");
  const uint64_t units = (uint64_t)num_batches * num_heads;
  if (units * ((num_queries + 31) / 32) > 0x7fffffffull || (uint64_t)num_keys * head_size * 2 >= kOob ||
      (uint64_t)num_queries * head_size * 2 >= kOob)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: shape too large");
  if (!xmk::aligned(query, 16) || !xmk::aligned(key, 16) || !xmk::aligned(value, 16) ||
      !xmk::aligned(out, 16))
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: tensors must be 16-byte aligned");
  FmhaParams p;
  p.q = query; p.k = key; p.v = value; p.bias = bias; p.out = out; p.lse = lse;
  p.H = (int)head_size; p.F = (int)num_queries; p.T = (int)num_keys;
  p.nqb = p.total = p.per_xcd = 0;
  p.scale2 = head_scale * kLog2e;
  xmk::trace("fmha_fwd B=%u N=%u F=%u T=%u H=%u causal=%d bias=%d lse=%d", num_batches, num_heads,
             num_queries, num_keys, head_size, causal, bias != nullptr, lse != nullptr);
  hipStream_t st = (hipStream_t)stream;
  // The staged bias path needs whole 16-byte chunks per row and offsets inside one query block
  // that fit the 31-bit buffer offset.
  const int bias_mode = !bias ? 0
                        : (num_keys % 8 == 0 && xmk::aligned(bias, 16) && (uint64_t)num_keys * 2 * 128 < kOob) ? 2
                                                                                                            : 1;
  if (dtype == XMK_BF16) launch_t<__bf16>(p, dtype, units, num_queries, causal != 0, bias_mode, st);
  else launch_t<_Float16>(p, dtype, units, num_queries, causal != 0, bias_mode, st);
  return xmk::check_launch("fmha_fwd");
}
