/*
 * xmk_probe.h — measurement aid: what the matrix cores of the whole device sustain.
 *
 * No counterpart in the reference: it has no such probe.  The benchmark uses it to report, next to a
 * kernel's fraction of the published MFMA peak, the rate a loop of nothing but MFMA instructions
 * reaches on the same device under its power limit.
 */
#ifndef XMK_PROBE_H_
#define XMK_PROBE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Runs 1024 work-groups of 4 waves; every wave issues `iters` rounds of independent MFMA
 * instructions on pseudo-random operands held in registers:
 *   tile = 32: 16 x v_mfma_f32_32x32x16_{bf16,f16}  (XMK_F8E4M3FN: v_mfma_scale_f32_32x32x64_f8f6f4) per round
 *   tile = 16: 64 x v_mfma_f32_16x16x32_{bf16,f16}  (XMK_F8E4M3FN: v_mfma_scale_f32_16x16x128_f8f6f4) per round
 * dtype: XMK_BF16, XMK_F16 or XMK_F8E4M3FN.  sink: device buffer of at least 1 MiB that receives one float per
 * lane (so that the work is observable).  Returns 0 or an xmk_status code. */
int xmk_probe_mfma_rate(int32_t dtype, int32_t tile, int32_t iters, void* sink, uint64_t sink_bytes,
                        void* stream);

/* Floating-point operations one call of xmk_probe_mfma_rate(dtype, tile, iters, …) performs. */
double xmk_probe_mfma_flops(int32_t dtype, int32_t tile, int32_t iters);

#ifdef __cplusplus
}
#endif
#endif /* XMK_PROBE_H_ */
