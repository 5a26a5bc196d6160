/*
 * xmk_ffi.h — XLA typed-FFI handlers for the custom-call targets of the hot path.
 *
 * Each function is an XLA_FFI_Handler: it decodes one call frame (operands, results, attribute
 * dictionary, stream from the execution context) exactly as the reference's handlers do and
 * calls the kernel-level entry point of xmk.h.  Registering them under the reference's target
 * names lets an XLA host dispatch the same lowered HLO unchanged.
 */
#ifndef XMK_FFI_H_
#define XMK_FFI_H_

#ifdef XMK_HAVE_XLA_FFI_H
#include "xla/ffi/api/c_api.h"
#else
#include "xla_ffi_min.h"
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* "__cublas$gemm": replaces SyclGemm (xla/service/gpu/sycl_custom_call.cc:154-166).
 * operands (lhs, rhs) -> results (out, ...); epilogue DEFAULT; attributes as read by RunGemm
 * (xla/service/gpu/onednn_matmul_utils.cc:533-621): {lhs,rhs,output}_order i32,
 * {lhs,rhs,output}_{num_rows,num_cols,batch_stride,leading_dim_stride} i64, batch_size i64,
 * alpha f32, beta f32, algorithm i64, {lhs,rhs,output}_layout_dtype i32. */
XLA_FFI_Error* xmk_ffi_cublas_gemm(XLA_FFI_CallFrame* call_frame);

/* "__cublas$lt$matmul": replaces SyclLtMatmul (sycl_custom_call.cc:168-205).  Adds the
 * attribute epilogue i32 (xla::gpu::GemmBackendConfig::Epilogue numbering).  beta != 0: the
 * matrix addend is operand 2 and aliases the result, computed in place (:181,191-195); a vector
 * bias is operand 3 if there is a matrix addend, else operand 2 (:198); with an auxiliary
 * output the result is results[1] (:186,194), which this library rejects like the reference
 * (onednn_matmul_utils.cc:321-322). */
XLA_FFI_Error* xmk_ffi_cublas_lt_matmul(XLA_FFI_CallFrame* call_frame);

/* "__cudnn$fmhaSoftmax" / "__cudnn$fmhaScaleBiasSoftmax": replace RunXetlaGpuFMHA
 * (xla/service/gpu/xetla_gpu_fused_mha_runner.cc:45-221).  operands (Q [B,N,F,H] or [N,F,H],
 * K [.., T, H], V [.., T, H] [, bias [B,N,F,T]]) -> results (out [.., F, H], scratch
 * [, activation f32 [B,N,F]]).  Attributes (all optional): fmha_scale f64|f32 (default 1),
 * dropout_rate f64|f32 (must be 0, :57-61), is_causal_mask pred|i32 (default 0).  A scale above
 * 1 is replaced by 1/sqrt(H) as the reference does (:129).  Rank 3 (one batch, the batch dimension
 * left out) is accepted beside the rank 4 the reference's runner CHECKs for (:114-116), in the
 * forward and the backward handlers alike; every operand's element count must match the shape. */
XLA_FFI_Error* xmk_ffi_fmha_softmax(XLA_FFI_CallFrame* call_frame);
XLA_FFI_Error* xmk_ffi_fmha_scale_bias_softmax(XLA_FFI_CallFrame* call_frame);

/* "__cudnn$fmhaSoftmaxBackward" / "__cudnn$fmhaScaleBiasSoftmaxBackward": replace
 * RunXetlaGpuFMHABackward (xetla_gpu_fused_mha_runner.cc:419-445; kinds dispatched at :404-416).
 * operands, in the runner's order: (Q, K, activation f32 [B,N,F] as written by the forward call, V,
 * d_output [, bias [B,N,F,T]], fwd_output) -> results (dQ, dK, dV [, scratch ...]).  Attributes as
 * for the forward targets.  Needs a host API table with XLA_FFI_DeviceMemory_Allocate / _Free (the
 * reference takes its dp_sum / accumulation buffers from the thunk's scratch, :392-399).  The
 * operand order the compiler emits is fixed in a patch that is not part of the reference tree. */
XLA_FFI_Error* xmk_ffi_fmha_softmax_backward(XLA_FFI_CallFrame* call_frame);
XLA_FFI_Error* xmk_ffi_fmha_scale_bias_softmax_backward(XLA_FFI_CallFrame* call_frame);

/* "__xmk$int4_gemm" (no counterpart in the reference): operands (act f16 [M,K], qweight s32|u32
 * [K/8,N], scales f16 [K/g,N], zeros f16 [K/g,N] [, bias f16 [N]]) -> results (out f16 [M,N]);
 * the group size is K / scales.dims[0]. */
XLA_FFI_Error* xmk_ffi_int4_gemm(XLA_FFI_CallFrame* call_frame);

/* "__cublas$lt$matmul$f8" (not in the reference snapshot; XLA's operand convention): operands
 * (a f8e4m3fn, b f8e4m3fn, a_scale f32[], b_scale f32[] [, c_scale f32[], d_scale f32[]] [, bias
 * bf16 [N]]) -> results (out bf16, ...), out = bf16(d_scale * (a_scale * b_scale * A B + bias)).
 * The bias is there exactly when the epilogue is BIAS.  c_scale multiplies the matrix addend, which
 * this target does not take (beta must be 0), so its value has no effect.  Every other operand
 * count, a matrix addend (beta != 0) and every other epilogue are rejected with UNIMPLEMENTED or
 * INVALID_ARGUMENT: no operand is dropped silently.  Attributes as for "__cublas$lt$matmul"; lhs
 * and output row-major, alpha 1, batch 1. */
XLA_FFI_Error* xmk_ffi_cublas_lt_matmul_f8(XLA_FFI_CallFrame* call_frame);

typedef struct xmk_ffi_target {
  const char* target;       /* custom_call_target string */
  XLA_FFI_Handler* handler; /* execute-stage handler */
} xmk_ffi_target;

/* The table of (target, handler) pairs above; *count receives its length. */
const xmk_ffi_target* xmk_ffi_targets(int32_t* count);

/* Registers every target with api->XLA_FFI_Handler_Register for `platform` (e.g. "ROCM"); the
 * counterpart of the XLA_FFI_REGISTER_HANDLER lines at sycl_custom_call.cc:223-226.  Returns
 * the first error, or NULL. */
XLA_FFI_Error* xmk_ffi_register_all(const XLA_FFI_Api* api, const char* platform);

#ifdef __cplusplus
}
#endif
#endif /* XMK_FFI_H_ */
