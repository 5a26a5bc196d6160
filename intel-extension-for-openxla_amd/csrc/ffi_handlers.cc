// XLA typed-FFI handlers: decode a call frame the way the reference's handlers do
// (xla/service/gpu/sycl_custom_call.cc:154-226, xla/service/gpu/onednn_matmul_utils.cc:533-621,
// xla/service/gpu/xetla_gpu_fused_mha_runner.cc:45-149) and call the kernel-level C ABI.
// Host code only: no device work happens here apart from the entry points it calls.
#include <cmath>
#include <cstdio>
#include <cstddef>
#include <cstring>
#include <string>

#include "common.h"
#include "xmk_ffi.h"

namespace {

struct Frame {
  XLA_FFI_CallFrame* f;
  std::string err;  // first decoding error
  int code = XMK_OK;

  void fail(int c, const std::string& msg) {
    if (code == XMK_OK) { code = c; err = msg; }
  }
  const XLA_FFI_Buffer* arg(int64_t i) {
    if (i < 0 || i >= f->args.size || f->args.types[i] != XLA_FFI_ArgType_BUFFER) {
      fail(XMK_INVALID_ARGUMENT, "operand " + std::to_string(i) + " is missing or not a buffer");
      return nullptr;
    }
    return static_cast<const XLA_FFI_Buffer*>(f->args.args[i]);
  }
  const XLA_FFI_Buffer* ret(int64_t i) {
    if (i < 0 || i >= f->rets.size || f->rets.types[i] != XLA_FFI_RetType_BUFFER) {
      fail(XMK_INVALID_ARGUMENT, "result " + std::to_string(i) + " is missing or not a buffer");
      return nullptr;
    }
    return static_cast<const XLA_FFI_Buffer*>(f->rets.rets[i]);
  }
  const XLA_FFI_Scalar* scalar(const char* name) const {
    const size_t n = std::strlen(name);
    for (int64_t i = 0; i < f->attrs.size; ++i) {
      const XLA_FFI_ByteSpan* s = f->attrs.names[i];
      if (s->len == n && std::memcmp(s->ptr, name, n) == 0)
        return f->attrs.types[i] == XLA_FFI_AttrType_SCALAR ? static_cast<const XLA_FFI_Scalar*>(f->attrs.attrs[i])
                                                             : nullptr;
    }
    return nullptr;
  }
  // Integer attribute of either width (the reference reads each key with one fixed type and
  // fails on the other; accepting both costs nothing).
  int64_t i64(const char* name) {
    const XLA_FFI_Scalar* s = scalar(name);
    if (s && s->dtype == XLA_FFI_DataType_S64) return *static_cast<const int64_t*>(s->value);
    if (s && s->dtype == XLA_FFI_DataType_S32) return *static_cast<const int32_t*>(s->value);
    if (s && s->dtype == XLA_FFI_DataType_PRED) return *static_cast<const uint8_t*>(s->value) != 0;
    fail(XMK_INVALID_ARGUMENT, std::string("attribute '") + name + "' is missing or not an integer");
    return 0;
  }
  double f64(const char* name) {
    const XLA_FFI_Scalar* s = scalar(name);
    if (s && s->dtype == XLA_FFI_DataType_F32) return *static_cast<const float*>(s->value);
    if (s && s->dtype == XLA_FFI_DataType_F64) return *static_cast<const double*>(s->value);
    fail(XMK_INVALID_ARGUMENT, std::string("attribute '") + name + "' is missing or not a float");
    return 0;
  }
  bool has(const char* name) const { return scalar(name) != nullptr; }

  void* stream() {
    XLA_FFI_Stream_Get_Args a;
    a.struct_size = sizeof(a);
    a.extension_start = nullptr;
    a.ctx = f->ctx;
    a.stream = nullptr;
    if (!f->api || !f->api->XLA_FFI_Stream_Get) {
      fail(XMK_INTERNAL, "call frame carries no XLA_FFI_Api");
      return nullptr;
    }
    if (XLA_FFI_Error* e = f->api->XLA_FFI_Stream_Get(&a)) {
      // The host's error object is handed back as is.
      host_error = e;
      fail(XMK_INTERNAL, "XLA_FFI_Stream_Get failed");
    }
    return a.stream;
  }
  XLA_FFI_Error* host_error = nullptr;
};

XLA_FFI_Error* make_error(XLA_FFI_CallFrame* f, int code, const std::string& msg) {
  // Without a host API there is no way to build an error object: hand back a non-null token.
  static char no_api_error_token;
  if (!f->api || !f->api->XLA_FFI_Error_Create) return reinterpret_cast<XLA_FFI_Error*>(&no_api_error_token);
  XLA_FFI_Error_Create_Args a;
  a.struct_size = sizeof(a);
  a.extension_start = nullptr;
  a.message = msg.c_str();
  a.errc = static_cast<XLA_FFI_Error_Code>(code);  // xmk_status uses absl::StatusCode values
  return f->api->XLA_FFI_Error_Create(&a);
}

XLA_FFI_Error* finish(Frame& fr, int rc) {
  if (fr.host_error) return fr.host_error;
  if (fr.code != XMK_OK) return make_error(fr.f, fr.code, fr.err);
  if (rc != XMK_OK) return make_error(fr.f, rc, xmk_last_error());
  return nullptr;
}

// A handler is called once per execution stage it was registered for, and with a metadata
// extension when the host asks for its API version.  Returns true if the call was such a query
// (nothing else to do).
bool metadata_query(XLA_FFI_CallFrame* f) {
  for (XLA_FFI_Extension_Base* e = f->extension_start; e; e = e->next) {
    if (e->type == XLA_FFI_Extension_Metadata) {
      XLA_FFI_Metadata* m = reinterpret_cast<XLA_FFI_Metadata_Extension*>(e)->metadata;
      m->api_version.major_version = XLA_FFI_API_MAJOR;
      m->api_version.minor_version = XLA_FFI_API_MINOR;
      m->traits = 0;
      return true;
    }
  }
  return false;
}

int64_t elements(const XLA_FFI_Buffer* b) {
  int64_t n = 1;
  for (int64_t i = 0; i < b->rank; ++i) n *= b->dims[i];
  return n;
}

// xla::gpu::GemmBackendConfig::Epilogue -> xmk_epilogue; the counterpart of AsSYCLEpilogue
// (onednn_matmul_utils.cc:111-135).
int as_xmk_epilogue(int64_t e) {
  switch (e) {
    case 0: return XMK_EPI_DEFAULT;
    case 1: return XMK_EPI_BIAS;
    case 2: return XMK_EPI_RELU;
    case 3: return XMK_EPI_BIAS_RELU;
    case 4: return XMK_EPI_GELU;
    case 5: return XMK_EPI_GELU_AUX;
    case 6: return XMK_EPI_BIAS_GELU;
    case 7: return XMK_EPI_BIAS_GELU_AUX;
    default: return -1;
  }
}
bool adds_vector_bias(int e) {
  return e == XMK_EPI_BIAS || e == XMK_EPI_BIAS_RELU || e == XMK_EPI_BIAS_GELU || e == XMK_EPI_BIAS_GELU_AUX;
}
bool has_aux_output(int e) { return e == XMK_EPI_GELU_AUX || e == XMK_EPI_BIAS_GELU_AUX; }

// The three descriptors RunGemm builds from the dictionary (onednn_matmul_utils.cc:544-584):
// a column-major layout becomes `transpose` with rows and columns swapped.
xmk_matrix matrix_from_dict(Frame& fr, const char* who, void* data) {
  const std::string p(who);
  const bool t = fr.i64((p + "_order").c_str()) == 1;  // MatrixLayout::Order::kColumnMajor
  const int64_t rows = fr.i64((p + "_num_rows").c_str()), cols = fr.i64((p + "_num_cols").c_str());
  xmk_matrix m;
  m.data = data;
  m.transpose = t;
  m.num_rows = t ? cols : rows;
  m.num_cols = t ? rows : cols;
  m.batch_stride = fr.i64((p + "_batch_stride").c_str());
  m.leading_dim_stride = fr.i64((p + "_leading_dim_stride").c_str());
  return m;
}

void destroy_error(const XLA_FFI_Api* api, XLA_FFI_Error* e) {
  if (!api->XLA_FFI_Error_Destroy) return;
  XLA_FFI_Error_Destroy_Args a;
  a.struct_size = sizeof(a);
  a.extension_start = nullptr;
  a.error = e;
  api->XLA_FFI_Error_Destroy(&a);
}

// Runs body(workspace) with `need` bytes of the executor's scratch when the API table has the allocator
// entries and the allocation succeeds, else body(nullptr).  The scratch is handed back right after the
// work is enqueued: the executor's allocator frees in stream order, so later work on the stream may reuse it.
template <typename Body>
int with_scratch(XLA_FFI_CallFrame* f, size_t need, Body&& body) {
  const XLA_FFI_Api* api = f->api;
  const bool can_allocate = need > 0 && api &&
                            api->struct_size >= offsetof(XLA_FFI_Api, XLA_FFI_DeviceMemory_Free) + sizeof(void*) &&
                            api->XLA_FFI_DeviceMemory_Allocate && api->XLA_FFI_DeviceMemory_Free;
  if (can_allocate) {
    XLA_FFI_DeviceMemory_Allocate_Args al;
    al.struct_size = sizeof(al);
    al.extension_start = nullptr;
    al.ctx = f->ctx;
    al.size = need;
    al.alignment = 256;
    al.data = nullptr;
    XLA_FFI_Error* e = api->XLA_FFI_DeviceMemory_Allocate(&al);
    if (!e && al.data) {
      const int rc = body(al.data);
      XLA_FFI_DeviceMemory_Free_Args fa;
      fa.struct_size = sizeof(fa);
      fa.extension_start = nullptr;
      fa.ctx = f->ctx;
      fa.size = need;
      fa.data = al.data;
      XLA_FFI_Error* fe = api->XLA_FFI_DeviceMemory_Free(&fa);
      if (fe) destroy_error(api, fe);
      return rc;
    }
    if (e) destroy_error(api, e);
  }
  return body(nullptr);
}

XLA_FFI_Error* gemm_common(XLA_FFI_CallFrame* f, bool lt) {
  if (metadata_query(f) || f->stage != XLA_FFI_ExecutionStage_EXECUTE) return nullptr;
  Frame fr{f};
  int epilogue = XMK_EPI_DEFAULT;
  if (lt) {
    epilogue = as_xmk_epilogue(fr.i64("epilogue"));
    if (epilogue < 0) fr.fail(XMK_INTERNAL, "Unsupported Epilogue.");  // onednn_matmul_utils.cc:133
  }
  const float beta = (float)fr.f64("beta");
  const bool matrix_bias = lt && beta != 0.0f;  // sycl_custom_call.cc:181
  const XLA_FFI_Buffer* lhs = fr.arg(0);
  const XLA_FFI_Buffer* rhs = fr.arg(1);
  // With a matrix addend the result aliases operand 2 and is computed in place (:191-195).
  const XLA_FFI_Buffer* out = matrix_bias ? fr.arg(2) : fr.ret(has_aux_output(epilogue) ? 1 : 0);
  const XLA_FFI_Buffer* bias = (lt && adds_vector_bias(epilogue)) ? fr.arg(matrix_bias ? 3 : 2) : nullptr;
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);

  xmk_gemm_desc d;
  std::memset(&d, 0, sizeof(d));
  d.lhs = matrix_from_dict(fr, "lhs", lhs->data);
  d.rhs = matrix_from_dict(fr, "rhs", rhs->data);
  d.out = matrix_from_dict(fr, "output", out->data);
  d.c = beta != 0.0f ? out->data : nullptr;
  d.bias = bias ? bias->data : nullptr;
  d.dtype_in = (int32_t)fr.i64("lhs_layout_dtype");
  d.dtype_out = (int32_t)fr.i64("output_layout_dtype");
  if (fr.code == XMK_OK && fr.i64("rhs_layout_dtype") != d.dtype_in)
    fr.fail(XMK_INTERNAL, "Unexpected GEMM lhs type / rhs type");  // onednn_matmul_utils.cc:613
  d.batch_size = fr.i64("batch_size");
  d.alpha = (float)fr.f64("alpha");
  d.beta = beta;
  d.epilogue = epilogue;
  void* stream = fr.stream();
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  // Shapes that gain from a K split take their fp32 partial sums from the executor's scratch allocator
  // (the reference's handlers hold one too, sycl_custom_call.cc:154-156), when the API table has it.
  const size_t need = xmk_gemm_workspace_bytes(&d);
  return finish(fr, with_scratch(f, need, [&](void* ws) {
    return ws ? xmk_gemm_ws(&d, ws, need, stream) : xmk_gemm(&d, stream);  // no scratch: the unsplit kernel
  }));
}

XLA_FFI_Error* fmha_common(XLA_FFI_CallFrame* f, bool with_bias) {
  if (metadata_query(f) || f->stage != XLA_FFI_ExecutionStage_EXECUTE) return nullptr;
  Frame fr{f};
  const XLA_FFI_Buffer* q = fr.arg(0);
  const XLA_FFI_Buffer* k = fr.arg(1);
  const XLA_FFI_Buffer* v = fr.arg(2);
  const XLA_FFI_Buffer* bias = with_bias ? fr.arg(3) : nullptr;
  const XLA_FFI_Buffer* out = fr.ret(0);
  // results: (out, scratch [, activation]); the activation (log-sum-exp) marks a training call
  // (xetla_gpu_fused_mha_runner.cc:159-164).
  const XLA_FFI_Buffer* act = f->rets.size > 2 ? fr.ret(2) : nullptr;
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  if (fr.has("dropout_rate") && fr.f64("dropout_rate") != 0.0)
    fr.fail(XMK_UNIMPLEMENTED, "Unimplemented dropout");  // :57-61
  const int64_t rank = q->rank;
  if ((rank != 3 && rank != 4) || k->rank != rank || v->rank != rank || out->rank != rank)
    fr.fail(XMK_INVALID_ARGUMENT, "fmha: operands must all have rank 3 or 4");
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  // [B,N,F,H] * [B,N,T,H] * [B,N,T,H] (:118-127)
  const int64_t B = rank == 4 ? q->dims[0] : 1;
  const int64_t N = q->dims[rank - 3], F = q->dims[rank - 2], H = q->dims[rank - 1];
  const int64_t T = k->dims[rank - 2];
  if (k->dims[rank - 1] != H || v->dims[rank - 1] != H || v->dims[rank - 2] != T || k->dims[rank - 3] != N ||
      v->dims[rank - 3] != N || elements(q) != B * N * F * H || elements(k) != B * N * T * H ||
      elements(v) != B * N * T * H || elements(out) != B * N * F * H || (bias && elements(bias) != B * N * F * T) ||
      (act && elements(act) != B * N * F))
    fr.fail(XMK_INVALID_ARGUMENT, "fmha: operand shapes do not agree");
  if (q->dtype != k->dtype || q->dtype != v->dtype || q->dtype != out->dtype || (bias && bias->dtype != q->dtype))
    fr.fail(XMK_INVALID_ARGUMENT, "fmha: operand types do not agree");
  if (act && act->dtype != XLA_FFI_DataType_F32) fr.fail(XMK_INVALID_ARGUMENT, "fmha: activation must be f32");
  float scale = fr.has("fmha_scale") ? (float)fr.f64("fmha_scale") : 1.0f;
  // "Recalculate scale since scale attr has accuracy issue" (:128-129)
  if ((scale - 1.0f) > 1e-6f) scale = 1.0f / std::sqrt((float)H);
  const int causal = fr.has("is_causal_mask") ? (int)fr.i64("is_causal_mask") : 0;
  void* stream = fr.stream();
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  // dtype other than F16 / BF16 is rejected by the entry point with the reference's message.
  return finish(fr, xmk_fmha_fwd(q->data, k->data, v->data, bias ? bias->data : nullptr, out->data,
                                 act ? static_cast<float*>(act->data) : nullptr, (int32_t)q->dtype, (uint32_t)B,
                                 (uint32_t)N, (uint32_t)H, (uint32_t)F, (uint32_t)T, scale, causal, stream));
}

// Backward kinds (CudnnfMHAKind::kBackwardSoftmax / kBackwardScaleBiasSoftmax, dispatched at
// xetla_gpu_fused_mha_runner.cc:404-416).  Operands in the runner's order (:419-433):
// bmm1_grad_gemm1_rhs = Q, bmm1_grad_gemm2_rhs = K, bmm2_grad_gemm1_lhs = the forward activation
// (log-sum-exp, f32 [B,N,F]), bmm2_grad_gemm2_rhs = V, d_output [, bias], fwd_output.
// Results: d_bmm1_lhs = dQ, d_bmm1_rhs = dK, d_bmm2_rhs = dV [, scratch ...]; d_s and d_bias are not
// produced (the reference passes d_bias on but its kernel never writes it, :383-385).
XLA_FFI_Error* fmha_bwd_common(XLA_FFI_CallFrame* f, bool with_bias) {
  if (metadata_query(f) || f->stage != XLA_FFI_ExecutionStage_EXECUTE) return nullptr;
  Frame fr{f};
  const XLA_FFI_Buffer* q = fr.arg(0);
  const XLA_FFI_Buffer* k = fr.arg(1);
  const XLA_FFI_Buffer* act = fr.arg(2);
  const XLA_FFI_Buffer* v = fr.arg(3);
  const XLA_FFI_Buffer* d_out = fr.arg(4);
  const XLA_FFI_Buffer* bias = with_bias ? fr.arg(5) : nullptr;
  const XLA_FFI_Buffer* fwd_out = fr.arg(with_bias ? 6 : 5);
  const XLA_FFI_Buffer* dq = fr.ret(0);
  const XLA_FFI_Buffer* dk = fr.ret(1);
  const XLA_FFI_Buffer* dv = fr.ret(2);
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  if (fr.has("dropout_rate") && fr.f64("dropout_rate") != 0.0)
    fr.fail(XMK_UNIMPLEMENTED, "Unimplemented dropout");  // :244-250
  const int64_t rank = q->rank;
  if ((rank != 3 && rank != 4) || k->rank != rank || v->rank != rank || d_out->rank != rank || fwd_out->rank != rank)
    fr.fail(XMK_INVALID_ARGUMENT, "fmha backward: operands must all have rank 3 or 4");
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  const int64_t B = rank == 4 ? q->dims[0] : 1;
  const int64_t N = q->dims[rank - 3], F = q->dims[rank - 2], H = q->dims[rank - 1];
  const int64_t T = k->dims[rank - 2];
  if (k->dims[rank - 1] != H || v->dims[rank - 1] != H || v->dims[rank - 2] != T || k->dims[rank - 3] != N ||
      v->dims[rank - 3] != N || elements(k) != B * N * T * H || elements(v) != B * N * T * H ||
      elements(d_out) != B * N * F * H || elements(fwd_out) != B * N * F * H ||
      elements(act) != B * N * F || elements(dq) != B * N * F * H || elements(dk) != B * N * T * H ||
      elements(dv) != B * N * T * H || (bias && elements(bias) != B * N * F * T))
    fr.fail(XMK_INVALID_ARGUMENT, "fmha backward: operand shapes do not agree");
  for (const XLA_FFI_Buffer* b : {k, v, d_out, fwd_out, dq, dk, dv})
    if (b->dtype != q->dtype) fr.fail(XMK_INVALID_ARGUMENT, "fmha backward: operand types do not agree");
  if (bias && bias->dtype != q->dtype) fr.fail(XMK_INVALID_ARGUMENT, "fmha backward: operand types do not agree");
  if (act->dtype != XLA_FFI_DataType_F32) fr.fail(XMK_INVALID_ARGUMENT, "fmha backward: activation must be f32");
  float scale = fr.has("fmha_scale") ? (float)fr.f64("fmha_scale") : 1.0f;
  if ((scale - 1.0f) > 1e-6f) scale = 1.0f / std::sqrt((float)H);  // as in the forward handler
  const int causal = fr.has("is_causal_mask") ? (int)fr.i64("is_causal_mask") : 0;
  void* stream = fr.stream();
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  // dp_sum / grad_query_accum of the reference (:392-399) are one workspace here, from the
  // executor's scratch allocator.
  const size_t need = xmk_fmha_bwd_workspace_bytes((uint32_t)B, (uint32_t)N, (uint32_t)H, (uint32_t)F, (uint32_t)T);
  return finish(fr, with_scratch(f, need, [&](void* ws) {
    if (!ws) return xmk::fail(XMK_INTERNAL, "fmha backward: the host's API table has no scratch allocator");
    return xmk_fmha_bwd(q->data, k->data, v->data, bias ? bias->data : nullptr, fwd_out->data, d_out->data,
                        static_cast<const float*>(act->data), dq->data, dk->data, dv->data, (int32_t)q->dtype,
                        (uint32_t)B, (uint32_t)N, (uint32_t)H, (uint32_t)F, (uint32_t)T, scale, causal, ws, need, stream);
  }));
}

const xmk_ffi_target kTargets[] = {
    {"__cublas$gemm", xmk_ffi_cublas_gemm},
    {"__cublas$lt$matmul", xmk_ffi_cublas_lt_matmul},
    {"__cudnn$fmhaSoftmax", xmk_ffi_fmha_softmax},
    {"__cudnn$fmhaScaleBiasSoftmax", xmk_ffi_fmha_scale_bias_softmax},
    {"__cudnn$fmhaSoftmaxBackward", xmk_ffi_fmha_softmax_backward},
    {"__cudnn$fmhaScaleBiasSoftmaxBackward", xmk_ffi_fmha_scale_bias_softmax_backward},
    {"__xmk$int4_gemm", xmk_ffi_int4_gemm},
    {"__cublas$lt$matmul$f8", xmk_ffi_cublas_lt_matmul_f8},
};

}  // namespace

extern "C" XLA_FFI_Error* xmk_ffi_cublas_gemm(XLA_FFI_CallFrame* f) { return gemm_common(f, false); }
extern "C" XLA_FFI_Error* xmk_ffi_cublas_lt_matmul(XLA_FFI_CallFrame* f) { return gemm_common(f, true); }
extern "C" XLA_FFI_Error* xmk_ffi_fmha_softmax(XLA_FFI_CallFrame* f) { return fmha_common(f, false); }
extern "C" XLA_FFI_Error* xmk_ffi_fmha_scale_bias_softmax(XLA_FFI_CallFrame* f) { return fmha_common(f, true); }
extern "C" XLA_FFI_Error* xmk_ffi_fmha_softmax_backward(XLA_FFI_CallFrame* f) { return fmha_bwd_common(f, false); }
extern "C" XLA_FFI_Error* xmk_ffi_fmha_scale_bias_softmax_backward(XLA_FFI_CallFrame* f) {
  return fmha_bwd_common(f, true);
}

extern "C" XLA_FFI_Error* xmk_ffi_int4_gemm(XLA_FFI_CallFrame* f) {
  if (metadata_query(f) || f->stage != XLA_FFI_ExecutionStage_EXECUTE) return nullptr;
  Frame fr{f};
  const XLA_FFI_Buffer* act = fr.arg(0);
  const XLA_FFI_Buffer* qw = fr.arg(1);
  const XLA_FFI_Buffer* sc = fr.arg(2);
  const XLA_FFI_Buffer* zp = fr.arg(3);
  const XLA_FFI_Buffer* bias = f->args.size > 4 ? fr.arg(4) : nullptr;
  const XLA_FFI_Buffer* out = fr.ret(0);
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  if (act->rank != 2 || qw->rank != 2 || sc->rank != 2 || zp->rank != 2 || out->rank != 2 || (bias && bias->rank != 1))
    fr.fail(XMK_INVALID_ARGUMENT, "int4_gemm: act, qweight, scales, zeros, out must have rank 2, bias rank 1");
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  const int64_t M = act->dims[0], K = act->dims[1], N = out->dims[1];
  if (act->dtype != XLA_FFI_DataType_F16 || out->dtype != XLA_FFI_DataType_F16 || sc->dtype != XLA_FFI_DataType_F16 ||
      zp->dtype != XLA_FFI_DataType_F16 || (qw->dtype != XLA_FFI_DataType_S32 && qw->dtype != XLA_FFI_DataType_U32) ||
      (bias && bias->dtype != XLA_FFI_DataType_F16))
    fr.fail(XMK_INVALID_ARGUMENT, "int4_gemm: act/scales/zeros/bias/out must be f16 and qweight s32 or u32");
  const int64_t groups = sc->dims[0];
  if (out->dims[0] != M || qw->dims[0] * 8 != K || qw->dims[1] != N || sc->dims[1] != N || zp->dims[0] != groups ||
      zp->dims[1] != N || groups <= 0 || K % groups != 0 || (bias && bias->dims[0] != N))
    fr.fail(XMK_INVALID_ARGUMENT, "int4_gemm: operand shapes do not agree");
  void* stream = fr.stream();
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  // Many rows (prompt processing): the dequantised weights go to executor scratch and the dense GEMM runs.
  const size_t need = xmk_int4_gemm_workspace_bytes(M, K, N);
  return finish(fr, with_scratch(f, need, [&](void* ws) {
    return xmk_int4_gemm_ws(act->data, qw->data, sc->data, zp->data, bias ? bias->data : nullptr, out->data, M, K, N,
                            K / groups, ws, ws ? need : 0, stream);
  }));
}

extern "C" XLA_FFI_Error* xmk_ffi_cublas_lt_matmul_f8(XLA_FFI_CallFrame* f) {
  if (metadata_query(f) || f->stage != XLA_FFI_ExecutionStage_EXECUTE) return nullptr;
  Frame fr{f};
  const XLA_FFI_Buffer* a = fr.arg(0);
  const XLA_FFI_Buffer* b = fr.arg(1);
  const XLA_FFI_Buffer* a_scale = fr.arg(2);
  const XLA_FFI_Buffer* b_scale = fr.arg(3);
  const XLA_FFI_Buffer* out = fr.ret(0);
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  const int epilogue = fr.has("epilogue") ? as_xmk_epilogue(fr.i64("epilogue")) : XMK_EPI_DEFAULT;
  if (epilogue != XMK_EPI_DEFAULT && epilogue != XMK_EPI_BIAS)
    fr.fail(XMK_UNIMPLEMENTED, "matmul$f8: epilogue must be DEFAULT or BIAS");
  if (fr.f64("beta") != 0.0 || fr.f64("alpha") != 1.0 || fr.i64("batch_size") != 1)
    fr.fail(XMK_UNIMPLEMENTED, "matmul$f8: needs alpha 1, beta 0 (no matrix addend), batch 1");
  // Operands after b_scale: [c_scale, d_scale] [, bias].  Like the reference's handlers
  // (sycl_custom_call.cc:168-205) every operand handed over is either used or refused.
  const bool with_bias = epilogue == XMK_EPI_BIAS;
  const int64_t rest = f->args.size - 4 - (with_bias ? 1 : 0);
  if (fr.code == XMK_OK && rest != 0 && rest != 2)
    fr.fail(XMK_INVALID_ARGUMENT, "matmul$f8: " + std::to_string(f->args.size) + " operands do not fit (a, b, a_scale, "
            "b_scale [, c_scale, d_scale] [, bias]) with epilogue " + (with_bias ? "BIAS" : "DEFAULT"));
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  const XLA_FFI_Buffer* c_scale = rest == 2 ? fr.arg(4) : nullptr;
  const XLA_FFI_Buffer* d_scale = rest == 2 ? fr.arg(5) : nullptr;
  const XLA_FFI_Buffer* bias = with_bias ? fr.arg(4 + rest) : nullptr;
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  if (a->dtype != XLA_FFI_DataType_F8E4M3FN || b->dtype != XLA_FFI_DataType_F8E4M3FN)
    fr.fail(XMK_UNIMPLEMENTED, "matmul$f8: operands must be f8e4m3fn");
  if (out->dtype != XLA_FFI_DataType_BF16) fr.fail(XMK_UNIMPLEMENTED, "matmul$f8: output must be bf16");
  for (const XLA_FFI_Buffer* s : {a_scale, b_scale, c_scale, d_scale})
    if (s && (s->dtype != XLA_FFI_DataType_F32 || elements(s) != 1))
      fr.fail(XMK_INVALID_ARGUMENT, "matmul$f8: a_scale, b_scale, c_scale and d_scale must be f32 scalars");
  if (fr.i64("lhs_order") != 0 || fr.i64("output_order") != 0)
    fr.fail(XMK_UNIMPLEMENTED, "matmul$f8: lhs and output must be row-major");
  const int64_t M = fr.i64("lhs_num_rows"), K = fr.i64("lhs_num_cols"), N = fr.i64("rhs_num_cols");
  const int rhs_t = fr.i64("rhs_order") == 1;  // column-major [k,n] is stored as [n,k]
  if (fr.code == XMK_OK && (fr.i64("rhs_num_rows") != K || elements(a) != M * K || elements(b) != K * N ||
                            elements(out) != M * N || fr.i64("lhs_leading_dim_stride") != K ||
                            fr.i64("rhs_leading_dim_stride") != (rhs_t ? K : N) ||
                            fr.i64("output_leading_dim_stride") != N))
    fr.fail(XMK_INVALID_ARGUMENT, "matmul$f8: shapes do not agree or operands are not packed");
  if (bias && (bias->dtype != XLA_FFI_DataType_BF16 || elements(bias) != N))
    fr.fail(XMK_INVALID_ARGUMENT, "matmul$f8: bias must be bf16 [N]");
  void* stream = fr.stream();
  if (fr.code != XMK_OK) return finish(fr, XMK_OK);
  return finish(fr, xmk_fp8_gemm_ex(a->data, b->data, static_cast<const float*>(a_scale->data),
                                    static_cast<const float*>(b_scale->data),
                                    d_scale ? static_cast<const float*>(d_scale->data) : nullptr,
                                    bias ? bias->data : nullptr, out->data, M, N, K, rhs_t, stream));
}

extern "C" const xmk_ffi_target* xmk_ffi_targets(int32_t* count) {
  if (count) *count = (int32_t)(sizeof(kTargets) / sizeof(kTargets[0]));
  return kTargets;
}

extern "C" XLA_FFI_Error* xmk_ffi_register_all(const XLA_FFI_Api* api, const char* platform) {
  if (!api || !api->XLA_FFI_Handler_Register || !platform) return nullptr;
  for (const xmk_ffi_target& t : kTargets) {
    XLA_FFI_Handler_Register_Args a;
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.name.ptr = t.target;
    a.name.len = std::strlen(t.target);
    a.platform.ptr = platform;
    a.platform.len = std::strlen(platform);
    a.bundle.execute = t.handler;
    a.traits = 0;
    if (XLA_FFI_Error* e = api->XLA_FFI_Handler_Register(&a)) return e;
  }
  return nullptr;
}
