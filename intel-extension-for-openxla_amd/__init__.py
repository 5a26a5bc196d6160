"""MI355X (gfx950) kernels behind the XLA custom calls of the reference PJRT plugin.

The product is ``libxmk.so`` (``include/xmk.h``): hand-written HIP kernels behind a
C ABI.  This module is the thin ctypes binding the tests and the benchmark use;
torch only supplies device memory and the stream.  There is no CPU fallback: if
the library is missing or a call fails, the wrappers raise.

Function names follow the reference's host entry points:
``run_gemm`` <-> RunGemm (xla/service/gpu/onednn_matmul_utils.h:58-73),
``fmha_forward`` <-> fmha_forward_kernel_{fp16,bf16} (xla/service/gpu/xetla/sdp/sdp_forward.h:22-36).
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("XMK_LIB") or os.path.join(_HERE, "libxmk.so")  # XMK_LIB: load another build

# xla::PrimitiveType numbering
S8, S32, F16, F32, BF16, F8E4M3FN = 2, 4, 10, 11, 16, 20
# SYCLGemm::GemmBackendEpilogue numbering (onednn_matmul_utils.h:35-45)
(EPI_DEFAULT, EPI_RELU, EPI_GELU, EPI_BIAS, EPI_BIAS_RELU, EPI_BIAS_GELU, EPI_GELU_AUX,
 EPI_BIAS_GELU_AUX) = range(8)

OK, INVALID_ARGUMENT, UNIMPLEMENTED, INTERNAL = 0, 3, 12, 13

_TORCH_DTYPE = {torch.float16: F16, torch.bfloat16: BF16, torch.float32: F32,
                torch.float8_e4m3fn: F8E4M3FN, torch.int8: S8, torch.int32: S32}


class XmkError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"xmk status {code}: {message}")
        self.code = code
        self.message = message


class Matrix(ctypes.Structure):
    """xmk_matrix (mirrors xla::gpu::MatrixDescriptor, matrix_descriptor.h:30-46)."""
    _fields_ = [("data", ctypes.c_void_p), ("transpose", ctypes.c_int32),
                ("num_rows", ctypes.c_int64), ("num_cols", ctypes.c_int64),
                ("batch_stride", ctypes.c_int64), ("leading_dim_stride", ctypes.c_int64)]


class GemmDesc(ctypes.Structure):
    """xmk_gemm_desc."""
    _fields_ = [("lhs", Matrix), ("rhs", Matrix), ("out", Matrix), ("c", ctypes.c_void_p),
                ("bias", ctypes.c_void_p), ("dtype_in", ctypes.c_int32),
                ("dtype_out", ctypes.c_int32), ("batch_size", ctypes.c_int64),
                ("alpha", ctypes.c_float), ("beta", ctypes.c_float), ("epilogue", ctypes.c_int32)]


_lib = None


def lib():
    """Loads libxmk.so; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run `python {_HERE}/build.py` "
                               "(there is no CPU fallback)")
        L = ctypes.CDLL(LIB_PATH)
        for name, restype in (("xmk_version", ctypes.c_char_p),
                              ("xmk_last_error", ctypes.c_char_p),
                              ("xmk_gemm_policy_name", ctypes.c_char_p),
                              ("xmk_fmha_decode_workspace_bytes", ctypes.c_size_t),
                              ("xmk_fmha_decode_cache_workspace_bytes", ctypes.c_size_t),
                              ("xmk_fmha_decode_static_max_bytes", ctypes.c_size_t),
                              ("xmk_fmha_bwd_workspace_bytes", ctypes.c_size_t),
                              ("xmk_gemm_workspace_bytes", ctypes.c_size_t),
                              ("xmk_int4_gemm_workspace_bytes", ctypes.c_size_t)):
            if hasattr(L, name):
                getattr(L, name).restype = restype
        _lib = L
    return _lib


def _check(code):
    if code != 0:
        raise XmkError(code, lib().xmk_last_error().decode())


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(stream=None):
    s = torch.cuda.current_stream() if stream is None else stream
    return ctypes.c_void_p(s.cuda_stream)


def dtype_code(t):
    return _TORCH_DTYPE[t.dtype]


def version():
    return lib().xmk_version().decode()


# ----------------------------------------------------------------------- GEMM
def matrix(t, transpose=False, batch_stride=None):
    """Describes a 2-D (or batched 3-D) row-major tensor as an xmk_matrix."""
    rows, cols = t.shape[-2], t.shape[-1]
    ld = t.stride(-2)
    bs = (t.stride(0) if t.dim() == 3 else 0) if batch_stride is None else batch_stride
    return Matrix(t.data_ptr(), int(bool(transpose)), rows, cols, bs, ld)


def run_gemm_desc(desc, stream=None):
    _check(lib().xmk_gemm(ctypes.byref(desc), _stream(stream)))


def run_gemm(lhs, rhs, out, *, lhs_transpose=False, rhs_transpose=False, out_transpose=False,
             c=None, bias=None, alpha=1.0, beta=0.0, epilogue=EPI_DEFAULT, stream=None, workspace=None):
    """out = act(alpha * op(lhs) op(rhs) + beta * c + bias).  Tensors are the *stored*
    row-major matrices; ``*_transpose`` marks the operand as the transpose of what is
    stored (a column-major XLA layout)."""
    batch = lhs.shape[0] if lhs.dim() == 3 else 1
    d = GemmDesc(matrix(lhs, lhs_transpose), matrix(rhs, rhs_transpose),
                 matrix(out, out_transpose), None if c is None else c.data_ptr(),
                 None if bias is None else bias.data_ptr(), dtype_code(lhs), dtype_code(out),
                 batch, alpha, beta, epilogue)
    if workspace is not None:
        _check(lib().xmk_gemm_ws(ctypes.byref(d), _ptr(workspace), ctypes.c_size_t(workspace.numel() * workspace.element_size()),
                                 _stream(stream)))
    else:
        run_gemm_desc(d, stream)
    return out


def gemm_workspace_bytes(lhs, rhs, out, *, lhs_transpose=False, rhs_transpose=False, out_transpose=False):
    d = GemmDesc(matrix(lhs, lhs_transpose), matrix(rhs, rhs_transpose), matrix(out, out_transpose), None, None,
                 dtype_code(lhs), dtype_code(out), 1, 1.0, 0.0, EPI_DEFAULT)
    return lib().xmk_gemm_workspace_bytes(ctypes.byref(d))


def run_gemm_qkv(lhs, weights, out_q, out_k, out_v, *, rhs_transpose=False, bias=None, epilogue=EPI_DEFAULT,
                 stream=None):
    """out_i = act(lhs @ weights[i] + bias[i]) for the three stacked weights [3, k, n] (or [3, n, k] with
    ``rhs_transpose``) in one launch; bias is [3, n] or None."""
    rhs = matrix(weights[0], rhs_transpose)
    rhs.batch_stride = weights.stride(0)
    d = GemmDesc(matrix(lhs, False), rhs, matrix(out_q, False), None,
                 None if bias is None else bias.data_ptr(), dtype_code(lhs), dtype_code(out_q), 1, 1.0, 0.0, epilogue)
    _check(lib().xmk_gemm_qkv(ctypes.byref(d), _ptr(out_k), _ptr(out_v), _stream(stream)))
    return out_q, out_k, out_v


def gemm_policy_name(m, n, k, rhs_transpose=False, dtype_in=BF16, dtype_out=BF16):
    return lib().xmk_gemm_policy_name(ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k),
                                      ctypes.c_int32(int(rhs_transpose)), ctypes.c_int32(dtype_in),
                                      ctypes.c_int32(dtype_out)).decode()


# ------------------------------------------------------------------ attention
def fmha_forward(query, key, value, out, *, bias=None, lse=None, head_scale=None, causal=False,
                 stream=None):
    """query [B,N,F,H], key/value [B,N,T,H], out [B,N,F,H]; bias [B,N,F,T]; lse fp32 [B*N,F]."""
    B, N, F, H = query.shape
    T = key.shape[2]
    scale = (H ** -0.5) if head_scale is None else head_scale
    _check(lib().xmk_fmha_fwd(_ptr(query), _ptr(key), _ptr(value), _ptr(bias), _ptr(out),
                              _ptr(lse), ctypes.c_int32(dtype_code(query)), ctypes.c_uint32(B),
                              ctypes.c_uint32(N), ctypes.c_uint32(H), ctypes.c_uint32(F),
                              ctypes.c_uint32(T), ctypes.c_float(scale),
                              ctypes.c_int32(int(causal)), _stream(stream)))
    return out


def fmha_backward(query, key, value, out, grad_out, lse, *, bias=None, head_scale=None, causal=False, stream=None):
    """Gradients (dq, dk, dv) of fmha_forward's output with respect to query, key, value."""
    B, N, F, H = query.shape
    T = key.shape[2]
    scale = (H ** -0.5) if head_scale is None else head_scale
    nbytes = lib().xmk_fmha_bwd_workspace_bytes(ctypes.c_uint32(B), ctypes.c_uint32(N), ctypes.c_uint32(H),
                                                ctypes.c_uint32(F), ctypes.c_uint32(T))
    ws = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=query.device)
    dq, dk, dv = torch.empty_like(query), torch.empty_like(key), torch.empty_like(value)
    _check(lib().xmk_fmha_bwd(_ptr(query), _ptr(key), _ptr(value), _ptr(bias), _ptr(out), _ptr(grad_out), _ptr(lse),
                              _ptr(dq), _ptr(dk), _ptr(dv), ctypes.c_int32(dtype_code(query)), ctypes.c_uint32(B),
                              ctypes.c_uint32(N), ctypes.c_uint32(H), ctypes.c_uint32(F), ctypes.c_uint32(T),
                              ctypes.c_float(scale), ctypes.c_int32(int(causal)), _ptr(ws), ctypes.c_size_t(nbytes),
                              _stream(stream)))
    return dq, dk, dv


def fmha_decode_workspace_bytes(B, N, H, T):
    return lib().xmk_fmha_decode_workspace_bytes(ctypes.c_uint32(B), ctypes.c_uint32(N),
                                                 ctypes.c_uint32(H), ctypes.c_uint32(T))


def fmha_decode_cache_workspace_bytes(B, N, H, capacity):
    """Workspace that serves fmha_decode for every num_keys in 1..capacity."""
    return lib().xmk_fmha_decode_cache_workspace_bytes(ctypes.c_uint32(B), ctypes.c_uint32(N),
                                                       ctypes.c_uint32(H), ctypes.c_uint32(capacity))


def fmha_decode(query, key, value, out, workspace, *, num_keys=None, kv_head_stride=None,
                head_scale=None, stream=None):
    """query/out [B,N,1,H] (or [B,N,H]); key/value [B,N,Tcap,H] caches of which the first
    ``num_keys`` rows are attended."""
    B, N = query.shape[0], query.shape[1]
    H = query.shape[-1]
    T = key.shape[2] if num_keys is None else num_keys
    stride = key.stride(1) if kv_head_stride is None else kv_head_stride
    scale = (H ** -0.5) if head_scale is None else head_scale
    _check(lib().xmk_fmha_decode(_ptr(query), _ptr(key), _ptr(value), _ptr(out),
                                 ctypes.c_int32(dtype_code(query)), ctypes.c_uint32(B),
                                 ctypes.c_uint32(N), ctypes.c_uint32(H), ctypes.c_uint32(T),
                                 ctypes.c_int64(stride), ctypes.c_float(scale), _ptr(workspace),
                                 ctypes.c_size_t(workspace.numel() * workspace.element_size()),
                                 _stream(stream)))
    return out


def fmha_decode_static(query, key, value, out, *, num_keys=None, kv_head_stride=None, head_scale=None,
                       stream=None):
    """fmha_decode without a workspace argument: the key splits' partial results go to an array
    inside the library image (xmk_fmha_decode_static: it allocates nothing)."""
    B, N = query.shape[0], query.shape[1]
    H = query.shape[-1]
    T = key.shape[2] if num_keys is None else num_keys
    stride = key.stride(1) if kv_head_stride is None else kv_head_stride
    scale = (H ** -0.5) if head_scale is None else head_scale
    _check(lib().xmk_fmha_decode_static(_ptr(query), _ptr(key), _ptr(value), _ptr(out),
                                        ctypes.c_int32(dtype_code(query)), ctypes.c_uint32(B),
                                        ctypes.c_uint32(N), ctypes.c_uint32(H), ctypes.c_uint32(T),
                                        ctypes.c_int64(stride), ctypes.c_float(scale), _stream(stream)))
    return out


def fmha_decode_static_max_bytes():
    return lib().xmk_fmha_decode_static_max_bytes()


def fmha_decode_static_init():
    """Looks up the built-in scratch array on the current device (to be done before stream capture)."""
    _check(lib().xmk_fmha_decode_static_init())


# ----------------------------------------------------------------------- int4
def int4_gemm(act, qweight, scales, zeros, out, *, group=128, bias=None, stream=None):
    m, k = act.shape
    n = qweight.shape[1]
    _check(lib().xmk_int4_gemm(_ptr(act), _ptr(qweight), _ptr(scales), _ptr(zeros), _ptr(bias),
                               _ptr(out), ctypes.c_int64(m), ctypes.c_int64(k), ctypes.c_int64(n),
                               ctypes.c_int64(group), _stream(stream)))
    return out


def int4_gemm_workspace_bytes(m, k, n):
    return lib().xmk_int4_gemm_workspace_bytes(ctypes.c_int64(m), ctypes.c_int64(k), ctypes.c_int64(n))


def int4_gemm_ws(act, qweight, scales, zeros, out, workspace, *, group=128, bias=None, stream=None):
    """xmk_int4_gemm_ws: with enough scratch and rows, dequantise once and run the dense fp16 GEMM."""
    m, k = act.shape
    n = qweight.shape[1]
    nbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _check(lib().xmk_int4_gemm_ws(_ptr(act), _ptr(qweight), _ptr(scales), _ptr(zeros), _ptr(bias),
                                  _ptr(out), ctypes.c_int64(m), ctypes.c_int64(k), ctypes.c_int64(n),
                                  ctypes.c_int64(group), _ptr(workspace), ctypes.c_size_t(nbytes),
                                  _stream(stream)))
    return out


def int4_dequant(qweight, scales, zeros, w_out, *, group=128, stream=None):
    k, n = qweight.shape[0] * 8, qweight.shape[1]
    _check(lib().xmk_int4_dequant(_ptr(qweight), _ptr(scales), _ptr(zeros), _ptr(w_out),
                                  ctypes.c_int64(k), ctypes.c_int64(n), ctypes.c_int64(group),
                                  _stream(stream)))
    return w_out


# ------------------------------------------------------------------------ fp8
def fp8_gemm(a, b, a_scale, b_scale, out, *, rhs_transpose=False, d_scale=None, bias=None, stream=None):
    """out = bf16(d_scale * (a_scale * b_scale * a b + bias)); d_scale / bias given: xmk_fp8_gemm_ex."""
    m, k = a.shape
    n = b.shape[0] if rhs_transpose else b.shape[1]
    if d_scale is None and bias is None:
        _check(lib().xmk_fp8_gemm(_ptr(a), _ptr(b), _ptr(a_scale), _ptr(b_scale), _ptr(out),
                                  ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k),
                                  ctypes.c_int32(int(rhs_transpose)), _stream(stream)))
    else:
        _check(lib().xmk_fp8_gemm_ex(_ptr(a), _ptr(b), _ptr(a_scale), _ptr(b_scale), _ptr(d_scale), _ptr(bias),
                                     _ptr(out), ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k),
                                     ctypes.c_int32(int(rhs_transpose)), _stream(stream)))
    return out


# ------------------------------------------------------------ GPT-J decode step
class Int4Linear(ctypes.Structure):
    """xmk_int4_linear."""
    _fields_ = [("qweight", ctypes.c_void_p), ("scales", ctypes.c_void_p), ("zeros", ctypes.c_void_p),
                ("bias", ctypes.c_void_p), ("k", ctypes.c_int64), ("n", ctypes.c_int64)]


class GptjLayer(ctypes.Structure):
    """xmk_gptj_layer."""
    _fields_ = [("ln_gamma", ctypes.c_void_p), ("ln_beta", ctypes.c_void_p), ("qkv", Int4Linear),
                ("out_proj", Int4Linear), ("fc_in", Int4Linear), ("fc_out", Int4Linear),
                ("k_cache", ctypes.c_void_p), ("v_cache", ctypes.c_void_p)]


class GptjConfig(ctypes.Structure):
    """xmk_gptj_config."""
    _fields_ = [(n, ctypes.c_int32) for n in ("n_layer", "n_head", "head_dim", "rotary_dim", "d_model",
                                              "d_ff", "vocab", "group", "batch", "cache_capacity")] + \
               [("ln_eps", ctypes.c_float)]


def int4_linear(qweight, scales, zeros, bias=None):
    return Int4Linear(qweight.data_ptr(), scales.data_ptr(), zeros.data_ptr(),
                      None if bias is None else bias.data_ptr(), qweight.shape[0] * 8, qweight.shape[1])


class GptjDecoder:
    """Holds the descriptor arrays of a GPT-J-shaped int4 model and runs decode steps.

    ``layers``: list of dicts with torch tensors ln_gamma, ln_beta, k_cache, v_cache and, for each
    of qkv / out_proj / fc_in / fc_out, a tuple (qweight, scales, zeros, bias-or-None).
    """

    def __init__(self, cfg, layers, lnf_gamma, lnf_beta, lm_head):
        self.cfg = cfg
        self._keep = (layers, lnf_gamma, lnf_beta, lm_head)  # keep the tensors alive
        arr = (GptjLayer * len(layers))()
        for i, L in enumerate(layers):
            arr[i] = GptjLayer(L["ln_gamma"].data_ptr(), L["ln_beta"].data_ptr(), int4_linear(*L["qkv"]),
                               int4_linear(*L["out_proj"]), int4_linear(*L["fc_in"]),
                               int4_linear(*L["fc_out"]), L["k_cache"].data_ptr(), L["v_cache"].data_ptr())
        self.layers = arr
        self.lnf = (lnf_gamma, lnf_beta)
        self.lm_head = int4_linear(*lm_head)
        lib().xmk_gptj_decode_workspace_bytes.restype = ctypes.c_size_t
        nbytes = lib().xmk_gptj_decode_workspace_bytes(ctypes.byref(cfg))
        if nbytes == 0:
            raise XmkError(INVALID_ARGUMENT, lib().xmk_last_error().decode())
        self.workspace = torch.empty((nbytes,), dtype=torch.uint8, device=lnf_gamma.device)

    def step(self, hidden_in, position, logits, stream=None):
        _check(lib().xmk_gptj_decode_step(ctypes.byref(self.cfg), self.layers, _ptr(self.lnf[0]),
                                          _ptr(self.lnf[1]), ctypes.byref(self.lm_head), _ptr(hidden_in),
                                          ctypes.c_int32(position), _ptr(logits), _ptr(self.workspace),
                                          ctypes.c_size_t(self.workspace.numel()), _stream(stream)))
        return logits
