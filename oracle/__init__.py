"""ctypes front end of the CPU oracle (``xmk_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke test and by the
benchmark's ``cpu_baseline`` leg as the checker.  The product package never
imports this module.

Arrays cross the boundary as numpy arrays holding raw bit patterns:
``uint16`` for bf16 / fp16, ``uint8`` for e4m3fn, ``float32`` for fp32.
"""
import ctypes
import os
import subprocess

import numpy as np

F16, F32, BF16, F8E4M3FN = 10, 11, 16, 20
EPI_DEFAULT, EPI_RELU, EPI_GELU, EPI_BIAS, EPI_BIAS_RELU, EPI_BIAS_GELU = range(6)

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libxmk_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (seconds)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


class _Matrix(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("transpose", ctypes.c_int32),
                ("num_rows", ctypes.c_int64), ("num_cols", ctypes.c_int64),
                ("batch_stride", ctypes.c_int64), ("leading_dim_stride", ctypes.c_int64)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.xo_f32_to_bf16.restype = ctypes.c_uint16
        _lib.xo_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.xo_f32_to_f16.restype = ctypes.c_uint16
        _lib.xo_f32_to_f16.argtypes = [ctypes.c_float]
        _lib.xo_f32_to_e4m3fn.restype = ctypes.c_uint8
        _lib.xo_f32_to_e4m3fn.argtypes = [ctypes.c_float]
        _lib.xo_bf16_to_f32.restype = ctypes.c_float
        _lib.xo_bf16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.xo_f16_to_f32.restype = ctypes.c_float
        _lib.xo_f16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.xo_e4m3fn_to_f32.restype = ctypes.c_float
        _lib.xo_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
    return _lib


def _p(a):
    return None if a is None else ctypes.c_void_p(a.ctypes.data)


_NP = {F16: np.uint16, BF16: np.uint16, F8E4M3FN: np.uint8, F32: np.float32}


def storage(dtype):
    """numpy dtype that holds the bit patterns of oracle dtype ``dtype``."""
    return _NP[dtype]


# ------------------------------------------------------------------ codecs
def from_f32(x, dtype):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=_NP[dtype])
    lib().xo_convert_from_f32(ctypes.c_int(dtype), _p(x), _p(out), ctypes.c_int64(x.size))
    return out


def to_f32(bits, dtype):
    bits = np.ascontiguousarray(bits, dtype=_NP[dtype])
    out = np.empty(bits.shape, dtype=np.float32)
    lib().xo_convert_to_f32(ctypes.c_int(dtype), _p(bits), _p(out), ctypes.c_int64(bits.size))
    return out


# ------------------------------------------------------------------ inputs
def normal(shape, seed, scale=1.0):
    out = np.empty(shape, dtype=np.float32)
    lib().xo_fill_normal(_p(out), ctypes.c_int64(out.size), ctypes.c_uint64(seed),
                         ctypes.c_float(scale))
    return out


def uniform(shape, seed, lo, hi):
    out = np.empty(shape, dtype=np.float32)
    lib().xo_fill_uniform(_p(out), ctypes.c_int64(out.size), ctypes.c_uint64(seed),
                          ctypes.c_float(lo), ctypes.c_float(hi))
    return out


def words(shape, seed):
    out = np.empty(shape, dtype=np.uint32)
    lib().xo_fill_words(_p(out), ctypes.c_int64(out.size), ctypes.c_uint64(seed))
    return out


# -------------------------------------------------------------------- GEMM
def _matrix(arr, transpose, rows, cols, batch_stride, ld):
    return _Matrix(arr.ctypes.data, int(transpose), rows, cols, batch_stride, ld)


def gemm(lhs, rhs, dtype_in, dtype_out, *, lhs_t=False, rhs_t=False, out_t=False, c=None,
         bias=None, alpha=1.0, beta=0.0, epilogue=EPI_DEFAULT, ld_out=None):
    """General GEMM oracle.  ``lhs``/``rhs`` are stored [batch?, rows, cols]
    bit-pattern arrays (rows x cols is the *stored* matrix; ``*_t`` marks the
    operand as the transpose of what is stored).  Returns (out_bits, out_f32):
    out_bits is the stored output ([n, m] when ``out_t``), out_f32 the
    unrounded logical [batch, m, n] result."""
    lhs = np.ascontiguousarray(lhs)
    rhs = np.ascontiguousarray(rhs)
    if lhs.ndim == 2:
        lhs = lhs[None]
    if rhs.ndim == 2:
        rhs = rhs[None]
    batch = lhs.shape[0]
    lr, lc = lhs.shape[1:]
    rr, rc = rhs.shape[1:]
    m = lc if lhs_t else lr
    n = rr if rhs_t else rc
    orows, ocols = (n, m) if out_t else (m, n)
    ld = ocols if ld_out is None else ld_out
    if c is not None:
        out = np.array(c, dtype=_NP[dtype_out], copy=True).reshape(batch, orows, ld)
        cbuf = out  # aliasing is allowed and exercised
    else:
        out = np.zeros((batch, orows, ld), dtype=_NP[dtype_out])
        cbuf = None
    out_f32 = np.empty((batch, m, n), dtype=np.float32)
    ml = _matrix(lhs, lhs_t, lr, lc, lr * lc, lc)
    mr = _matrix(rhs, rhs_t, rr, rc, rr * rc if rhs.shape[0] > 1 else 0, rc)
    mo = _matrix(out, out_t, orows, ocols, orows * ld, ld)
    rcode = lib().xo_gemm(ctypes.byref(ml), ctypes.byref(mr), ctypes.byref(mo), _p(out),
                          _p(cbuf), _p(bias), ctypes.c_int(dtype_in), ctypes.c_int(dtype_out),
                          ctypes.c_int64(batch), ctypes.c_float(alpha), ctypes.c_float(beta),
                          ctypes.c_int(epilogue), _p(out_f32))
    if rcode != 0:
        raise ValueError(f"xo_gemm status {rcode}")
    return out, out_f32


def gemm_packed(a, b, dtype_in, dtype_out, *, rhs_t=False, bias=None, epilogue=EPI_DEFAULT,
                scale=1.0, want_bits=True):
    """Fast packed row-major A[M,K] x B[K,N] (or B[N,K] with rhs_t)."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    m, k = a.shape
    n = b.shape[0] if rhs_t else b.shape[1]
    out = np.empty((m, n), dtype=_NP[dtype_out]) if want_bits else None
    out_f32 = np.empty((m, n), dtype=np.float32)
    rcode = lib().xo_gemm_packed(_p(a), _p(b), _p(bias), _p(out), _p(out_f32),
                                 ctypes.c_int(dtype_in), ctypes.c_int(dtype_out),
                                 ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k),
                                 ctypes.c_int(int(rhs_t)), ctypes.c_int(epilogue),
                                 ctypes.c_float(scale))
    if rcode != 0:
        raise ValueError(f"xo_gemm_packed status {rcode}")
    return out, out_f32


# -------------------------------------------------------------------- int4
def int4_dequant(qweight, scales, zeros, group):
    qweight = np.ascontiguousarray(qweight, dtype=np.uint32)
    k, n = qweight.shape[0] * 8, qweight.shape[1]
    out = np.empty((k, n), dtype=np.uint16)
    lib().xo_int4_dequant(_p(qweight), _p(scales), _p(zeros), _p(out), ctypes.c_int64(k),
                          ctypes.c_int64(n), ctypes.c_int64(group))
    return out


def int4_gemm(act, qweight, scales, zeros, group, bias=None, round_weights=False):
    """round_weights=False: the GEMM contract (fp32 dequantised weights); True: weights rounded
    to fp16 first, i.e. act @ int4_dequant(...)."""
    act = np.ascontiguousarray(act, dtype=np.uint16)
    qweight = np.ascontiguousarray(qweight, dtype=np.uint32)
    m, k = act.shape
    n = qweight.shape[1]
    out = np.empty((m, n), dtype=np.uint16)
    out_f32 = np.empty((m, n), dtype=np.float32)
    lib().xo_int4_gemm(_p(act), _p(qweight), _p(scales), _p(zeros), _p(bias), _p(out),
                       _p(out_f32), ctypes.c_int64(m), ctypes.c_int64(k), ctypes.c_int64(n),
                       ctypes.c_int64(group), ctypes.c_int(int(round_weights)))
    return out, out_f32


# --------------------------------------------------------------------- fp8
def fp8_quantize(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    q = np.empty(x.shape, dtype=np.uint8)
    scale = ctypes.c_float(0.0)
    lib().xo_fp8_quantize(_p(x), ctypes.c_int64(x.size), _p(q), ctypes.byref(scale))
    return q, np.float32(scale.value)


def fp8_gemm(a, b, a_scale, b_scale, rhs_t=False):
    m, k = a.shape
    n = b.shape[0] if rhs_t else b.shape[1]
    out = np.empty((m, n), dtype=np.uint16)
    out_f32 = np.empty((m, n), dtype=np.float32)
    lib().xo_fp8_gemm(_p(a), _p(b), ctypes.c_float(a_scale), ctypes.c_float(b_scale), _p(out),
                      _p(out_f32), ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k),
                      ctypes.c_int(int(rhs_t)))
    return out, out_f32


# --------------------------------------------------------------- attention
def fmha_fwd(q, k, v, dtype, scale, *, bias=None, causal=False, want_lse=False,
             first_unit=0, num_units=None, f_stride=1):
    """q [B,N,F,H], k/v [B,N,T,H] bit patterns.  Returns (out_bits, out_f32, lse);
    units outside [first_unit, first_unit+num_units) are left zero."""
    q = np.ascontiguousarray(q)
    k = np.ascontiguousarray(k)
    v = np.ascontiguousarray(v)
    B, N, F, H = q.shape
    T = k.shape[2]
    units = B * N
    if num_units is None:
        num_units = units - first_unit
    out = np.zeros(q.shape, dtype=_NP[dtype])
    out_f32 = np.zeros(q.shape, dtype=np.float32)
    lse = np.zeros((units, F), dtype=np.float32) if want_lse else None
    lib().xo_fmha_fwd(ctypes.c_int(dtype), _p(q), _p(k), _p(v), _p(bias), _p(out), _p(out_f32),
                      _p(lse), ctypes.c_int64(num_units), ctypes.c_int64(first_unit),
                      ctypes.c_int64(H), ctypes.c_int64(F), ctypes.c_int64(T),
                      ctypes.c_int64(T * H), ctypes.c_float(scale), ctypes.c_int(int(causal)),
                      ctypes.c_int64(f_stride))
    return out, out_f32, lse


def fmha_fwd_online(q, k, v, dtype, scale, *, bias=None, causal=False, kBc=128):
    q = np.ascontiguousarray(q)
    B, N, F, H = q.shape
    T = k.shape[2]
    out_f32 = np.zeros(q.shape, dtype=np.float32)
    lib().xo_fmha_fwd_online(ctypes.c_int(dtype), _p(q), _p(np.ascontiguousarray(k)),
                             _p(np.ascontiguousarray(v)), _p(bias), _p(out_f32),
                             ctypes.c_int64(B * N), ctypes.c_int64(H), ctypes.c_int64(F),
                             ctypes.c_int64(T), ctypes.c_float(scale), ctypes.c_int(int(causal)),
                             ctypes.c_int64(kBc))
    return out_f32


def fmha_bwd(q, k, v, d_out, dtype, scale, *, bias=None, causal=False):
    """Gradients of softmax(scale q k^T + bias + mask) v with respect to q, k, v, in float64 from the
    rounded inputs (numpy; for test sizes).  The closed form the reference's backward kernel follows
    (xetla/sdp/fmha_backward.h): P = softmax(S); dV = P^T dO; dP = dO V^T;
    dS = P o (dP - rowsum(dP o P)); dQ = scale dS K; dK = scale dS^T Q.  Returns (dq, dk, dv) float64."""
    qf, kf, vf, gf = (to_f32(x, dtype).astype(np.float64) for x in (q, k, v, d_out))
    s = scale * np.einsum("bnfh,bnth->bnft", qf, kf)
    if bias is not None:
        s = s + to_f32(bias, dtype).astype(np.float64)
    F, T = s.shape[-2:]
    if causal:
        s = np.where(np.arange(T)[None, :] > np.arange(F)[:, None], -np.inf, s)
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    p /= p.sum(axis=-1, keepdims=True)
    dv = np.einsum("bnft,bnfh->bnth", p, gf)
    dp = np.einsum("bnfh,bnth->bnft", gf, vf)
    ds = p * (dp - (dp * p).sum(axis=-1, keepdims=True))
    dq = scale * np.einsum("bnft,bnth->bnfh", ds, kf)
    dk = scale * np.einsum("bnft,bnfh->bnth", ds, qf)
    return dq, dk, dv


def num_threads():
    return int(lib().xo_num_threads())


# ------------------------------------------------------------- error metrics
def rel_err(x, ref, label=None):
    """Two readings of "max relative error" against the fp32 recompute ``ref``:
    g = max|x-ref| / max|ref|                    (error relative to the tensor's scale)
    e = max |x-ref| / (|ref| + rms(ref))         (elementwise; the rms term keeps outputs that
        cancel to ~0 from dividing rounding noise by ~0: it is allclose with rtol = tol and
        atol = tol * rms(ref)).
    With ``label`` a line with both, and with the stricter elementwise reading
    max |x-ref| / (|ref| + 1e-2 rms(ref)), is printed (pytest -s shows it): the strict figure is
    reported, not enforced: a 16-bit result of a sum that cancels to 1e-2 rms carries rounding
    noise of the terms, not of the result."""
    x = np.asarray(x, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    d = np.abs(x - ref)
    g = d.max() / max(np.abs(ref).max(), 1e-30)
    eps = max(np.sqrt(np.mean(ref * ref)), 1e-30)
    e = (d / (np.abs(ref) + eps)).max()
    if label is not None:
        strict = (d / (np.abs(ref) + 1e-2 * eps)).max()
        print(f"[parity] {label}: max|d|/max|ref| = {g:.3e}; elementwise eps=rms(ref) (enforced) = {e:.3e}; "
              f"eps=1e-2*rms(ref) (reported) = {strict:.3e}", flush=True)
    return float(g), float(e)


def cond_err(x, ref, cond):
    """max |x-ref| / cond, elementwise, where ``cond`` is the sum of the absolute values of the terms
    each output is the sum of (for attention: softmax(S) |V|).  This is the componentwise relative
    error of numerical analysis: rounding one operand of a dot product to p bits perturbs the result
    by up to 2^-p of that sum, however far the terms cancel."""
    x = np.asarray(x, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    cond = np.maximum(np.asarray(cond, dtype=np.float64), 1e-30)
    return float((np.abs(x - ref) / cond).max())
