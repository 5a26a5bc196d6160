"""GPU parity through the XLA-FFI handlers: call frames built by a fake host (ffi_util.FakeHost),
dispatched to the exported handlers, results against the oracle.  Operand order, in-place matrix
addend and attribute decoding follow the reference's handlers (sycl_custom_call.cc:154-205)."""
import ctypes as C
import os

import numpy as np
import pytest
import torch

import ffi_util as F
from util import to_dev

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def ffi():
    lib = C.CDLL(os.path.join(ROOT, "intel-extension-for-openxla_amd", "libxmk.so"))
    for name in ("xmk_ffi_cublas_gemm", "xmk_ffi_cublas_lt_matmul", "xmk_ffi_fmha_softmax",
                 "xmk_ffi_fmha_scale_bias_softmax", "xmk_ffi_int4_gemm", "xmk_ffi_cublas_lt_matmul_f8",
                 "xmk_ffi_fmha_softmax_backward", "xmk_ffi_fmha_scale_bias_softmax_backward"):
        getattr(lib, name).restype = C.c_void_p
        getattr(lib, name).argtypes = [C.POINTER(F.CallFrame)]
    return lib


def _host():
    return F.FakeHost(stream=torch.cuda.current_stream().cuda_stream)


def _buf(t, dtype):
    return (dtype, t.data_ptr(), list(t.shape))


def _ok(host, rc):
    assert rc is None, host.errors
    torch.cuda.synchronize()


def test_cublas_gemm_column_major_rhs(ffi, oracle):
    m, n, k = 192, 136, 264
    a = oracle.from_f32(oracle.normal((m, k), 1, 0.3), oracle.F16)
    b = oracle.from_f32(oracle.normal((n, k), 2, 0.3), oracle.F16)  # column-major [k,n]
    _, ref = oracle.gemm(a, b, oracle.F16, oracle.F16, rhs_t=True)
    da, db = to_dev(a, "f16"), to_dev(b, "f16")
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    host = _host()
    f = host.frame([_buf(da, F.F16), _buf(db, F.F16)], [_buf(out, F.F16)],
                   F.gemm_attrs(m, n, k, F.F16, F.F16, rhs_col_major=True))
    _ok(host, ffi.xmk_ffi_cublas_gemm(C.byref(f)))
    g, e = oracle.rel_err(out.float().cpu().numpy(), ref[0])
    assert g <= 1e-2 and e <= 1e-2, (g, e)


@pytest.mark.parametrize("epilogue,xepi", [(1, "EPI_BIAS"), (6, "EPI_BIAS_GELU"), (4, "EPI_GELU"), (3, "EPI_BIAS_RELU")])
def test_lt_matmul_epilogues(ffi, oracle, epilogue, xepi):
    m, n, k = 256, 320, 192
    a = oracle.from_f32(oracle.normal((m, k), 3, 0.2), oracle.BF16)
    b = oracle.from_f32(oracle.normal((k, n), 4, 0.2), oracle.BF16)
    bias = oracle.from_f32(oracle.normal((n,), 5, 0.5), oracle.BF16)
    has_bias = xepi.startswith("EPI_BIAS")
    _, ref = oracle.gemm(a, b, oracle.BF16, oracle.BF16, bias=bias if has_bias else None,
                         epilogue=getattr(oracle, xepi))
    da, db, dbias = to_dev(a, "bf16"), to_dev(b, "bf16"), to_dev(bias, "bf16")
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    host = _host()
    args = [_buf(da, F.BF16), _buf(db, F.BF16)] + ([_buf(dbias, F.BF16)] if has_bias else [])
    f = host.frame(args, [_buf(out, F.BF16)], F.gemm_attrs(m, n, k, F.BF16, F.BF16, epilogue=epilogue))
    _ok(host, ffi.xmk_ffi_cublas_lt_matmul(C.byref(f)))
    g, e = oracle.rel_err(out.float().cpu().numpy(), ref[0])
    assert g <= 1e-2 and e <= 1e-2, (g, e)


def test_lt_matmul_matrix_addend_in_place_with_bias(ffi, oracle):
    """beta != 0: operand 2 is the addend and the result, the vector bias moves to operand 3."""
    m, n, k = 128, 256, 128
    a = oracle.from_f32(oracle.normal((m, k), 6, 0.2), oracle.F16)
    b = oracle.from_f32(oracle.normal((k, n), 7, 0.2), oracle.F16)
    c = oracle.from_f32(oracle.normal((m, n), 8, 1.0), oracle.F16)
    bias = oracle.from_f32(oracle.normal((n,), 9, 0.5), oracle.F16)
    _, ref = oracle.gemm(a, b, oracle.F16, oracle.F16, c=c, bias=bias, beta=0.5, epilogue=oracle.EPI_BIAS)
    da, db, dc, dbias = (to_dev(x, "f16") for x in (a, b, c, bias))
    unused = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    host = _host()
    f = host.frame([_buf(da, F.F16), _buf(db, F.F16), _buf(dc, F.F16), _buf(dbias, F.F16)], [_buf(unused, F.F16)],
                   F.gemm_attrs(m, n, k, F.F16, F.F16, beta=0.5, epilogue=1))
    _ok(host, ffi.xmk_ffi_cublas_lt_matmul(C.byref(f)))
    g, e = oracle.rel_err(dc.float().cpu().numpy(), ref[0])
    assert g <= 1e-2 and e <= 1e-2, (g, e)
    assert float(unused.abs().max()) == 0.0


@pytest.mark.parametrize("with_bias,rank", [(False, 4), (True, 4), (False, 3)])
def test_fmha_handlers(ffi, oracle, with_bias, rank):
    B, N, Fq, T, H = (2 if rank == 4 else 1), 3, 200, 77, 64  # ragged T, as the reference's SD shapes
    q = oracle.from_f32(oracle.normal((B, N, Fq, H), 20, 1.0), oracle.BF16)
    k = oracle.from_f32(oracle.normal((B, N, T, H), 21, 1.0), oracle.BF16)
    v = oracle.from_f32(oracle.normal((B, N, T, H), 22, 1.0), oracle.BF16)
    bias = oracle.from_f32(oracle.normal((B, N, Fq, T), 23, 1.0), oracle.BF16) if with_bias else None
    scale = H ** -0.5
    _, ref, lse = oracle.fmha_fwd(q, k, v, oracle.BF16, scale, bias=bias, want_lse=True)
    shape = (lambda s: s if rank == 4 else s[1:])
    dq, dk, dv = (to_dev(x, "bf16").reshape(shape(x.shape)) for x in (q, k, v))
    out = torch.full(shape(q.shape), float("nan"), dtype=torch.bfloat16, device="cuda")
    act = torch.full(shape((B, N, Fq)), float("nan"), dtype=torch.float32, device="cuda")
    scratch = torch.empty((16,), dtype=torch.uint8, device="cuda")
    host = _host()
    args = [_buf(dq, F.BF16), _buf(dk, F.BF16), _buf(dv, F.BF16)]
    if with_bias:
        dbias = to_dev(bias, "bf16")
        args.append(_buf(dbias, F.BF16))
    f = host.frame(args, [_buf(out, F.BF16), _buf(scratch, 6), _buf(act, F.F32)],
                   {"fmha_scale": (F.F64, scale), "dropout_rate": (F.F64, 0.0)})
    handler = ffi.xmk_ffi_fmha_scale_bias_softmax if with_bias else ffi.xmk_ffi_fmha_softmax
    _ok(host, handler(C.byref(f)))
    g, e = oracle.rel_err(out.float().cpu().numpy().reshape(ref.shape), ref)
    assert g <= 1e-2 and e <= 1e-2, (g, e)
    assert np.abs(act.cpu().numpy().reshape(lse.shape) - lse).max() <= 2e-2


@pytest.mark.parametrize("with_bias", [False, True])
def test_fmha_backward_handlers(ffi, oracle, with_bias):
    """Forward handler (training call: writes the activation) then the backward handler on its results,
    gradients against the oracle's float64 closed form; the workspace comes from the fake host's
    allocator and goes back to it."""
    B, N, Fq, T, H = 2, 3, 136, 200, 64
    dt = oracle.BF16
    q = oracle.from_f32(oracle.normal((B, N, Fq, H), 30), dt)
    k = oracle.from_f32(oracle.normal((B, N, T, H), 31), dt)
    v = oracle.from_f32(oracle.normal((B, N, T, H), 32), dt)
    g = oracle.from_f32(oracle.normal((B, N, Fq, H), 33), dt)
    bias = oracle.from_f32(oracle.normal((B, N, Fq, T), 34), dt) if with_bias else None
    scale = H ** -0.5
    rq, rk, rv = oracle.fmha_bwd(q, k, v, g, dt, scale, bias=bias, causal=True)
    tq, tk, tv, tg = (to_dev(x, "bf16") for x in (q, k, v, g))
    tb = to_dev(bias, "bf16") if with_bias else None
    out = torch.empty_like(tq)
    act = torch.empty((B, N, Fq), dtype=torch.float32, device="cuda")
    scratch = torch.empty((16,), dtype=torch.uint8, device="cuda")
    attrs = {"fmha_scale": (F.F64, scale), "dropout_rate": (F.F64, 0.0), "is_causal_mask": (F.S32, 1)}
    host = _host()
    f = host.frame([_buf(tq, F.BF16), _buf(tk, F.BF16), _buf(tv, F.BF16)] + ([_buf(tb, F.BF16)] if with_bias else []),
                   [_buf(out, F.BF16), _buf(scratch, 6), _buf(act, F.F32)], attrs)
    _ok(host, (ffi.xmk_ffi_fmha_scale_bias_softmax if with_bias else ffi.xmk_ffi_fmha_softmax)(C.byref(f)))

    def allocator(size, alignment):
        t = torch.empty((size + alignment,), dtype=torch.uint8, device="cuda")
        return (t.data_ptr() + alignment - 1) // alignment * alignment, t
    dq, dk, dv = torch.empty_like(tq), torch.empty_like(tk), torch.empty_like(tv)
    host = F.FakeHost(stream=torch.cuda.current_stream().cuda_stream, allocator=allocator)
    f = host.frame([_buf(tq, F.BF16), _buf(tk, F.BF16), _buf(act, F.F32), _buf(tv, F.BF16), _buf(tg, F.BF16)]
                   + ([_buf(tb, F.BF16)] if with_bias else []) + [_buf(out, F.BF16)],
                   [_buf(dq, F.BF16), _buf(dk, F.BF16), _buf(dv, F.BF16), _buf(scratch, 6)], attrs)
    handler = ffi.xmk_ffi_fmha_scale_bias_softmax_backward if with_bias else ffi.xmk_ffi_fmha_softmax_backward
    _ok(host, handler(C.byref(f)))
    assert len(host.allocations) == 1 and host.freed == [host.allocations[0][0]]
    assert host.allocations[0][0] <= 2 * B * N * Fq * 4 + 512  # the fused kernels need rowsum(dO o O) only
    for name, got, ref in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        ge, ee = oracle.rel_err(got.float().cpu().numpy(), ref.astype(np.float32))
        assert ge <= 1e-2 and ee <= 8e-2, (name, ge, ee)
    # a host without an allocator cannot run the backward call
    host = _host()
    f = host.frame([_buf(tq, F.BF16), _buf(tk, F.BF16), _buf(act, F.F32), _buf(tv, F.BF16), _buf(tg, F.BF16)]
                   + ([_buf(tb, F.BF16)] if with_bias else []) + [_buf(out, F.BF16)],
                   [_buf(dq, F.BF16), _buf(dk, F.BF16), _buf(dv, F.BF16), _buf(scratch, 6)], attrs)
    assert handler(C.byref(f)) is not None and "scratch allocator" in host.errors[-1][1]


def test_fmha_scale_above_one_is_recomputed(ffi, oracle):
    """The reference replaces a scale attribute above 1 by 1/sqrt(H) (xetla_gpu_fused_mha_runner.cc:129)."""
    B, N, Fq, T, H = 1, 2, 64, 64, 64
    q, k, v = (oracle.from_f32(oracle.normal((B, N, Fq if i == 0 else T, H), 30 + i, 1.0), oracle.F16) for i in range(3))
    _, ref, _ = oracle.fmha_fwd(q, k, v, oracle.F16, H ** -0.5)
    dq, dk, dv = (to_dev(x, "f16") for x in (q, k, v))
    out = torch.empty(q.shape, dtype=torch.float16, device="cuda")
    scratch = torch.empty((16,), dtype=torch.uint8, device="cuda")
    host = _host()
    f = host.frame([_buf(dq, F.F16), _buf(dk, F.F16), _buf(dv, F.F16)], [_buf(out, F.F16), _buf(scratch, 6)],
                   {"fmha_scale": (F.F64, 8.0)})
    _ok(host, ffi.xmk_ffi_fmha_softmax(C.byref(f)))
    g, e = oracle.rel_err(out.float().cpu().numpy(), ref)
    assert g <= 1e-2 and e <= 1e-2, (g, e)


def test_int4_handler(ffi, oracle):
    m, k, n, group = 8, 512, 256, 128
    act = oracle.from_f32(oracle.normal((m, k), 40, 1.0), oracle.F16)
    qw = oracle.words((k // 8, n), 41)
    sc = oracle.from_f32(oracle.uniform((k // group, n), 42, 0.001, 0.02), oracle.F16)
    zp = oracle.from_f32(oracle.uniform((k // group, n), 43, 0.0, 15.0), oracle.F16)
    bias = oracle.from_f32(oracle.normal((n,), 44, 0.1), oracle.F16)
    _, ref = oracle.int4_gemm(act, qw, sc, zp, group, bias=bias)
    dact, dqw, dsc, dzp, dbias = to_dev(act, "f16"), to_dev(qw, "u32"), to_dev(sc, "f16"), to_dev(zp, "f16"), to_dev(bias, "f16")
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    host = _host()
    f = host.frame([_buf(dact, F.F16), _buf(dqw, F.S32), _buf(dsc, F.F16), _buf(dzp, F.F16), _buf(dbias, F.F16)],
                   [_buf(out, F.F16)], {})
    _ok(host, ffi.xmk_ffi_int4_gemm(C.byref(f)))
    g, e = oracle.rel_err(out.float().cpu().numpy(), ref)
    assert g <= 1e-2 and e <= 1e-2, (g, e)


def test_int4_handler_takes_scratch_for_many_rows(ffi, oracle):
    """256 rows: the handler asks the executor for K*N fp16 of scratch (dequantise once + dense GEMM) when the
    API table has an allocator, and streams the packed weights when it has none."""
    m, k, n, group = 256, 512, 256, 128
    act = oracle.from_f32(oracle.normal((m, k), 60, 1.0), oracle.F16)
    qw = oracle.words((k // 8, n), 61)
    sc = oracle.from_f32(oracle.uniform((k // group, n), 62, 0.001, 0.02), oracle.F16)
    zp = oracle.from_f32(oracle.uniform((k // group, n), 63, 0.0, 15.0), oracle.F16)
    _, ref = oracle.int4_gemm(act, qw, sc, zp, group)
    dact, dqw, dsc, dzp = to_dev(act, "f16"), to_dev(qw, "u32"), to_dev(sc, "f16"), to_dev(zp, "f16")

    def allocator(size, alignment):
        t = torch.empty((size + alignment,), dtype=torch.uint8, device="cuda")
        return (t.data_ptr() + alignment - 1) // alignment * alignment, t

    for alloc in (allocator, None):
        out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
        host = F.FakeHost(stream=torch.cuda.current_stream().cuda_stream, allocator=alloc)
        f = host.frame([_buf(dact, F.F16), _buf(dqw, F.S32), _buf(dsc, F.F16), _buf(dzp, F.F16)], [_buf(out, F.F16)], {})
        _ok(host, ffi.xmk_ffi_int4_gemm(C.byref(f)))
        if alloc:
            assert host.allocations == [(k * n * 2, 256)] and host.freed == [k * n * 2]
        else:
            assert host.allocations == []
        g, e = oracle.rel_err(out.float().cpu().numpy(), ref)
        assert g <= 1e-2 and e <= 1e-2, (alloc is not None, g, e)


def test_f8_matmul_handler(ffi, oracle):
    m, n, k = 320, 264, 208
    a, sa = oracle.fp8_quantize(oracle.normal((m, k), 50))
    b, sb = oracle.fp8_quantize(oracle.normal((n, k), 51))  # column-major [k,n]
    _, ref = oracle.fp8_gemm(a, b, sa, sb, rhs_t=True)
    da, db = to_dev(a, "f8"), to_dev(b, "f8")
    dsa, dsb = torch.tensor(float(sa), device="cuda"), torch.tensor(float(sb), device="cuda")
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    host = _host()
    f = host.frame([_buf(da, F.F8E4M3FN), _buf(db, F.F8E4M3FN), _buf(dsa, F.F32), _buf(dsb, F.F32)],
                   [_buf(out, F.BF16)], F.gemm_attrs(m, n, k, F.F8E4M3FN, F.BF16, rhs_col_major=True, epilogue=0))
    _ok(host, ffi.xmk_ffi_cublas_lt_matmul_f8(C.byref(f)))
    g, e = oracle.rel_err(out.float().cpu().numpy(), ref)
    assert g <= 5e-2 and e <= 5e-2, (g, e)


@pytest.mark.parametrize("with_bias", [False, True])
def test_f8_matmul_handler_applies_every_operand(ffi, oracle, with_bias):
    """(a, b, a_scale, b_scale, c_scale, d_scale [, bias]): out = bf16(d_scale * (a_scale b_scale A B + bias)).
    d_scale = 0.5 and a bias of the products' magnitude: dropping either operand misses the 5e-2 bound by far.
    Shapes cover the direct-to-LDS kernel (k % 16 == 0, n % 4 == 0) and the gathering one (k = 200)."""
    for (m, n, k) in ((320, 264, 208), (130, 76, 200)):
        a, sa = oracle.fp8_quantize(oracle.normal((m, k), 52))
        b, sb = oracle.fp8_quantize(oracle.normal((n, k), 53))  # column-major [k,n]
        bias = oracle.from_f32(oracle.normal((n,), 54, 10.0), oracle.BF16)
        _, prod = oracle.fp8_gemm(a, b, sa, sb, rhs_t=True)
        ref = np.float32(0.5) * (prod + (oracle.to_f32(bias, oracle.BF16)[None, :] if with_bias else np.float32(0)))
        da, db = to_dev(a, "f8"), to_dev(b, "f8")
        dsa, dsb = torch.tensor(float(sa), device="cuda"), torch.tensor(float(sb), device="cuda")
        dsc, dsd = torch.tensor(3.0, device="cuda"), torch.tensor(0.5, device="cuda")  # c_scale has no addend to scale
        dbias = to_dev(bias, "bf16")
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        host = _host()
        ops = [_buf(da, F.F8E4M3FN), _buf(db, F.F8E4M3FN), _buf(dsa, F.F32), _buf(dsb, F.F32), _buf(dsc, F.F32),
               _buf(dsd, F.F32)] + ([_buf(dbias, F.BF16)] if with_bias else [])
        f = host.frame(ops, [_buf(out, F.BF16)],
                       F.gemm_attrs(m, n, k, F.F8E4M3FN, F.BF16, rhs_col_major=True, epilogue=1 if with_bias else 0))
        _ok(host, ffi.xmk_ffi_cublas_lt_matmul_f8(C.byref(f)))
        g, e = oracle.rel_err(out.float().cpu().numpy(), ref)
        print(f"[parity] f8 handler {m}x{n}x{k} bias={with_bias}: g={g:.2e} e={e:.2e}")
        assert g <= 5e-2 and e <= 5e-2, (m, n, k, g, e)


def test_gemm_handler_takes_scratch_for_a_k_split(ffi, oracle):
    """A small-M product with a long reduction: with DeviceMemory_Allocate / Free in the API table the
    handler asks for exactly xmk_gemm_workspace_bytes of scratch, runs the K-split path and hands the
    scratch back; with a table that ends at Stream_Get it runs unsplit.  Same result either way."""
    m, n, k = 4, 4096, 16384
    a = oracle.from_f32(oracle.normal((m, k), 41, 0.05), oracle.BF16)
    b = oracle.from_f32(oracle.normal((n, k), 42, 0.05), oracle.BF16)
    _, ref = oracle.gemm(a, b, oracle.BF16, oracle.BF16, rhs_t=True)
    da, db = to_dev(a, "bf16"), to_dev(b, "bf16")

    def allocator(size, alignment):
        t = torch.empty((size + alignment,), dtype=torch.uint8, device="cuda")
        ptr = (t.data_ptr() + alignment - 1) // alignment * alignment
        return ptr, t

    outs = []
    for alloc in (allocator, None):
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        host = F.FakeHost(stream=torch.cuda.current_stream().cuda_stream, allocator=alloc)
        f = host.frame([_buf(da, F.BF16), _buf(db, F.BF16)], [_buf(out, F.BF16)],
                       F.gemm_attrs(m, n, k, F.BF16, F.BF16, rhs_col_major=True))
        _ok(host, ffi.xmk_ffi_cublas_gemm(C.byref(f)))
        if alloc:
            assert len(host.allocations) == 1 and host.allocations[0][0] > 0 and host.freed == [host.allocations[0][0]]
        else:
            assert host.allocations == []
        g, e = oracle.rel_err(out.float().cpu().numpy(), ref[0])
        assert g <= 1e-2 and e <= 1e-2, (g, e)
        outs.append(out)
    assert (outs[0].float() - outs[1].float()).abs().max().item() <= 2e-2
