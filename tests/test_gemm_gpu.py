"""GPU parity: bf16/fp16 GEMM with fused epilogue through the C ABI (xmk_gemm), against the oracle.

Tolerance (the tolerance stated for this path): max relative error <= 1e-2 for bf16/fp16 outputs against an
fp32 recompute from the same rounded inputs; both normalisations of oracle.rel_err are held to it.
"""
import numpy as np
import pytest
import torch

from util import to_bits, to_dev

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _kind(dt, oracle):
    return "bf16" if dt == oracle.BF16 else "f16"


def _check(oracle, got_f32, ref_f32, tol=TOL):
    g, e = oracle.rel_err(got_f32, ref_f32)
    assert g <= tol and e <= tol, (g, e)
    return g, e


def test_config1_bf16_bias(xmk, oracle):
    """benchmark configuration 1: C[512,4096] = A[512,4096] B[4096,4096] + bias, N(0,1)/sqrt(K) inputs."""
    m, k, n = 512, 4096, 4096
    sc = k ** -0.5
    a = oracle.from_f32(oracle.normal((m, k), 1, sc), oracle.BF16)
    b = oracle.from_f32(oracle.normal((k, n), 2, sc), oracle.BF16)
    bias = oracle.from_f32(oracle.normal((n,), 3, sc), oracle.BF16)
    _, ref = oracle.gemm_packed(a, b, oracle.BF16, oracle.BF16, bias=bias, epilogue=oracle.EPI_BIAS)
    out = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    xmk.run_gemm(to_dev(a, "bf16"), to_dev(b, "bf16"), out, bias=to_dev(bias, "bf16"),
                 epilogue=xmk.EPI_BIAS)
    torch.cuda.synchronize()
    g, e = _check(oracle, out.float().cpu().numpy(), ref)
    print(f"config1: global {g:.2e} elementwise {e:.2e}")


@pytest.mark.parametrize("dt_name", ["BF16", "F16"])
@pytest.mark.parametrize("lhs_t,rhs_t,out_t", [(0, 0, 0), (0, 1, 0), (1, 0, 0), (1, 1, 0), (0, 0, 1), (1, 0, 1)])
@pytest.mark.parametrize("m,n,k", [(96, 136, 200), (300, 264, 72), (256, 256, 64)])
def test_layouts(xmk, oracle, dt_name, lhs_t, rhs_t, out_t, m, n, k):
    """Row/column-major operands and output (MakeBlasGemmCompatible), ragged tiles, K tails."""
    dt = getattr(oracle, dt_name)
    kind = _kind(dt, oracle)
    a = oracle.from_f32(oracle.normal((k, m) if lhs_t else (m, k), 10, 0.3), dt)
    b = oracle.from_f32(oracle.normal((n, k) if rhs_t else (k, n), 11, 0.3), dt)
    ref_bits, ref = oracle.gemm(a, b, dt, dt, lhs_t=lhs_t, rhs_t=rhs_t, out_t=out_t)
    tdt = torch.bfloat16 if kind == "bf16" else torch.float16
    out = torch.full((n, m) if out_t else (m, n), float("nan"), dtype=tdt, device="cuda")
    xmk.run_gemm(to_dev(a, kind), to_dev(b, kind), out, lhs_transpose=lhs_t, rhs_transpose=rhs_t,
                 out_transpose=out_t)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    _check(oracle, got.T if out_t else got, ref[0])


@pytest.mark.parametrize("dt_name", ["BF16", "F16"])
@pytest.mark.parametrize("lhs_t,rhs_t", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(2048, 4096, 200), (1800, 4000, 136)])
def test_tile_256x128(xmk, oracle, dt_name, lhs_t, rhs_t, m, n, k):
    """Shapes whose 256x128 tiles number about one per CU take that tile (K step 64, three stages):
    every operand layout, a K tail, and tiles that hang over the last rows and columns."""
    assert xmk.gemm_policy_name(m, n, k, rhs_transpose=bool(rhs_t)) == "mfma_256x128x64_w2x2_s3"
    dt = getattr(oracle, dt_name)
    kind = _kind(dt, oracle)
    a = oracle.from_f32(oracle.normal((k, m) if lhs_t else (m, k), 12, 0.3), dt)
    b = oracle.from_f32(oracle.normal((n, k) if rhs_t else (k, n), 13, 0.3), dt)
    bias = oracle.from_f32(oracle.normal((n,), 14, 0.5), dt)
    _, ref = oracle.gemm(a, b, dt, dt, lhs_t=lhs_t, rhs_t=rhs_t, bias=bias, epilogue=oracle.EPI_BIAS)
    tdt = torch.bfloat16 if kind == "bf16" else torch.float16
    out = torch.full((m, n), float("nan"), dtype=tdt, device="cuda")
    xmk.run_gemm(to_dev(a, kind), to_dev(b, kind), out, lhs_transpose=lhs_t, rhs_transpose=rhs_t,
                 bias=to_dev(bias, kind), epilogue=xmk.EPI_BIAS)
    torch.cuda.synchronize()
    _check(oracle, out.float().cpu().numpy(), ref[0])


@pytest.mark.parametrize("epi", ["DEFAULT", "RELU", "GELU", "BIAS", "BIAS_RELU", "BIAS_GELU"])
@pytest.mark.parametrize("beta", [0.0, 1.0, 0.5])
def test_epilogues(xmk, oracle, epi, beta):
    """out = act(A.B + beta*C + bias) with C aliasing the output (sycl_custom_call.cc:191-195)."""
    dt = oracle.BF16
    m, n, k = 200, 328, 256
    a = oracle.from_f32(oracle.normal((m, k), 20, 0.2), dt)
    b = oracle.from_f32(oracle.normal((k, n), 21, 0.2), dt)
    bias = oracle.from_f32(oracle.normal((n,), 22), dt)
    c = oracle.from_f32(oracle.normal((m, n), 23), dt)
    code = getattr(oracle, "EPI_" + epi)
    _, ref = oracle.gemm(a, b, dt, dt, bias=bias, c=c if beta else None, beta=beta, epilogue=code)
    out = to_dev(c, "bf16") if beta else torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    xmk.run_gemm(to_dev(a, "bf16"), to_dev(b, "bf16"), out, c=out if beta else None,
                 bias=to_dev(bias, "bf16") if "BIAS" in epi else None, beta=beta,
                 epilogue=getattr(xmk, "EPI_" + epi))
    torch.cuda.synchronize()
    _check(oracle, out.float().cpu().numpy(), ref[0])


def test_identity_is_bit_exact(xmk, oracle):
    dt = oracle.BF16
    m, k = 320, 256
    a = oracle.from_f32(oracle.normal((m, k), 30), dt)
    eye = to_dev(oracle.from_f32(np.eye(k, dtype=np.float32), dt), "bf16")
    out = torch.empty((m, k), dtype=torch.bfloat16, device="cuda")
    xmk.run_gemm(to_dev(a, "bf16"), eye, out)
    torch.cuda.synchronize()
    assert np.array_equal(to_bits(out), a)


@pytest.mark.parametrize("dt_name", ["BF16", "F16"])
@pytest.mark.parametrize("shape", [(1, 256, 128, 8), (1, 1024, 64, 128)])
def test_reference_gemm_ut_shapes(xmk, oracle, dt_name, shape):
    """Shapes of the reference's gemm_ut (test/jax_ut.patch:505-518): B column-major, GELU epilogue."""
    _, m, k, n = shape
    dt = getattr(oracle, dt_name)
    kind = _kind(dt, oracle)
    a = oracle.from_f32(oracle.normal((m, k), 40, 0.1), dt)
    bt = oracle.from_f32(oracle.normal((n, k), 41, 0.1), dt)
    _, ref = oracle.gemm(a, bt, dt, dt, rhs_t=True, epilogue=oracle.EPI_GELU)
    out = torch.empty((m, n), dtype=torch.bfloat16 if kind == "bf16" else torch.float16, device="cuda")
    xmk.run_gemm(to_dev(a, kind), to_dev(bt, kind), out, rhs_transpose=True, epilogue=xmk.EPI_GELU)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    _check(oracle, got, ref[0])
    if dt == oracle.F16:  # the reference's own bound for fp16 (test/jax_ut.patch:614)
        assert np.abs(got - ref[0]).max() < 1e-3


def test_batched_f32_out_and_strides(xmk, oracle):
    dt = oracle.F16
    bsz, m, n, k = 3, 72, 88, 128
    a = oracle.from_f32(oracle.normal((bsz, m, k), 50, 0.2), dt)
    b = oracle.from_f32(oracle.normal((bsz, k, n), 51, 0.2), dt)
    _, ref = oracle.gemm(a, b, dt, oracle.F32)
    out = torch.empty((bsz, m, n), dtype=torch.float32, device="cuda")
    xmk.run_gemm(to_dev(a, "f16"), to_dev(b, "f16"), out)
    torch.cuda.synchronize()
    _check(oracle, out.cpu().numpy(), ref, tol=1e-4)  # fp32 output: accumulation-order noise only
    # padded leading dimensions: views into wider buffers
    ap = torch.zeros((m, k + 24), dtype=torch.float16, device="cuda")
    bp = torch.zeros((k, n + 40), dtype=torch.float16, device="cuda")
    op = torch.full((m, n + 8), 7.0, dtype=torch.float16, device="cuda")
    ap[:, :k] = to_dev(a[0], "f16")
    bp[:, :n] = to_dev(b[0], "f16")
    xmk.run_gemm(ap[:, :k], bp[:, :n], op[:, :n])
    torch.cuda.synchronize()
    _check(oracle, op[:, :n].float().cpu().numpy(), ref[0])
    assert (op[:, n:] == 7.0).all()  # nothing written outside the logical matrix


def test_generic_path(xmk, oracle):
    """Shapes and types the MFMA kernel does not take: K % 8 != 0, fp32, s8 -> s32."""
    dt = oracle.BF16
    m, n, k = 37, 50, 45
    a = oracle.from_f32(oracle.normal((m, k), 60, 0.3), dt)
    b = oracle.from_f32(oracle.normal((k, n), 61, 0.3), dt)
    bias = oracle.from_f32(oracle.normal((n,), 62), dt)
    _, ref = oracle.gemm(a, b, dt, dt, bias=bias, epilogue=oracle.EPI_BIAS_GELU)
    out = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    assert xmk.gemm_policy_name(m, n, k, dtype_in=xmk.F32, dtype_out=xmk.F32) == "mfma_f32_128x128x16"
    assert xmk.gemm_policy_name(m, n, k, dtype_in=xmk.S8, dtype_out=xmk.S32) == "mfma_s8_128x128x64"
    xmk.run_gemm(to_dev(a, "bf16"), to_dev(b, "bf16"), out, bias=to_dev(bias, "bf16"),
                 epilogue=xmk.EPI_BIAS_GELU)
    torch.cuda.synchronize()
    _check(oracle, out.float().cpu().numpy(), ref[0])
    af, bf = oracle.normal((m, k), 63), oracle.normal((n, k), 64)
    outf = torch.empty((m, n), dtype=torch.float32, device="cuda")
    xmk.run_gemm(to_dev(af, "f32"), to_dev(bf, "f32"), outf, rhs_transpose=True)
    torch.cuda.synchronize()
    assert np.allclose(outf.cpu().numpy(), af.astype(np.float64) @ bf.T.astype(np.float64), rtol=1e-4, atol=1e-4)
    ai = torch.randint(-128, 128, (m, k), dtype=torch.int8, device="cuda")
    bi = torch.randint(-128, 128, (k, n), dtype=torch.int8, device="cuda")
    oi = torch.empty((m, n), dtype=torch.int32, device="cuda")
    xmk.run_gemm(ai, bi, oi)
    torch.cuda.synchronize()
    assert torch.equal(oi.cpu(), ai.cpu().int() @ bi.cpu().int())  # integer path: bit exact


@pytest.mark.parametrize("rhs_t", [False, True])
def test_full_size_8192_sampled_rows(xmk, oracle, rhs_t):
    """The 8192^3 shape of the north-star target: one output row per 512 against the oracle, each at a
    different place of its 256-row tile and of a wave's 32-row slab."""
    n = 8192
    sc = n ** -0.5
    a = oracle.from_f32(oracle.normal((n, n), 70, sc), oracle.BF16)
    b = oracle.from_f32(oracle.normal((n, n), 71, sc), oracle.BF16)
    out = torch.empty((n, n), dtype=torch.bfloat16, device="cuda")
    xmk.run_gemm(to_dev(a, "bf16"), to_dev(b, "bf16"), out, rhs_transpose=rhs_t)
    torch.cuda.synchronize()
    rows = np.array([(5 + 37 * i) % 256 + 512 * i for i in range(n // 512)])
    _, ref = oracle.gemm_packed(a[rows], b, oracle.BF16, oracle.BF16, rhs_t=rhs_t)
    _check(oracle, out[torch.from_numpy(rows).cuda()].float().cpu().numpy(), ref)
    # checksum of checksums: sum of every output row equals A @ rowsum(B) (linearity), fp64 on host
    bs = oracle.to_f32(b, oracle.BF16).astype(np.float64)
    colsum = bs.sum(axis=0 if rhs_t else 1)
    expect = oracle.to_f32(a, oracle.BF16).astype(np.float64) @ colsum
    got = out.double().sum(dim=1).cpu().numpy()
    # a row sum adds 8192 bf16 roundings of elements near 0.011: about 2e-3 in all
    assert np.abs(got - expect).max() <= 1e-2 * np.abs(expect).max() + 0.02


def test_errors(xmk):
    a = torch.zeros((16, 32), dtype=torch.bfloat16, device="cuda")
    b = torch.zeros((32, 16), dtype=torch.bfloat16, device="cuda")
    out = torch.zeros((16, 16), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(xmk.XmkError) as e:
        xmk.run_gemm(a, b, out, epilogue=xmk.EPI_GELU_AUX)
    assert e.value.code == xmk.UNIMPLEMENTED and "Unsupported Activation mode" in e.value.message
    with pytest.raises(xmk.XmkError) as e:
        xmk.run_gemm(a, b, out, epilogue=xmk.EPI_BIAS)  # bias missing
    assert e.value.code == xmk.INVALID_ARGUMENT
    with pytest.raises(xmk.XmkError) as e:
        xmk.run_gemm(a, a, out)  # reduction sizes differ
    assert e.value.code == xmk.INVALID_ARGUMENT
    with pytest.raises(xmk.XmkError) as e:
        xmk.run_gemm(a, b, out.float().half())  # bf16 x bf16 -> f16 is not an accepted triple
    assert e.value.code == xmk.INTERNAL


@pytest.mark.parametrize("dt_name", ["BF16", "F16"])
@pytest.mark.parametrize("m,n,k,rhs_t,with_bias", [(4, 4096, 4096, False, False), (200, 264, 136, True, True),
                                                   (512, 1024, 256, False, True), (33, 72, 100, False, False)])
def test_qkv_fused_gemm(xmk, oracle, dt_name, m, n, k, rhs_t, with_bias):
    """Three products sharing A in one launch (the reference's hgemm_qkv / hgemm_qkv_bias; its own
    check is example/qkv_fusion/test_qkv_fusion.py: m=4, k=n=4096 fp16, fused vs separate)."""
    dt = getattr(oracle, dt_name)
    kind = _kind(dt, oracle)
    tdt = torch.bfloat16 if kind == "bf16" else torch.float16
    a = oracle.from_f32(oracle.normal((m, k), 70, k ** -0.5), dt)
    w = oracle.from_f32(oracle.normal((3, n, k) if rhs_t else (3, k, n), 71, 1.0), dt)
    bias = oracle.from_f32(oracle.normal((3, n), 72, 0.5), dt) if with_bias else None
    outs = [torch.full((m, n), float("nan"), dtype=tdt, device="cuda") for _ in range(3)]
    xmk.run_gemm_qkv(to_dev(a, kind), to_dev(w, kind), *outs, rhs_transpose=rhs_t,
                     bias=None if bias is None else to_dev(bias, kind),
                     epilogue=xmk.EPI_BIAS if with_bias else xmk.EPI_DEFAULT)
    torch.cuda.synchronize()
    for i in range(3):
        _, ref = oracle.gemm(a, w[i], dt, dt, rhs_t=rhs_t, bias=None if bias is None else bias[i],
                             epilogue=oracle.EPI_BIAS if with_bias else oracle.EPI_DEFAULT)
        _check(oracle, outs[i].float().cpu().numpy(), ref[0])
    # fused == separate, bit for bit (same kernel, same tile order)
    sep = torch.empty((m, n), dtype=tdt, device="cuda")
    xmk.run_gemm(to_dev(a, kind), to_dev(w[1], kind), sep, rhs_transpose=rhs_t,
                 bias=None if bias is None else to_dev(bias[1], kind),
                 epilogue=xmk.EPI_BIAS if with_bias else xmk.EPI_DEFAULT)
    torch.cuda.synchronize()
    assert torch.equal(sep.view(torch.int16), outs[1].view(torch.int16))


@pytest.mark.parametrize("dt_name", ["BF16", "F16"])
@pytest.mark.parametrize("m,n,k,rhs_t,epi", [(1, 4096, 4096, False, "EPI_DEFAULT"), (4, 4096, 16384, True, "EPI_BIAS_GELU"),
                                             (16, 1024, 8192, False, "EPI_BIAS"), (3, 520, 2048, True, "EPI_RELU")])
def test_split_k_with_workspace(xmk, oracle, dt_name, m, n, k, rhs_t, epi):
    """Small-M decode shapes: K split over work-groups into caller scratch, second pass applies
    the epilogue (beta * C included)."""
    dt = getattr(oracle, dt_name)
    kind = _kind(dt, oracle)
    tdt = torch.bfloat16 if kind == "bf16" else torch.float16
    a = oracle.from_f32(oracle.normal((m, k), 80, k ** -0.5), dt)
    b = oracle.from_f32(oracle.normal((n, k) if rhs_t else (k, n), 81, 1.0), dt)
    c = oracle.from_f32(oracle.normal((m, n), 82, 1.0), dt)
    bias = oracle.from_f32(oracle.normal((n,), 83, 0.5), dt) if "BIAS" in epi else None
    _, ref = oracle.gemm(a, b, dt, dt, rhs_t=rhs_t, c=c, bias=bias, beta=0.5, epilogue=getattr(oracle, epi))
    da, db, dc = to_dev(a, kind), to_dev(b, kind), to_dev(c, kind)
    nbytes = xmk.gemm_workspace_bytes(da, db, dc, rhs_transpose=rhs_t)
    assert nbytes > 0, "these shapes are meant to split"
    ws = torch.empty((nbytes,), dtype=torch.uint8, device="cuda")
    xmk.run_gemm(da, db, dc, rhs_transpose=rhs_t, c=dc, beta=0.5, bias=None if bias is None else to_dev(bias, kind),
                 epilogue=getattr(xmk, epi), workspace=ws)
    torch.cuda.synchronize()
    _check(oracle, dc.float().cpu().numpy(), ref[0])
    # a large-M shape does not ask for scratch
    big = torch.empty((2048, 4096), dtype=tdt, device="cuda")
    w = torch.empty((4096, 4096), dtype=tdt, device="cuda")
    assert xmk.gemm_workspace_bytes(big, w, big) == 0


@pytest.mark.parametrize("m,rhs_t", [(1, False), (4, False), (4, True), (32, False)])
def test_vocabulary_projection_n50400(xmk, oracle, m, rhs_t):
    """The decode rows of the reference's tile table against a vocabulary of 50400 columns
    (`1_50400_4096`, `4_50400_4096`, xla/service/gpu/xetla/gemm/gemm.cc:77-80): 50400 = 787.5 x 64, so the
    last tile of every policy is ragged.  With and without caller scratch (the K-split and the unsplit
    path), fp16 like the reference's decode."""
    n, k = 50400, 4096
    dt, kind = oracle.F16, "f16"
    # one to eight rows stream the matrix (either storage order); the others take a matrix-core tile
    streamed = xmk.gemm_policy_name(m, n, k, rhs_t, xmk.F16, xmk.F16) == "stream_rows_8x512_w8"
    assert streamed == (m <= 8)
    a = oracle.from_f32(oracle.normal((m, k), 84, k ** -0.5), dt)
    b = oracle.from_f32(oracle.normal((n, k) if rhs_t else (k, n), 85, 1.0), dt)
    bias = oracle.from_f32(oracle.normal((n,), 86, 0.5), dt)
    _, ref = oracle.gemm(a, b, dt, dt, rhs_t=rhs_t, bias=bias, epilogue=oracle.EPI_BIAS)
    da, db, dbias = to_dev(a, kind), to_dev(b, kind), to_dev(bias, kind)
    for with_ws in (False, True):
        out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
        nbytes = xmk.gemm_workspace_bytes(da, db, out, rhs_transpose=rhs_t)
        ws = torch.empty((max(nbytes, 16),), dtype=torch.uint8, device="cuda") if with_ws else None
        xmk.run_gemm(da, db, out, rhs_transpose=rhs_t, bias=dbias, epilogue=xmk.EPI_BIAS, workspace=ws)
        torch.cuda.synchronize()
        _check(oracle, out.float().cpu().numpy(), ref[0])


@pytest.mark.parametrize("dt_name", ["BF16", "F16"])
@pytest.mark.parametrize("m,n,k,epi,beta", [
    (1, 16384, 4096, "EPI_DEFAULT", 0.0),   # `1_16384_4096`, xla/service/gpu/xetla/gemm/gemm.cc:33
    (4, 4096, 16384, "EPI_BIAS", 0.5),      # `4_4096_16384`, gemm.cc:44
    (8, 1032, 72, "EPI_BIAS_GELU", 0.0),    # columns ragged in the third block; nine batches of rows: a wave with two, seven with one
    (3, 520, 8, "EPI_RELU", 1.0),           # one batch of rows: seven waves have nothing to add
    (5, 8, 264, "EPI_BIAS_RELU", 0.0),      # one lane's worth of columns
    (2, 33000, 512, "EPI_GELU", 0.0),       # enough column blocks to be chosen without being forced
    (7, 2048, 1000, "EPI_DEFAULT", 0.0),
    (6, 1088, 5000, "EPI_BIAS", 0.0),       # [N, K] storage: two loads per row and wave, the second partly past K
])
@pytest.mark.parametrize("with_ws", [False, True])
@pytest.mark.parametrize("rhs_t", [False, True])
def test_streamed_rows(xmk, oracle, monkeypatch, dt_name, m, n, k, epi, beta, with_ws, rhs_t):
    """One to eight rows against a [K, N] or an [N, K] matrix on the streaming kernels (policy 5; forced here,
    since the smaller shapes would take a matrix-core tile), unsplit and K-split into caller scratch."""
    monkeypatch.setenv("XMK_GEMM_POLICY", "5")
    dt = getattr(oracle, dt_name)
    kind = _kind(dt, oracle)
    a = oracle.from_f32(oracle.normal((m, k), 90, k ** -0.5), dt)
    b = oracle.from_f32(oracle.normal((n, k) if rhs_t else (k, n), 91, 1.0), dt)
    c = oracle.from_f32(oracle.normal((m, n), 92, 1.0), dt)
    bias = oracle.from_f32(oracle.normal((n,), 93, 0.5), dt) if "BIAS" in epi else None
    _, ref = oracle.gemm(a, b, dt, dt, rhs_t=rhs_t, c=c, bias=bias, beta=beta, epilogue=getattr(oracle, epi))
    assert xmk.gemm_policy_name(m, n, k, rhs_t, getattr(xmk, dt_name), getattr(xmk, dt_name)) == "stream_rows_8x512_w8"
    da, db, dc = to_dev(a, kind), to_dev(b, kind), to_dev(c, kind)
    ws = None
    if with_ws:
        nbytes = xmk.gemm_workspace_bytes(da, db, dc, rhs_transpose=rhs_t)
        ws = torch.empty((max(nbytes, 16),), dtype=torch.uint8, device="cuda")
    xmk.run_gemm(da, db, dc, rhs_transpose=rhs_t, c=dc, beta=beta, bias=None if bias is None else to_dev(bias, kind),
                 epilogue=getattr(xmk, epi), workspace=ws)
    torch.cuda.synchronize()
    _check(oracle, dc.float().cpu().numpy(), ref[0])


@pytest.mark.parametrize("rhs_t", [False, True])
def test_streamed_rows_batched_f32_out(xmk, oracle, monkeypatch, rhs_t):
    """The streaming kernels with a batch, fp32 output and padded leading dimensions."""
    monkeypatch.setenv("XMK_GEMM_POLICY", "5")
    bsz, m, n, k, lda, ldc = 3, 4, 1000, 136, 144, 1004
    ldb = 152 if rhs_t else 1008  # stored [n, k] or [k, n]
    brows = n if rhs_t else k
    dt, kind = oracle.BF16, "bf16"
    a = oracle.from_f32(oracle.normal((bsz, m, lda), 94, k ** -0.5), dt)
    b = oracle.from_f32(oracle.normal((bsz, brows, ldb), 95, 1.0), dt)
    da, db = to_dev(a, kind), to_dev(b, kind)
    out = torch.full((bsz, m, ldc), -7.0, dtype=torch.float32, device="cuda")
    rhs = xmk.Matrix(db.data_ptr(), 1, n, k, n * ldb, ldb) if rhs_t else xmk.Matrix(db.data_ptr(), 0, k, n, k * ldb, ldb)
    d = xmk.GemmDesc(xmk.Matrix(da.data_ptr(), 0, m, k, m * lda, lda), rhs,
                     xmk.Matrix(out.data_ptr(), 0, m, n, m * ldc, ldc), None, None, xmk.BF16, xmk.F32, bsz, 2.0, 0.0,
                     xmk.EPI_DEFAULT)
    xmk.run_gemm_desc(d)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    af, bf = oracle.to_f32(a, dt), oracle.to_f32(b, dt)
    for z in range(bsz):
        bz = bf[z, :n, :k].T if rhs_t else bf[z, :k, :n]
        ref = 2.0 * (af[z, :, :k].astype(np.float64) @ bz.astype(np.float64))
        _check(oracle, got[z, :, :n], ref.astype(np.float32))
    assert (got[:, :, n:] == -7.0).all(), "columns past N were written"


@pytest.mark.parametrize("dt_name", ["BF16", "F16"])
@pytest.mark.parametrize("lhs_t,rhs_t,out_t", [(0, 0, 0), (0, 1, 0), (1, 0, 0), (1, 1, 0), (0, 1, 1)])
@pytest.mark.parametrize("m,n,k", [(37, 50, 45), (300, 515, 1027), (130, 258, 77), (513, 100, 264)])
def test_gathered_operands(xmk, oracle, dt_name, lhs_t, rhs_t, out_t, m, n, k):
    """16-bit shapes whose rows do not start on 16-byte boundaries or whose K is not a multiple of 8
    run on the matrix cores with gathered operands: odd sizes in every layout, both tile sizes."""
    dt = getattr(oracle, dt_name)
    kind = _kind(dt, oracle)
    a = oracle.from_f32(oracle.normal((k, m) if lhs_t else (m, k), 70, 0.3), dt)
    b = oracle.from_f32(oracle.normal((n, k) if rhs_t else (k, n), 71, 0.3), dt)
    bias = oracle.from_f32(oracle.normal((n,), 72), dt)
    _, ref = oracle.gemm(a, b, dt, dt, lhs_t=lhs_t, rhs_t=rhs_t, out_t=out_t, bias=None if out_t else bias,
                         epilogue=oracle.EPI_DEFAULT if out_t else oracle.EPI_BIAS_RELU)
    tdt = torch.bfloat16 if kind == "bf16" else torch.float16
    out = torch.full((n, m) if out_t else (m, n), float("nan"), dtype=tdt, device="cuda")
    xmk.run_gemm(to_dev(a, kind), to_dev(b, kind), out, lhs_transpose=lhs_t, rhs_transpose=rhs_t,
                 out_transpose=out_t, bias=None if out_t else to_dev(bias, kind),
                 epilogue=xmk.EPI_DEFAULT if out_t else xmk.EPI_BIAS_RELU)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    _check(oracle, got.T if out_t else got, ref[0])


def test_gathered_operands_batched_f32_out(xmk, oracle):
    """Batched product with odd sizes and fp32 output through the gathering kernel, and a padded
    leading dimension that is not a multiple of 8."""
    dt = oracle.F16
    bsz, m, n, k = 3, 70, 45, 100
    a = oracle.from_f32(oracle.normal((bsz, m, k), 80, 0.3), dt)
    b = oracle.from_f32(oracle.normal((bsz, k, n), 81, 0.3), dt)
    out = torch.full((bsz, m, n), float("nan"), dtype=torch.float32, device="cuda")
    xmk.run_gemm(to_dev(a, "f16"), to_dev(b, "f16"), out)
    torch.cuda.synchronize()
    for i in range(bsz):
        _, ref = oracle.gemm(a[i], b[i], dt, oracle.F32)
        _check(oracle, out[i].cpu().numpy(), ref[0])
    # rows of 104 stored in a buffer with leading dimension 107 (odd: rows start 2-byte aligned only)
    ap = torch.zeros((m, 107), dtype=torch.float16, device="cuda")
    a2 = oracle.from_f32(oracle.normal((m, 104), 82, 0.3), dt)
    b2 = oracle.from_f32(oracle.normal((104, 48), 83, 0.3), dt)
    ap[:, :104] = to_dev(a2, "f16")
    o2 = torch.full((m, 48), float("nan"), dtype=torch.float16, device="cuda")
    xmk.run_gemm(ap[:, :104], to_dev(b2, "f16"), o2)
    torch.cuda.synchronize()
    _, ref = oracle.gemm(a2, b2, dt, dt)
    _check(oracle, o2.float().cpu().numpy(), ref[0])


@pytest.mark.parametrize("lhs_t,rhs_t,out_t", [(0, 0, 0), (0, 1, 0), (1, 0, 0), (1, 1, 0), (0, 0, 1)])
@pytest.mark.parametrize("m,n,k", [(37, 50, 45), (256, 384, 512), (300, 515, 1027), (129, 64, 20)])
def test_f32_gemm(xmk, oracle, lhs_t, rhs_t, out_t, m, n, k):
    """fp32 x fp32 -> fp32 on the fp32 matrix cores, every layout, aligned and odd sizes, with bias + ReLU.
    Against a float64 product: fp32 accumulation over K terms, so rtol 1e-4 on the tensor's scale."""
    a = oracle.normal((k, m) if lhs_t else (m, k), 90, 0.3).astype(np.float32)
    b = oracle.normal((n, k) if rhs_t else (k, n), 91, 0.3).astype(np.float32)
    bias = oracle.normal((n,), 92).astype(np.float32)
    A = a.T if lhs_t else a
    B = b.T if rhs_t else b
    ref = A.astype(np.float64) @ B.astype(np.float64)
    use_bias = not out_t
    if use_bias:
        ref = np.maximum(ref + bias.astype(np.float64), 0.0)
    out = torch.full((n, m) if out_t else (m, n), float("nan"), dtype=torch.float32, device="cuda")
    xmk.run_gemm(to_dev(a, "f32"), to_dev(b, "f32"), out, lhs_transpose=lhs_t, rhs_transpose=rhs_t,
                 out_transpose=out_t, bias=to_dev(bias, "f32") if use_bias else None,
                 epilogue=xmk.EPI_BIAS_RELU if use_bias else xmk.EPI_DEFAULT)
    torch.cuda.synchronize()
    got = out.cpu().numpy().astype(np.float64)
    got = got.T if out_t else got
    assert np.abs(got - ref).max() <= 1e-4 * max(np.abs(ref).max(), 1.0), np.abs(got - ref).max()


def test_f32_gemm_batched_beta(xmk, oracle):
    """Batched fp32 product accumulated in place (beta = 1, alpha = 0.5)."""
    bsz, m, n, k = 3, 130, 70, 96
    a = oracle.normal((bsz, m, k), 93, 0.3).astype(np.float32)
    b = oracle.normal((bsz, k, n), 94, 0.3).astype(np.float32)
    c = oracle.normal((bsz, m, n), 95).astype(np.float32)
    out = to_dev(c, "f32").clone()
    xmk.run_gemm(to_dev(a, "f32"), to_dev(b, "f32"), out, c=out, alpha=0.5, beta=1.0)
    torch.cuda.synchronize()
    ref = 0.5 * (a.astype(np.float64) @ b.astype(np.float64)) + c
    assert np.abs(out.cpu().numpy() - ref).max() <= 1e-4 * np.abs(ref).max()


@pytest.mark.parametrize("lhs_t,rhs_t,out_t", [(0, 0, 0), (0, 1, 0), (1, 0, 0), (1, 1, 0), (0, 1, 1)])
@pytest.mark.parametrize("m,n,k", [(37, 50, 45), (256, 384, 512), (300, 515, 1027), (129, 64, 20)])
def test_s8_gemm_is_bit_exact(xmk, lhs_t, rhs_t, out_t, m, n, k):
    """s8 x s8 -> s32 on the int8 matrix cores: integer arithmetic, so bit exact against an int64 product,
    in every layout, for aligned and odd sizes; and a batched product."""
    g = torch.Generator(device="cpu").manual_seed(m * 131 + n * 7 + k)
    a = torch.randint(-128, 128, (k, m) if lhs_t else (m, k), dtype=torch.int8, generator=g)
    b = torch.randint(-128, 128, (n, k) if rhs_t else (k, n), dtype=torch.int8, generator=g)
    A = (a.T if lhs_t else a).to(torch.int64)
    B = (b.T if rhs_t else b).to(torch.int64)
    ref = (A @ B).to(torch.int32)
    out = torch.full((n, m) if out_t else (m, n), -7, dtype=torch.int32, device="cuda")
    xmk.run_gemm(a.cuda(), b.cuda(), out, lhs_transpose=lhs_t, rhs_transpose=rhs_t, out_transpose=out_t)
    torch.cuda.synchronize()
    got = out.cpu()
    assert torch.equal(got.T if out_t else got, ref)


def test_s8_gemm_batched(xmk):
    g = torch.Generator(device="cpu").manual_seed(5)
    a = torch.randint(-128, 128, (3, 70, 96), dtype=torch.int8, generator=g)
    b = torch.randint(-128, 128, (3, 96, 130), dtype=torch.int8, generator=g)
    out = torch.empty((3, 70, 130), dtype=torch.int32, device="cuda")
    xmk.run_gemm(a.cuda(), b.cuda(), out)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), torch.bmm(a.to(torch.int64), b.to(torch.int64)).to(torch.int32))
