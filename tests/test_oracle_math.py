"""Pins the oracle's GEMM / int4 / fp8 / attention arithmetic against numpy float64
brute force, closed forms and invariants (none of these retype the oracle's loops:
they use numpy/scipy library routines on the decoded values)."""
import numpy as np
import pytest
from scipy.special import logsumexp


def _bits(oracle, shape, seed, dtype, scale=1.0):
    return oracle.from_f32(oracle.normal(shape, seed, scale), dtype)


def _gelu(x):
    return 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3)))


@pytest.mark.parametrize("dtype_name", ["BF16", "F16"])
@pytest.mark.parametrize("lhs_t,rhs_t,out_t", [(0, 0, 0), (0, 1, 0), (1, 0, 0), (1, 1, 1), (0, 0, 1)])
def test_gemm_vs_numpy(oracle, dtype_name, lhs_t, rhs_t, out_t):
    dt = getattr(oracle, dtype_name)
    m, n, k = 13, 20, 36
    a = _bits(oracle, (k, m) if lhs_t else (m, k), 1, dt)
    b = _bits(oracle, (n, k) if rhs_t else (k, n), 2, dt)
    af = oracle.to_f32(a, dt).astype(np.float64)
    bf = oracle.to_f32(b, dt).astype(np.float64)
    ref = (af.T if lhs_t else af) @ (bf.T if rhs_t else bf)
    out, out_f32 = oracle.gemm(a, b, dt, dt, lhs_t=lhs_t, rhs_t=rhs_t, out_t=out_t)
    assert np.allclose(out_f32[0], ref, rtol=1e-6, atol=1e-6)
    stored = oracle.to_f32(out[0], dt)
    logical = stored.T if out_t else stored
    assert np.array_equal(logical, oracle.to_f32(oracle.from_f32(out_f32[0], dt), dt))


def test_gemm_identity_and_epilogues(oracle):
    dt = oracle.BF16
    m, k = 9, 16
    a = _bits(oracle, (m, k), 3, dt)
    eye = oracle.from_f32(np.eye(k, dtype=np.float32), dt)
    out, _ = oracle.gemm(a, eye, dt, dt)
    assert np.array_equal(out[0], a)  # identity B => C == A bit for bit
    n = 12
    b = _bits(oracle, (k, n), 4, dt)
    bias = _bits(oracle, (n,), 5, dt)
    c = _bits(oracle, (m, n), 6, dt)
    af, bf = oracle.to_f32(a, dt).astype(np.float64), oracle.to_f32(b, dt).astype(np.float64)
    biasf, cf = oracle.to_f32(bias, dt).astype(np.float64), oracle.to_f32(c, dt).astype(np.float64)
    base = af @ bf
    cases = {
        oracle.EPI_DEFAULT: lambda x: x, oracle.EPI_RELU: lambda x: np.maximum(x, 0),
        oracle.EPI_GELU: _gelu, oracle.EPI_BIAS: lambda x: x + biasf,
        oracle.EPI_BIAS_RELU: lambda x: np.maximum(x + biasf, 0),
        oracle.EPI_BIAS_GELU: lambda x: _gelu(x + biasf),
    }
    for epi, fn in cases.items():
        for beta in (0.0, 1.0, 0.5):
            _, f32 = oracle.gemm(a, b, dt, dt, bias=bias, c=c if beta else None, beta=beta,
                                 epilogue=epi)
            # act(A.B + beta*C + bias): sum before the activation (onednn_matmul_utils.cc:439-448)
            pre = base + beta * cf
            assert np.allclose(f32[0], fn(pre), rtol=2e-6, atol=2e-6), (epi, beta)
    # linearity in beta for the DEFAULT epilogue
    _, f0 = oracle.gemm(a, b, dt, dt)
    _, f2 = oracle.gemm(a, b, dt, dt, c=c, beta=2.0)
    assert np.allclose(f2[0] - f0[0], 2.0 * cf, rtol=1e-5, atol=1e-6)


def test_gemm_batched_and_f32_out(oracle):
    dt = oracle.F16
    a = _bits(oracle, (3, 5, 8), 7, dt)
    b = _bits(oracle, (3, 8, 4), 8, dt)
    out, f32 = oracle.gemm(a, b, dt, oracle.F32)
    ref = np.einsum("bmk,bkn->bmn", oracle.to_f32(a, dt).astype(np.float64),
                    oracle.to_f32(b, dt).astype(np.float64))
    assert np.allclose(out, ref, rtol=1e-6, atol=1e-7)
    assert np.array_equal(out, f32)


def test_gemm_packed_matches_general(oracle):
    dt = oracle.BF16
    m, n, k = 17, 24, 520
    a, b = _bits(oracle, (m, k), 9, dt, 0.1), _bits(oracle, (k, n), 10, dt, 0.1)
    bias = _bits(oracle, (n,), 11, dt)
    _, f_gen = oracle.gemm(a, b, dt, dt, bias=bias, epilogue=oracle.EPI_BIAS_GELU)
    out_p, f_p = oracle.gemm_packed(a, b, dt, dt, bias=bias, epilogue=oracle.EPI_BIAS_GELU)
    assert np.allclose(f_p, f_gen[0], rtol=1e-5, atol=1e-6)
    bt = np.ascontiguousarray(b.T)
    _, f_t = oracle.gemm_packed(a, bt, dt, dt, rhs_t=True, bias=bias, epilogue=oracle.EPI_BIAS_GELU)
    assert np.array_equal(f_t, f_p)


# ----------------------------------------------------------------------- int4
def _int4_case(oracle, k, n, group, seed):
    qw = oracle.words((k // 8, n), seed)
    s = oracle.from_f32(oracle.uniform((k // group, n), seed + 1, 0.001, 0.02), oracle.F16)
    z = oracle.from_f32(oracle.uniform((k // group, n), seed + 2, 0.0, 15.0), oracle.F16)
    return qw, s, z


def _np_dequant(qw, s, z, group):
    k = qw.shape[0] * 8
    j = (np.arange(k) % 8).astype(np.uint32)[:, None]
    q = ((np.repeat(qw, 8, axis=0) >> (4 * j)) & 0xF).astype(np.float32)
    zf = np.repeat(z.view(np.float16).astype(np.float32), group, axis=0)
    sf = np.repeat(s.view(np.float16).astype(np.float32), group, axis=0)
    d = (q - zf).astype(np.float32)           # one fp32 rounding
    return (d * sf).astype(np.float32).astype(np.float16)  # second fp32 rounding, then RNE to fp16


def test_int4_dequant_bruteforce(oracle):
    qw, s, z = _int4_case(oracle, 512, 96, 128, 21)
    got = oracle.int4_dequant(qw, s, z, 128)
    assert np.array_equal(got, _np_dequant(qw, s, z, 128).view(np.uint16))


def test_int4_dequant_table(oracle):
    # every nibble value x a grid of (zero, scale): k = 8 rows hold nibbles; columns sweep z, s
    zs = np.linspace(0, 15, 61, dtype=np.float32)
    ss = np.linspace(0.001, 0.02, 40, dtype=np.float32)
    Z, S = np.meshgrid(zs, ss, indexing="ij")
    n = Z.size
    for base in (0, 8):
        word = sum(((base + j) & 0xF) << (4 * j) for j in range(8))
        qw = np.full((1, n), word, dtype=np.uint32)
        s = oracle.from_f32(S.reshape(1, n), oracle.F16)
        z = oracle.from_f32(Z.reshape(1, n), oracle.F16)
        got = oracle.int4_dequant(qw, s, z, 8)
        assert np.array_equal(got, _np_dequant(qw, s, z, 8).view(np.uint16))
        # nibble order: row j holds value base + j (low nibble first)
        sf, zf = s.view(np.float16).astype(np.float64), z.view(np.float16).astype(np.float64)
        approx = (np.arange(base, base + 8)[:, None] - zf) * sf
        assert np.allclose(got.view(np.float16).astype(np.float64), approx, rtol=2e-3, atol=1e-7)


def test_int4_gemm(oracle):
    k, n, m = 256, 40, 3
    qw, s, z = _int4_case(oracle, k, n, 128, 31)
    act = oracle.from_f32(oracle.normal((m, k), 33), oracle.F16)
    bias = oracle.from_f32(oracle.normal((n,), 34), oracle.F16)
    w = _np_dequant(qw, s, z, 128).astype(np.float64)
    ref = act.view(np.float16).astype(np.float64) @ w + bias.view(np.float16).astype(np.float64)
    out, f32 = oracle.int4_gemm(act, qw, s, z, 128, bias=bias, round_weights=True)
    assert np.allclose(f32, ref, rtol=1e-6, atol=1e-6)
    assert np.array_equal(out, f32.astype(np.float16).view(np.uint16))
    # the GEMM contract proper: fp32 dequantised weights, no fp16 rounding in between
    qf = ((np.repeat(qw, 8, axis=0) >> (4 * (np.arange(k) % 8).astype(np.uint32)[:, None])) & 0xF)
    zf = np.repeat(z.view(np.float16).astype(np.float32), 128, axis=0)
    sf = np.repeat(s.view(np.float16).astype(np.float32), 128, axis=0)
    w32 = ((qf.astype(np.float32) - zf).astype(np.float32) * sf).astype(np.float32)
    ref32 = (act.view(np.float16).astype(np.float64) @ w32.astype(np.float64)
             + bias.view(np.float16).astype(np.float64))
    _, f32u = oracle.int4_gemm(act, qw, s, z, 128, bias=bias)
    assert np.allclose(f32u, ref32, rtol=1e-6, atol=1e-6)
    assert oracle.rel_err(f32u, f32)[0] < 2e-3  # the two definitions differ by fp16 weight rounding only


# ------------------------------------------------------------------------ fp8
def test_fp8_quantize_and_gemm(oracle):
    import torch
    x = oracle.normal((48, 64), 41)
    q, scale = oracle.fp8_quantize(x)
    assert scale == np.float32(np.abs(x).max()) / np.float32(448.0)
    ref_q = torch.from_numpy(x / scale).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(q, ref_q)
    y = oracle.normal((64, 24), 42)
    qb, sb = oracle.fp8_quantize(y)
    table = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).double().numpy()
    ref = (table[q] @ table[qb]) * float(scale) * float(sb)
    out, f32 = oracle.fp8_gemm(q, qb, scale, sb)
    assert np.allclose(f32, ref, rtol=1e-5, atol=1e-6)
    assert np.array_equal(out, oracle.from_f32(f32, oracle.BF16))
    _, f32t = oracle.fp8_gemm(q, np.ascontiguousarray(qb.T), scale, sb, rhs_t=True)
    assert np.array_equal(f32t, f32)
    # quantisation error of a unit normal through e4m3 with amax scaling stays small
    assert np.abs(table[q] * scale - x).max() <= 0.0625 * np.abs(x).max()


# ------------------------------------------------------------------ attention
def _np_attention(qf, kf, vf, scale, bias=None, causal=False):
    s = np.einsum("bnfh,bnth->bnft", qf, kf).astype(np.float32).astype(np.float64) * np.float32(scale)
    if bias is not None:
        s = s + bias
    if causal:
        F, T = s.shape[-2:]
        s = np.where(np.arange(T)[None, :] > np.arange(F)[:, None], -np.inf, s)
    lse = logsumexp(s, axis=-1)
    p = np.exp(s - lse[..., None])
    return np.einsum("bnft,bnth->bnfh", p, vf), lse


@pytest.mark.parametrize("dtype_name", ["BF16", "F16"])
@pytest.mark.parametrize("causal,use_bias", [(False, False), (True, False), (False, True), (True, True)])
def test_fmha_vs_numpy(oracle, dtype_name, causal, use_bias):
    dt = getattr(oracle, dtype_name)
    B, N, F, T, H = 2, 3, 7, 11, 8
    q, k, v = (_bits(oracle, (B, N, F if i == 0 else T, H), 50 + i, dt) for i in range(3))
    bias = _bits(oracle, (B, N, F, T), 60, dt) if use_bias else None
    qf, kf, vf = (oracle.to_f32(x, dt).astype(np.float64) for x in (q, k, v))
    bf = oracle.to_f32(bias, dt).astype(np.float64) if use_bias else None
    ref, lse_ref = _np_attention(qf, kf, vf, H ** -0.5, bf, causal)
    out, f32, lse = oracle.fmha_fwd(q, k, v, dt, H ** -0.5, bias=bias, causal=causal, want_lse=True)
    assert np.allclose(f32, ref, rtol=1e-5, atol=1e-6)
    assert np.allclose(lse.reshape(B, N, F), lse_ref, rtol=1e-5, atol=1e-5)
    assert np.array_equal(out, oracle.from_f32(f32, dt))
    if causal:  # causal row 0 sees key 0 only
        assert np.allclose(f32[:, :, 0, :], vf[:, :, 0, :], rtol=1e-6)


def test_fmha_invariants(oracle):
    dt = oracle.BF16
    B, N, F, T, H = 1, 2, 5, 9, 16
    q, k = _bits(oracle, (B, N, F, H), 70, dt), _bits(oracle, (B, N, T, H), 71, dt)
    ones = oracle.from_f32(np.ones((B, N, T, H), np.float32), dt)
    _, f32, _ = oracle.fmha_fwd(q, k, ones, dt, 0.25)
    assert np.allclose(f32, 1.0, rtol=1e-6)  # V = 1 => O = 1
    v = _bits(oracle, (B, N, T, H), 72, dt)
    perm = np.random.default_rng(0).permutation(T)
    _, a, _ = oracle.fmha_fwd(q, k, v, dt, 0.25)
    _, b, _ = oracle.fmha_fwd(q, k[:, :, perm], v[:, :, perm], dt, 0.25)
    assert np.allclose(a, b, rtol=1e-5, atol=1e-6)  # key-permutation invariance (non-causal)
    # a per-row constant added through the bias changes nothing
    rowc = np.repeat(oracle.normal((B, N, F, 1), 73), T, axis=3)
    _, c, _ = oracle.fmha_fwd(q, k, v, dt, 0.25, bias=oracle.from_f32(rowc, dt))
    assert np.allclose(a, c, rtol=1e-5, atol=1e-6)
    # partial unit range leaves other units untouched and equals the full run on its units
    _, d, _ = oracle.fmha_fwd(q, k, v, dt, 0.25, first_unit=1, num_units=1)
    assert np.array_equal(d[0, 1], a[0, 1]) and not d[0, 0].any()


@pytest.mark.parametrize("causal", [False, True])
def test_fmha_online_form_agrees(oracle, causal):
    """The reference's streaming recurrence (fmha_forward.h:331-385, P rounded to the
    element type) stays within the reference test's own tolerance of the closed form
    (test/jax_ut.patch:997: atol 3e-2 bf16)."""
    dt = oracle.BF16
    B, N, F, T, H = 1, 2, 70, 77, 40
    q, k, v = (_bits(oracle, (B, N, F if i == 0 else T, H), 80 + i, dt) for i in range(3))
    _, closed, _ = oracle.fmha_fwd(q, k, v, dt, H ** -0.5, causal=causal)
    online = oracle.fmha_fwd_online(q, k, v, dt, H ** -0.5, causal=causal, kBc=32)
    assert np.abs(online - closed).max() < 3e-2
    assert oracle.rel_err(online, closed)[0] < 1e-2


@pytest.mark.parametrize("causal,use_bias", [(False, False), (True, True)])
def test_fmha_bwd_matches_finite_differences(oracle, causal, use_bias):
    """The backward closed form against central differences of the forward closed form (float64,
    fp16-exact inputs so that the rounding in from_f32 is the identity)."""
    rng = np.random.default_rng(3)
    B, N, F, T, H = 1, 2, 5, 7, 8
    scale = 0.37

    def r(shape):
        return (rng.integers(-8, 9, size=shape) / 8.0).astype(np.float32)  # exact in fp16
    q, k, v, g = r((B, N, F, H)), r((B, N, T, H)), r((B, N, T, H)), r((B, N, F, H))
    bias = r((B, N, F, T)) if use_bias else None

    def fwd(q_, k_, v_):
        s = scale * np.einsum("bnfh,bnth->bnft", q_, k_)
        if bias is not None:
            s = s + bias
        if causal:
            s = np.where(np.arange(T)[None, :] > np.arange(F)[:, None], -np.inf, s)
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        return np.einsum("bnft,bnth->bnfh", p, v_)

    bits = lambda x: oracle.from_f32(x, oracle.F16)
    dq, dk, dv = oracle.fmha_bwd(bits(q), bits(k), bits(v), bits(g), oracle.F16, scale,
                                 bias=None if bias is None else bits(bias), causal=causal)
    eps = 1e-5
    for name, x, grad in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        num = np.zeros(x.shape)
        xd = x.astype(np.float64)
        for idx in np.ndindex(*x.shape):
            xp, xm = xd.copy(), xd.copy()
            xp[idx] += eps
            xm[idx] -= eps
            args_p = [q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)]
            args_m = list(args_p)
            i = "qkv".index(name)
            args_p[i], args_m[i] = xp, xm
            num[idx] = ((fwd(*args_p) - fwd(*args_m)) * g).sum() / (2 * eps)
        assert np.abs(num - grad).max() <= 1e-6 * max(1.0, np.abs(grad).max()), name
