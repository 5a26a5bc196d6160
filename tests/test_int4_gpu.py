"""GPU parity: int4 dequantisation (bit-exact) and the int4 weight-only GEMM, through the C ABI."""
import numpy as np
import pytest
import torch

from util import to_bits, to_dev

pytestmark = pytest.mark.gpu


def _case(oracle, m, k, n, group, seed):
    qw = oracle.words((k // 8, n), seed)
    s = oracle.from_f32(oracle.uniform((k // group, n), seed + 1, 0.001, 0.02), oracle.F16)
    z = oracle.from_f32(oracle.uniform((k // group, n), seed + 2, 0.0, 15.0), oracle.F16)
    act = oracle.from_f32(oracle.normal((m, k), seed + 3), oracle.F16)
    return act, qw, s, z


@pytest.mark.parametrize("k,n,group", [(4096, 16384, 128), (256, 64, 32), (512, 1024, 64), (1024, 200, 256)])
def test_int4_dequant_bit_exact(xmk, oracle, k, n, group):
    _, qw, s, z = _case(oracle, 1, k, n, group, 100 + n)
    ref = oracle.int4_dequant(qw, s, z, group)
    w = torch.empty((k, n), dtype=torch.float16, device="cuda")
    xmk.int4_dequant(to_dev(qw, "u32"), to_dev(s, "f16"), to_dev(z, "f16"), w, group=group)
    torch.cuda.synchronize()
    assert np.array_equal(to_bits(w), ref)


@pytest.mark.parametrize("m", [1, 8, 32])
def test_int4_gemm_gptj_mlp_shape(xmk, oracle, m):
    """benchmark configuration 3: K=4096, N=16384, group 128, M in {1, 8, 32}; <= 1e-2 vs fp32 recompute."""
    k, n, group = 4096, 16384, 128
    act, qw, s, z = _case(oracle, m, k, n, group, 7)
    _, ref = oracle.int4_gemm(act, qw, s, z, group)
    out = torch.empty((m, n), dtype=torch.float16, device="cuda")
    xmk.int4_gemm(to_dev(act, "f16"), to_dev(qw, "u32"), to_dev(s, "f16"), to_dev(z, "f16"), out,
                  group=group)
    torch.cuda.synchronize()
    g, e = oracle.rel_err(out.float().cpu().numpy(), ref)
    print(f"int4 m={m}: max|d|/max|ref|={g:.2e} elementwise={e:.2e}")
    assert g <= 1e-2 and e <= 1e-2
    # against act @ fp16-rounded weights the difference is the weights' fp16 rounding only
    _, ref16 = oracle.int4_gemm(act, qw, s, z, group, round_weights=True)
    assert oracle.rel_err(out.float().cpu().numpy(), ref16)[0] <= 1e-2


@pytest.mark.parametrize("m,k,n,group,with_bias", [
    (1, 4096, 4096, 128, False),    # attention projections of the decode step (narrow-N path)
    (4, 4096, 4096, 128, False),
    (4, 16384, 4096, 128, True),    # fc_out
    (3, 256, 8, 32, True),          # smallest legal N
    (17, 512, 200, 64, True),       # ragged N (not a multiple of the block's columns), two row tiles
    (33, 256, 72, 256, False),      # M > 32: second launch
    (16, 1024, 1024, 128, True),
    (2, 512, 136, 128, True),       # 2-4 rows and 5-8 rows take the variants that feed the rows spread out
    (6, 1024, 200, 64, False),
    (7, 4096, 4096, 128, True),
    (36, 256, 72, 32, True),        # 32 rows + 4 in a second launch
    (40, 512, 264, 128, False),     # 32 rows + 8
    # 9 to 32 rows (one or two 16-row tiles per wave), group sizes 32 to 128
    (12, 1024, 1024, 32, True),     # one row tile, group 32
    (9, 512, 200, 64, False),       # ragged N
    (25, 16384, 264, 128, True),    # 16 groups per wave
    (32, 8192, 1024, 64, False),
    (20, 256, 72, 128, False),      # fewer groups than waves
    (31, 640, 136, 128, True),      # 5 groups: waves with one group and waves with none
    (48, 4096, 1024, 128, True),    # 32 rows + 16 in a second launch
    # more than eight groups per wave: the straight-line part is followed by the loop, which ends on an
    # odd count (9 and 11 groups per wave) and after one group of the loop (9)
    (10, 9216, 264, 128, True), (5, 5632, 136, 64, False), (30, 9216, 72, 128, False),
    # more than 256 column blocks with 2 to 16 rows: four-wave work-groups (ragged last block; 9 groups over 4 waves)
    (4, 512, 16640, 128, True), (12, 256, 16448, 64, False), (6, 1152, 16400, 128, True), (3, 128, 16392, 32, False),
    # 16 groups per wave with the activations staged through LDS (eight-wave and four-wave forms): the reads of
    # both staging buffers inside the loop have to wait for their loads
    (32, 16384, 1024, 128, False), (6, 8192, 16400, 128, True),
    # groups of 256 channels run as two batches of 128 with the same scale and zero point
    (1, 2048, 512, 256, True), (8, 1024, 264, 256, False), (32, 4096, 256, 256, True), (4, 4096, 4096, 256, False),
])
def test_int4_gemm_shapes(xmk, oracle, m, k, n, group, with_bias):
    act, qw, s, z = _case(oracle, m, k, n, group, 1000 + m + n)
    bias = oracle.from_f32(oracle.normal((n,), 55), oracle.F16) if with_bias else None
    _, ref = oracle.int4_gemm(act, qw, s, z, group, bias=bias)
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
    xmk.int4_gemm(to_dev(act, "f16"), to_dev(qw, "u32"), to_dev(s, "f16"), to_dev(z, "f16"), out,
                  group=group, bias=None if bias is None else to_dev(bias, "f16"))
    torch.cuda.synchronize()
    g, e = oracle.rel_err(out.float().cpu().numpy(), ref)
    assert g <= 1e-2 and e <= 1e-2, (g, e)


def test_int4_gemm_linearity_full_size(xmk, oracle):
    """Size-independent property at the full shape: f(a1 + a2) == f(a1) + f(a2) within rounding."""
    k, n, group = 4096, 16384, 128
    _, qw, s, z = _case(oracle, 1, k, n, group, 7)
    dq, ds, dz = to_dev(qw, "u32"), to_dev(s, "f16"), to_dev(z, "f16")
    a1 = torch.randn((8, k), device="cuda").half()
    a2 = torch.randn((8, k), device="cuda").half()
    a3 = (a1.float() + a2.float()).half()
    outs = []
    for a in (a1, a2, a3):
        o = torch.empty((8, n), dtype=torch.float16, device="cuda")
        xmk.int4_gemm(a, dq, ds, dz, o, group=group)
        outs.append(o.float())
    torch.cuda.synchronize()
    err = (outs[2] - outs[0] - outs[1]).abs().max().item() / outs[2].abs().max().item()
    assert err < 1e-2


@pytest.mark.parametrize("m,k,n,group,with_bias", [(256, 512, 1024, 128, True), (200, 1024, 328, 64, False)])
def test_int4_gemm_many_rows_with_scratch(xmk, oracle, m, k, n, group, with_bias):
    """Prompt-sized row counts: with the scratch xmk_int4_gemm_workspace_bytes asks for, the weights are
    dequantised once and the dense fp16 GEMM runs; without it the streaming kernel runs.  Both within
    1e-2 of the fp32 recompute, and of the recompute from fp16-rounded weights."""
    act, qw, s, z = _case(oracle, m, k, n, group, 2000 + m)
    bias = oracle.from_f32(oracle.normal((n,), 56), oracle.F16) if with_bias else None
    _, ref = oracle.int4_gemm(act, qw, s, z, group, bias=bias)
    _, ref16 = oracle.int4_gemm(act, qw, s, z, group, bias=bias, round_weights=True)
    need = xmk.int4_gemm_workspace_bytes(m, k, n)
    assert need == k * n * 2
    assert xmk.int4_gemm_workspace_bytes(32, k, n) == 0   # decode-sized calls never ask for scratch
    ws = torch.empty((need,), dtype=torch.uint8, device="cuda")
    dev = [to_dev(act, "f16"), to_dev(qw, "u32"), to_dev(s, "f16"), to_dev(z, "f16")]
    dbias = None if bias is None else to_dev(bias, "f16")
    outs = []
    for scratch in (ws, None):
        out = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
        xmk.int4_gemm_ws(*dev, out, scratch, group=group, bias=dbias)
        torch.cuda.synchronize()
        for r in (ref, ref16):
            g, e = oracle.rel_err(out.float().cpu().numpy(), r)
            assert g <= 1e-2 and e <= 1e-2, (scratch is not None, g, e)
        outs.append(out.float())
    assert (outs[0] - outs[1]).abs().max().item() <= 1e-2 * outs[1].abs().max().item()


def test_int4_errors(xmk):
    a = torch.zeros((1, 256), dtype=torch.float16, device="cuda")
    qw = torch.zeros((32, 64), dtype=torch.int32, device="cuda")
    sz = torch.zeros((2, 64), dtype=torch.float16, device="cuda")
    out = torch.zeros((1, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(xmk.XmkError) as e:
        xmk.int4_gemm(a, qw, sz, sz, out, group=100)
    assert e.value.code == xmk.INVALID_ARGUMENT
    with pytest.raises(xmk.XmkError) as e:
        xmk.int4_gemm(a, qw, sz, sz, out, group=8)
    assert e.value.code == xmk.UNIMPLEMENTED
    # the same contract on the dense path
    a2 = torch.zeros((256, 256), dtype=torch.float16, device="cuda")
    out2 = torch.zeros((256, 64), dtype=torch.float16, device="cuda")
    ws = torch.empty((xmk.int4_gemm_workspace_bytes(256, 256, 64),), dtype=torch.uint8, device="cuda")
    with pytest.raises(xmk.XmkError) as e:
        xmk.int4_gemm_ws(a2, qw, sz, sz, out2, ws, group=8)
    assert e.value.code == xmk.UNIMPLEMENTED
