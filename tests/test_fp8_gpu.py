"""GPU parity: FP8 (e4m3fn) GEMM through the C ABI (xmk_fp8_gemm) against the oracle.
Tolerance: max relative error <= 5e-2 for fp8 outputs against an fp32 recompute of the same
quantised inputs (the kernel accumulates exact products in fp32, so it lands far inside)."""
import numpy as np
import pytest
import torch

from util import to_bits, to_dev

pytestmark = pytest.mark.gpu


def _quant(oracle, shape, seed):
    q, s = oracle.fp8_quantize(oracle.normal(shape, seed))
    return q, s


@pytest.mark.parametrize("m,n,k,rhs_t", [
    (256, 256, 128, True), (512, 384, 1024, True), (300, 260, 208, True), (64, 8, 16, True),
    (4136, 4104, 208, True),  # ragged edges of the 256x256 tile (taken when there are >= 256 tiles)
    (130, 72, 80, False), (256, 256, 256, False),
    # the gathering kernel: [k,n]-stored B, K that is not a multiple of 16, odd N, both tile sizes
    (300, 515, 1027, False), (37, 52, 45, True), (2100, 2060, 200, False), (2100, 2060, 72, True),
    # about one 256 x 128 tile per CU: the third tile of the direct kernel, whole and with ragged edges
    (2048, 4096, 128, True), (1800, 4000, 144, True),
    # [k,n]-stored B on the direct kernel (N % 16 == 0, K % 16 == 0): LDS transpose reads; the three tiles,
    # ragged M / N / K-step edges
    (512, 384, 1024, False), (300, 272, 208, False), (64, 16, 16, False), (4136, 4112, 208, False),
    (2048, 4096, 128, False), (1800, 4000, 144, False),
])
def test_fp8_gemm_shapes(xmk, oracle, m, n, k, rhs_t):
    a, sa = _quant(oracle, (m, k), 1)
    b, sb = _quant(oracle, (n, k) if rhs_t else (k, n), 2)
    ref_bits, ref = oracle.fp8_gemm(a, b, sa, sb, rhs_t=rhs_t)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    xmk.fp8_gemm(to_dev(a, "f8"), to_dev(b, "f8"), torch.tensor([sa], device="cuda"),
                 torch.tensor([sb], device="cuda"), out, rhs_transpose=rhs_t)
    torch.cuda.synchronize()
    g, e = oracle.rel_err(out.float().cpu().numpy(), ref)
    assert g <= 5e-2 and e <= 5e-2, (g, e)
    # exact fp8 products accumulated in fp32: what is left is the bf16 rounding of the output
    assert g <= 5e-3 and e <= 5e-3, (g, e)


@pytest.mark.parametrize("m,n,k,rhs_t", [(512, 384, 256, True), (300, 272, 208, False), (37, 52, 45, True)])
def test_fp8_gemm_ex_output_scale_and_bias(xmk, oracle, m, n, k, rhs_t):
    """xmk_fp8_gemm_ex: out = bf16(d_scale * (a_scale b_scale A B + bias)), each of d_scale / bias alone and
    both; whole and ragged tiles of the direct kernel in both layouts, and the gathering kernel."""
    a, sa = _quant(oracle, (m, k), 5)
    b, sb = _quant(oracle, (n, k) if rhs_t else (k, n), 6)
    bias = oracle.from_f32(oracle.normal((n,), 7, 8.0), oracle.BF16)
    _, prod = oracle.fp8_gemm(a, b, sa, sb, rhs_t=rhs_t)
    bias_f = oracle.to_f32(bias, oracle.BF16)[None, :]
    da, db = to_dev(a, "f8"), to_dev(b, "f8")
    dsa, dsb = torch.tensor([sa], device="cuda"), torch.tensor([sb], device="cuda")
    dsd, dbias = torch.tensor([0.25], device="cuda"), to_dev(bias, "bf16")
    for use_d, use_b in ((True, False), (False, True), (True, True)):
        ref = np.float32(0.25 if use_d else 1.0) * (prod + (bias_f if use_b else np.float32(0)))
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        xmk.fp8_gemm(da, db, dsa, dsb, out, rhs_transpose=rhs_t, d_scale=dsd if use_d else None,
                     bias=dbias if use_b else None)
        torch.cuda.synchronize()
        g, e = oracle.rel_err(out.float().cpu().numpy(), ref)
        assert g <= 5e-3 and e <= 5e-3, (use_d, use_b, g, e)


@pytest.mark.parametrize("rhs_t", [True, False])
def test_config4_fp8_8192_sampled_rows(xmk, oracle, rhs_t):
    """benchmark configuration 4: A, B [8192,8192] e4m3fn from N(0,1) with amax/448 scales, bf16 output;
    B stored [N, K] (rhs_t) or [K, N]."""
    n = 8192
    a, sa = _quant(oracle, (n, n), 11)
    b, sb = _quant(oracle, (n, n), 12)
    out = torch.empty((n, n), dtype=torch.bfloat16, device="cuda")
    xmk.fp8_gemm(to_dev(a, "f8"), to_dev(b, "f8"), torch.tensor([sa], device="cuda"),
                 torch.tensor([sb], device="cuda"), out, rhs_transpose=rhs_t)
    torch.cuda.synchronize()
    # one row per 512, at a different place of the 256-row tile (and of a wave's 32-row slab) each time
    rows = np.array([(3 + 37 * i) % 256 + 512 * i for i in range(n // 512)])
    _, ref = oracle.fp8_gemm(a[rows], b, sa, sb, rhs_t=rhs_t)
    g, e = oracle.rel_err(out[torch.from_numpy(rows).cuda()].float().cpu().numpy(), ref)
    print(f"config4 fp8: global {g:.2e} elementwise {e:.2e}")
    assert g <= 5e-2 and e <= 5e-2
    # identity-like property over the whole output: row sums equal A @ rowsum(B^T) (linearity)
    table = oracle.to_f32(np.arange(256, dtype=np.uint8), oracle.F8E4M3FN).astype(np.float64)
    colsum = table[b].sum(axis=0 if rhs_t else 1)
    expect = (table[a] @ colsum) * float(sa) * float(sb)
    got = out.double().sum(dim=1).cpu().numpy()
    # a row sum adds 8192 bf16 roundings of elements near 90: about 10 in all, against sums of 1e4
    assert np.abs(got - expect).max() <= 2e-3 * np.abs(expect).max() + 1.0
