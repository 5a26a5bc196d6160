"""GPU parity: fused attention backward through the C ABI (xmk_fmha_bwd) against the oracle's
float64 closed form (pinned by finite differences in tests/test_oracle_math.py).

Tolerance: error relative to the tensor's scale (oracle.rel_err's first figure) <= 1e-2 as for the
forward outputs.  The elementwise figure (eps = rms(ref)) is held to 1e-2 for fp16 on every shape
(measured maximum 3.9e-3) and, for bf16, to 1.5 times the measured maximum of each group of cases:
8e-2 on the small shapes (measured 5.3e-2) and 1.5e-1 on the shapes with thousands of rows
(measured 9.9e-2: the maximum over 1.5 M elements of a rounding-dominated error sits further out
in the tail).  P, dS and the forward output O (which enters through D = rowsum(dO o O)) are rounded
to the 16-bit operand type before the products that consume them, here as in the reference
(xetla/sdp/fmha_backward.h:195-196); with three mantissa bits fewer than fp16 that rounding is the
bf16 error, largest under a causal mask, where late keys receive few terms, and the same for the
fused kernels and for the GEMM composition (XMK_FMHA_BWD_COMPOSED=1, which test_backward_composition
runs in a child process).  The reference's own attention test allows atol 3e-2 for bf16 and 1e-2 for
fp16 on O(1) outputs (test/jax_ut.patch:997)."""
import numpy as np
import pytest
import torch

from util import to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-2
TOL_ELEM = {"bf16": 8e-2, "fp16": 1e-2}        # small shapes
TOL_ELEM_LARGE = {"bf16": 1.5e-1, "fp16": 1e-2}  # thousands of rows


def _run(xmk, oracle, name, B, N, F, T, H, causal, use_bias, seed=0, tol_elem=None):
    dt = oracle.BF16 if name == "bf16" else oracle.F16
    tdt = torch.bfloat16 if name == "bf16" else torch.float16
    q = oracle.from_f32(oracle.normal((B, N, F, H), seed + 1), dt)
    k = oracle.from_f32(oracle.normal((B, N, T, H), seed + 2), dt)
    v = oracle.from_f32(oracle.normal((B, N, T, H), seed + 3), dt)
    g = oracle.from_f32(oracle.normal((B, N, F, H), seed + 4), dt)
    bias = oracle.from_f32(oracle.normal((B, N, F, T), seed + 5), dt) if use_bias else None
    scale = H ** -0.5
    dq, dk, dv = oracle.fmha_bwd(q, k, v, g, dt, scale, bias=bias, causal=causal)
    kind = "bf16" if name == "bf16" else "f16"
    tq, tk, tv, tg = (to_dev(x, kind) for x in (q, k, v, g))
    tb = None if bias is None else to_dev(bias, kind)
    out = torch.empty_like(tq)
    lse = torch.empty((B * N, F), dtype=torch.float32, device="cuda")
    xmk.fmha_forward(tq, tk, tv, out, bias=tb, lse=lse, causal=causal)
    gq, gk, gv = xmk.fmha_backward(tq, tk, tv, out, tg, lse, bias=tb, causal=causal)
    torch.cuda.synchronize()
    errs = {}
    for nm, got, ref in (("dq", gq, dq), ("dk", gk, dk), ("dv", gv, dv)):
        ge, ee = oracle.rel_err(got.float().cpu().numpy(), ref.astype(np.float32),
                                label=f"fmha_bwd {nm} {name} [{B},{N},{F}x{T},{H}] causal={causal} bias={use_bias}")
        errs[nm] = (ge, ee)
        assert ge <= TOL and ee <= (tol_elem or TOL_ELEM[name]), (nm, ge, ee)
    return errs


@pytest.mark.parametrize("name", ["bf16", "fp16"])
@pytest.mark.parametrize("causal,use_bias", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("F,T,H", [(128, 128, 64), (200, 136, 128), (64, 77, 40), (257, 64, 256)])
def test_backward_shapes(xmk, oracle, name, causal, use_bias, F, T, H):
    _run(xmk, oracle, name, 2, 3, F, T, H, causal, use_bias)


def test_backward_large(xmk, oracle):
    """Many blocks with a bias and a causal mask; the elementwise bound of the large shapes."""
    errs = _run(xmk, oracle, "bf16", 1, 12, 2048, 2048, 64, True, True, seed=9, tol_elem=TOL_ELEM_LARGE["bf16"])
    print(errs)


_COMPOSED_CHILD = """
import sys
sys.path.insert(0, {tests!r}); sys.path.insert(0, {root!r})
import importlib
import oracle
import test_fmha_bwd_gpu as t
xmk = importlib.import_module("intel-extension-for-openxla_amd")
t._run(xmk, oracle, "fp16", 2, 3, 200, 136, 128, True, True)
t._run(xmk, oracle, "bf16", 2, 3, 257, 64, 256, False, False)
# more units than fit one workspace chunk (score buffers are capped at 1 GiB)
t._run(xmk, oracle, "bf16", 1, 12, 2048, 2048, 64, True, False, seed=9, tol_elem=t.TOL_ELEM_LARGE["bf16"])
print("composed ok")
"""


def test_backward_composition():
    """The GEMM composition (the path behind XMK_FMHA_BWD_COMPOSED=1) in a child process, since the
    switch is read once per process: bias, head size 256, and chunking over units."""
    import os
    import subprocess
    import sys
    tests = os.path.dirname(os.path.abspath(__file__))
    env = dict(os.environ, XMK_FMHA_BWD_COMPOSED="1")
    r = subprocess.run([sys.executable, "-c", _COMPOSED_CHILD.format(tests=tests, root=os.path.dirname(tests))],
                       env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "composed ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


@pytest.mark.parametrize("name,causal", [("bf16", True), ("fp16", False)])
def test_backward_fused_long(xmk, oracle, name, causal):
    """The fused kernels over many blocks in both directions (16 key blocks, 8 owner blocks), ragged
    ends in F and T; the elementwise bound of the large shapes."""
    errs = _run(xmk, oracle, name, 1, 3, 1000, 1016, 128, causal, False, seed=21, tol_elem=TOL_ELEM_LARGE[name])
    print(errs)


def test_backward_errors(xmk):
    q = torch.zeros((1, 1, 8, 64), dtype=torch.float16, device="cuda")
    lse = torch.zeros((1, 8), dtype=torch.float32, device="cuda")
    with pytest.raises(xmk.XmkError) as e:
        xmk.fmha_backward(q.float(), q.float(), q.float(), q.float(), q.float(), lse)
    assert e.value.code == xmk.INTERNAL and "Invalid MHA datatype" in e.value.message
    q2 = torch.zeros((1, 1, 8, 60), dtype=torch.float16, device="cuda")
    with pytest.raises(xmk.XmkError) as e:
        xmk.fmha_backward(q2, q2, q2, q2, q2, lse)
    assert e.value.code == xmk.UNIMPLEMENTED
