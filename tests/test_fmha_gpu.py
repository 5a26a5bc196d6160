"""GPU parity: fused multi-head-attention forward through the C ABI (xmk_fmha_fwd) against the
oracle's closed form.  Tolerance 1e-2 (bf16/fp16) on (a) the error relative to the tensor's scale,
(b) the error relative to sum_t p_t |v_t|, the scale of the terms each output is the sum of, and
(c) the elementwise figure with eps = rms(ref); plus the reference test's own absolute bound
(test/jax_ut.patch:997: atol 3e-2 bf16, 1e-2 fp16).  One class of cases holds (c) to 2e-2 instead:
bf16 with a causal mask or an additive bias.  P is rounded to the 16-bit type before P V (as the
reference does, fmha_forward.h:378-384); a mask's first rows and a bias of N(0,1) in score units
give rows whose softmax rests on a few keys, so that the output is a few O(1) terms, larger than the
rms of the whole unit's output, and the rounding of their weights alone reaches 1.0e-2 (bias) to
1.3e-2 (first causal rows) of rms(ref) in bf16 (measured on every kernel version; fp16 stays below
2e-3 and is held to 1e-2 like bf16 without mask and bias)."""
import numpy as np
import pytest
import torch

from util import to_bits, to_dev

pytestmark = pytest.mark.gpu


def _dt(oracle, name):
    return (oracle.BF16, "bf16", torch.bfloat16) if name == "bf16" else (oracle.F16, "f16", torch.float16)


def _run(xmk, oracle, name, B, N, F, T, H, *, causal=False, use_bias=False, lse=False, seed=0,
         units=None, f_stride=1, scale=None):
    dt, kind, tdt = _dt(oracle, name)
    q = oracle.from_f32(oracle.normal((B, N, F, H), seed + 1), dt)
    k = oracle.from_f32(oracle.normal((B, N, T, H), seed + 2), dt)
    v = oracle.from_f32(oracle.normal((B, N, T, H), seed + 3), dt)
    bias = oracle.from_f32(oracle.normal((B, N, F, T), seed + 4), dt) if use_bias else None
    scale = H ** -0.5 if scale is None else scale
    out = torch.full((B, N, F, H), float("nan"), dtype=tdt, device="cuda")
    lse_t = torch.full((B * N, F), float("nan"), dtype=torch.float32, device="cuda") if lse else None
    xmk.fmha_forward(to_dev(q, kind), to_dev(k, kind), to_dev(v, kind), out,
                     bias=None if bias is None else to_dev(bias, kind), lse=lse_t,
                     head_scale=scale, causal=causal)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy().reshape(B * N, F, H)
    assert np.isfinite(got).all()
    units = list(range(B * N)) if units is None else units
    e_bound = 2e-2 if (name == "bf16" and (causal or use_bias)) else 1e-2
    for u in units:
        # f_stride: one stride for every unit, or a stride per unit (sampled rows 0, s, 2 s, ...)
        fs = f_stride[u] if isinstance(f_stride, dict) else f_stride
        _, ref, ref_lse = oracle.fmha_fwd(q, k, v, dt, scale, bias=bias, causal=causal, want_lse=True,
                                          first_unit=u, num_units=1, f_stride=fs)
        ref = ref.reshape(B * N, F, H)[u, ::fs]
        _, ref_abs, _ = oracle.fmha_fwd(q, k, v & 0x7FFF, dt, scale, bias=bias, causal=causal,
                                        first_unit=u, num_units=1, f_stride=fs)
        ref_abs = ref_abs.reshape(B * N, F, H)[u, ::fs]
        g, e = oracle.rel_err(got[u, ::fs], ref,
                              label=f"fmha_fwd {name} [{B},{N},{F}x{T},{H}] causal={causal} bias={use_bias} unit {u}")
        c = oracle.cond_err(got[u, ::fs], ref, ref_abs)
        assert g <= 1e-2 and c <= 1e-2 and e <= e_bound, (u, g, c, e)
        assert np.abs(got[u, ::fs] - ref).max() <= (3e-2 if name == "bf16" else 1e-2)
        if lse:
            gl = lse_t.cpu().numpy()[u, ::fs]
            assert np.allclose(gl, ref_lse[u, ::fs], rtol=1e-3, atol=1e-3)
    return out


def test_config2_causal_bf16(xmk, oracle):
    """benchmark configuration 2: bf16 [8,32,2048,128], causal, scale 1/sqrt(128); three units, every 7th, 9th
    and 11th row (strides coprime to the 32 rows of a wave, so the samples walk through every lane of the
    row tiles and every position against the key tiles)."""
    _run(xmk, oracle, "bf16", 8, 32, 2048, 2048, 128, causal=True, units=[0, 101, 255],
         f_stride={0: 7, 101: 9, 255: 11})


@pytest.mark.parametrize("H", [64, 128, 256])
@pytest.mark.parametrize("causal,use_bias", [(False, True), (True, True), (True, False)])
def test_many_key_tiles(xmk, oracle, H, causal, use_bias):
    """32 key tiles, so that the unmasked steady-state steps of the pipeline run; the bias (in score units,
    N(0,1)) makes the running reference max move in later tiles too, which exercises the deferred
    rescale of O and of the row sum."""
    _run(xmk, oracle, "bf16", 1, 2, 2048, 2048, H, causal=causal, use_bias=use_bias, lse=True, seed=31,
         f_stride={0: 3, 1: 5})


def test_config2_full_size_properties(xmk, oracle):
    """Size-independent properties at the full shape: V = 1 => O = 1; causal row 0 == V[0]."""
    B, N, S, H = 8, 32, 2048, 128
    q = torch.randn((B, N, S, H), device="cuda").bfloat16()
    k = torch.randn((B, N, S, H), device="cuda").bfloat16()
    ones = torch.ones((B, N, S, H), device="cuda").bfloat16()
    out = torch.empty_like(q)
    xmk.fmha_forward(q, k, ones, out, causal=True)
    torch.cuda.synchronize()
    assert (out.float() - 1.0).abs().max().item() <= 1e-2
    v = torch.randn((B, N, S, H), device="cuda").bfloat16()
    xmk.fmha_forward(q, k, v, out, causal=True)
    torch.cuda.synchronize()
    assert torch.equal(out[:, :, 0, :], v[:, :, 0, :])


SD_SHAPES = [  # (b, F, T, heads, head_dim) of the reference's mha_rewrite_test (test/jax_ut.patch:914-935)
    (2, 9216, 9216, 5, 64), (2, 9216, 77, 5, 64), (2, 2304, 2304, 10, 64), (2, 2304, 77, 10, 64),
    (2, 576, 576, 20, 64), (2, 576, 77, 20, 64), (2, 144, 144, 20, 64), (2, 144, 77, 20, 64),
    (2, 4096, 4096, 8, 40), (2, 4096, 77, 8, 40), (2, 4096, 4096, 10, 64), (2, 4096, 77, 10, 64),
    (2, 1024, 1024, 8, 80), (2, 1024, 77, 8, 80), (2, 1024, 1024, 20, 64), (2, 1024, 77, 20, 64),
    (2, 256, 256, 8, 160), (2, 256, 77, 8, 160), (2, 64, 64, 8, 160), (2, 64, 77, 8, 160),
]


@pytest.mark.parametrize("name", ["bf16", "fp16"])
@pytest.mark.parametrize("shape", SD_SHAPES)
def test_reference_mha_shapes(xmk, oracle, name, shape):
    """The reference's 20 shapes x 2 dtypes, no mask, no bias, scale head_dim**-0.5.  Large shapes
    are checked on two units and a stride of query rows so the oracle finishes in seconds."""
    b, F, T, n, h = shape
    work = F * T
    f_stride = 1 if work <= (1 << 20) else (13 if work <= (1 << 24) else 127)  # coprime to the 32-row tiles
    units = [0, b * n - 1] if work > (1 << 18) else None
    _run(xmk, oracle, name, b, n, F, T, h, units=units, f_stride=f_stride, seed=F + T)


@pytest.mark.parametrize("name", ["bf16", "fp16"])
@pytest.mark.parametrize("causal,use_bias", [(True, False), (False, True), (True, True)])
@pytest.mark.parametrize("F,T,H", [(130, 200, 128), (64, 333, 64), (257, 129, 256), (1, 77, 80), (200, 64, 8),
                                   (384, 512, 64), (100, 264, 256)])
def test_masks_bias_lse(xmk, oracle, name, causal, use_bias, F, T, H):
    """Causal (top-left aligned, fmha_utils.h:45-96), additive bias [B,N,F,T], ragged F/T (padding
    mask, fmha_forward.h:313-318), LSE output (fmha_forward.h:433-450).  Key counts that are multiples
    of 8 take the bias through LDS tiles, the others element by element from global memory."""
    _run(xmk, oracle, name, 2, 3, F, T, H, causal=causal, use_bias=use_bias, lse=True, seed=F * 7 + T)


def test_bias_paths_agree(xmk):
    """The same bias through the LDS-staged path (16-byte aligned) and, from a copy that starts 2 bytes
    later, through the element-wise path: identical scores, so identical outputs."""
    B, N, F, T, H = 2, 2, 160, 328, 128
    q, k, v = (torch.randn((B, N, n, H), device="cuda").bfloat16() for n in (F, T, T))
    bias = torch.randn((B, N, F, T), device="cuda").bfloat16()
    shifted = torch.empty((bias.numel() + 8,), dtype=torch.bfloat16, device="cuda")
    shifted[1:1 + bias.numel()] = bias.reshape(-1)
    bias_unaligned = shifted[1:1 + bias.numel()].view(B, N, F, T)
    assert bias.data_ptr() % 16 == 0 and bias_unaligned.data_ptr() % 16 != 0
    o1, o2 = torch.empty_like(q), torch.empty_like(q)
    xmk.fmha_forward(q, k, v, o1, bias=bias)
    xmk.fmha_forward(q, k, v, o2, bias=bias_unaligned)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2)


@pytest.mark.parametrize("H,big_k", [(64, 16.0), (128, 12.0), (256, 8.0)])
@pytest.mark.parametrize("causal", [False, True])
def test_row_max_sees_every_key_of_a_tile(xmk, oracle, causal, H, big_k):
    """A lane holds 16 of a half tile's 32 keys of its query row and gets the other 16 from lane l ^ 32.
    Keys whose scores tower over the rest sit, in turn, in each of the two lanes' positions (key % 8 < 4
    and >= 4) and only there: a row maximum that misses one lane's keys leaves the exponent reference
    far below those scores and the exponentials overflow (scaled score 128 or more: e^128 > fp32 max).
    Every head-size class of the kernel."""
    B, N, S = 1, 2, 256
    q = np.ones((B, N, S, H), dtype=np.float32)
    v = oracle.normal((B, N, S, H), 77)
    for upper in (0, 1):
        k = np.zeros((B, N, S, H), dtype=np.float32)
        big = (np.arange(S) % 8 >= 4) == bool(upper)
        big[:40] = False  # the first steps set the reference from ordinary keys
        k[:, :, big, :] = big_k
        qb, kb, vb = (oracle.from_f32(x, oracle.BF16) for x in (q, k, v))
        out = torch.full((B, N, S, H), float("nan"), dtype=torch.bfloat16, device="cuda")
        xmk.fmha_forward(to_dev(qb, "bf16"), to_dev(kb, "bf16"), to_dev(vb, "bf16"), out, causal=causal)
        torch.cuda.synchronize()
        got = out.float().cpu().numpy()
        assert np.isfinite(got).all(), f"overflow with the large keys in lane half {upper}"
        _, ref, _ = oracle.fmha_fwd(qb, kb, vb, oracle.BF16, H ** -0.5, causal=causal)
        g, e = oracle.rel_err(got, ref.reshape(got.shape))
        assert g <= 1e-2 and e <= 2e-2, (upper, g, e)


def test_key_permutation_invariance(xmk):
    B, N, F, T, H = 1, 4, 256, 320, 128
    q = torch.randn((B, N, F, H), device="cuda").bfloat16()
    k = torch.randn((B, N, T, H), device="cuda").bfloat16()
    v = torch.randn((B, N, T, H), device="cuda").bfloat16()
    perm = torch.randperm(T, device="cuda")
    o1, o2 = torch.empty_like(q), torch.empty_like(q)
    xmk.fmha_forward(q, k, v, o1)
    xmk.fmha_forward(q, k[:, :, perm].contiguous(), v[:, :, perm].contiguous(), o2)
    torch.cuda.synchronize()
    assert (o1.float() - o2.float()).abs().max().item() <= 2e-2


def test_errors(xmk):
    q = torch.zeros((1, 1, 8, 12), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(xmk.XmkError) as e:
        xmk.fmha_forward(q, q, q, q.clone())
    assert e.value.code == xmk.UNIMPLEMENTED
    q = torch.zeros((1, 1, 8, 16), dtype=torch.float32, device="cuda")
    with pytest.raises(xmk.XmkError) as e:
        xmk.fmha_forward(q, q, q, q.clone())
    assert e.value.code == xmk.INTERNAL and "Invalid MHA datatype" in e.value.message
