"""CPU restatement (numpy, float64) of one GPT-J decode step on int4 weights.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Structure follows GPT-J as the reference's example runs it (example/gptj/jax_gptj.py:57-68 loads
FlaxGPTJForCausalLM): per block  h = ln_1(x);  x' = x + out_proj(attn(h)) + fc_out(gelu_new(fc_in(h)));
q/k/v/out_proj without bias; rotary embedding on the first rotary_dim dims of each head, interleaved
pairs, inv_freq = 10000^(-2i/rotary_dim); scores / sqrt(head_dim); ln_f then lm_head.
Pinned by tests/golden/gptj_tiny_step.npz: the same step computed by the GPT-J implementation of the
`transformers` library on the dequantised weights (tests/golden/make_gptj_fixture.py).
Weights enter as (qweight uint32 [k/8,n], scales fp16 bits, zeros fp16 bits, bias fp16 bits | None);
the linear layers use the fp32 dequantised weight (q - z) * s, as xmk_int4_gemm is specified.
"""
import numpy as np

from . import F16, to_f32


def dequant_f32(qw, scales, zeros, group):
    k = qw.shape[0] * 8
    j = (np.arange(k) % 8).astype(np.uint32)[:, None]
    q = ((np.repeat(qw, 8, axis=0) >> (4 * j)) & 0xF).astype(np.float32)
    z = np.repeat(to_f32(zeros, F16), group, axis=0)
    s = np.repeat(to_f32(scales, F16), group, axis=0)
    return ((q - z).astype(np.float32) * s).astype(np.float32)


def predequantize(lin, group):
    """A linear layer with its weight dequantised once (for tests that apply one layer many times)."""
    qw, s, z, b = lin
    return {"dense": dequant_f32(qw, s, z, group), "bias": b}


def linear(x, lin, group):
    if isinstance(lin, dict):
        y = (x.astype(np.float64) @ lin["dense"]).astype(np.float64)  # fp32 weights, float64 accumulate
        b = lin["bias"]
    else:
        qw, s, z, b = lin
        y = x @ dequant_f32(qw, s, z, group).astype(np.float64)
    if b is not None:
        y = y + to_f32(b, F16).astype(np.float64)
    return y


def layernorm(x, gamma, beta, eps):
    mu = x.mean(axis=-1, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * gamma + beta


def gelu_new(x):
    return 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3)))


def rotary(x, position, rotary_dim):
    """x [B, N, H]; rotate interleaved pairs of the first rotary_dim dims."""
    out = x.copy()
    i = np.arange(rotary_dim // 2)
    ang = position * (10000.0 ** (-2.0 * i / rotary_dim))
    sn, cs = np.sin(ang), np.cos(ang)
    x0, x1 = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
    out[..., 0:rotary_dim:2] = x0 * cs - x1 * sn
    out[..., 1:rotary_dim:2] = x1 * cs + x0 * sn
    return out


def f16_round(x):
    """Round through fp16: what the kernels' fp16 intermediates (activations, cache rows) hold."""
    return x.astype(np.float16).astype(np.float64)


def decode_step(cfg, layers, lnf, lm_head, hidden, k_cache, v_cache, position, round_intermediates=True):
    """cfg: dict(n_head, head_dim, rotary_dim, group, ln_eps).  hidden float64 [B, d].
    k_cache / v_cache: lists (per layer) of float64 [B, N, cap, H]; row `position` is written in place.
    Returns (logits float64 [B, vocab], hidden_out float64 [B, d])."""
    r = f16_round if round_intermediates else (lambda a: a)
    N, H, group = cfg["n_head"], cfg["head_dim"], cfg["group"]
    B, d = hidden.shape
    x = hidden
    for l, L in enumerate(layers):
        h = r(layernorm(x, L["ln_gamma"], L["ln_beta"], cfg["ln_eps"]))
        qkv = r(linear(h, L["qkv"], group))
        q, k, v = (qkv[:, i * d:(i + 1) * d].reshape(B, N, H) for i in range(3))
        q = r(rotary(q, position, cfg["rotary_dim"]))
        k_cache[l][:, :, position, :] = r(rotary(k, position, cfg["rotary_dim"]))
        v_cache[l][:, :, position, :] = v
        kk, vv = k_cache[l][:, :, :position + 1, :], v_cache[l][:, :, :position + 1, :]
        s = np.einsum("bnh,bnth->bnt", q, kk) / np.sqrt(H)
        s = s - s.max(axis=-1, keepdims=True)
        p = np.exp(s)
        p = p / p.sum(axis=-1, keepdims=True)
        attn = r(np.einsum("bnt,bnth->bnh", p, vv).reshape(B, d))
        a = r(linear(attn, L["out_proj"], group))
        ff = r(gelu_new(linear(h, L["fc_in"], group)))
        x = r(x + a + linear(ff, L["fc_out"], group))
    hf = r(layernorm(x, lnf[0], lnf[1], cfg["ln_eps"]))
    return linear(hf, lm_head, group), x
