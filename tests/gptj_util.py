"""Shared by the GPT-J decode-step tests: fixture loading and random model construction."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gptj_tiny_step.npz")


def load_fixture(oracle):
    z = np.load(GOLDEN, allow_pickle=False)
    cfg = {k: v for k, v in zip(z["cfg_keys"].tolist(), z["cfg_vals"].tolist())}
    cfg = {k: (float(v) if k == "ln_eps" else int(v)) for k, v in cfg.items()}

    def lin(name, bias):
        return (z[name + ".qweight"], z[name + ".scales"], z[name + ".zeros"], z[name + ".bias"] if bias else None)

    layers = []
    for l in range(cfg["n_layer"]):
        layers.append(dict(ln_gamma=z[f"l{l}.ln_gamma"], ln_beta=z[f"l{l}.ln_beta"], qkv=lin(f"l{l}.qkv", False),
                           out_proj=lin(f"l{l}.out_proj", False), fc_in=lin(f"l{l}.fc_in", True),
                           fc_out=lin(f"l{l}.fc_out", True)))
    return cfg, layers, (z["lnf_gamma"], z["lnf_beta"]), lin("lm_head", True), z["hidden"], z["logits_all"]


def random_model(oracle, cfg, seed=0):
    """Random int4 model as bit patterns, inputs as benchmark configuration 5 describes them."""
    d, dff, V, g = cfg["d_model"], cfg["d_ff"], cfg["vocab"], cfg["group"]

    def lin(k, n, s, bias):
        qw = oracle.words((k // 8, n), s)
        sc = oracle.from_f32(oracle.uniform((k // g, n), s + 1, 0.001, 0.02), oracle.F16)
        zp = oracle.from_f32(oracle.uniform((k // g, n), s + 2, 0.0, 15.0), oracle.F16)
        b = oracle.from_f32(oracle.normal((n,), s + 3, 0.02), oracle.F16) if bias else None
        return qw, sc, zp, b

    layers = []
    for l in range(cfg["n_layer"]):
        s = seed + 1000 * (l + 1)
        layers.append(dict(
            ln_gamma=oracle.from_f32(1.0 + oracle.normal((d,), s + 10, 0.02), oracle.F16),
            ln_beta=oracle.from_f32(oracle.normal((d,), s + 11, 0.02), oracle.F16),
            qkv=lin(d, 3 * d, s + 20, False), out_proj=lin(d, d, s + 30, False),
            fc_in=lin(d, dff, s + 40, True), fc_out=lin(dff, d, s + 50, True)))
    lnf = (oracle.from_f32(1.0 + oracle.normal((d,), seed + 5, 0.02), oracle.F16),
           oracle.from_f32(oracle.normal((d,), seed + 6, 0.02), oracle.F16))
    return layers, lnf, lin(d, V, seed + 70, True)


def as_oracle_layers(oracle, layers):
    """LayerNorm parameters decoded to float64 for oracle.gptj.decode_step."""
    out = []
    for L in layers:
        M = dict(L)
        M["ln_gamma"] = oracle.to_f32(L["ln_gamma"], oracle.F16).astype(np.float64)
        M["ln_beta"] = oracle.to_f32(L["ln_beta"], oracle.F16).astype(np.float64)
        out.append(M)
    return out
