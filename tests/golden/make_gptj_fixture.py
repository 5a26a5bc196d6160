"""Writes tests/golden/gptj_tiny_step.npz: one decode step of a tiny random-init GPT-J computed by the
`transformers` library's GPTJForCausalLM (fp32, eager attention) on dequantised int4 weights.

Run from the repo root:  python tests/golden/make_gptj_fixture.py
The model is built from a GPTJConfig (nothing is downloaded).  The fixture holds the int4 weights,
LayerNorm parameters, the prefix hidden states, and transformers' logits for the last position; the
oracle's decode step (oracle/gptj.py) must reproduce them from the KV cache it builds itself.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402
from oracle import gptj as og  # noqa: E402

CFG = dict(n_layer=2, n_head=2, head_dim=32, rotary_dim=16, d_model=64, d_ff=128, vocab=96, group=32,
           ln_eps=1e-5)
T = 6  # prefix length + the new token


def rand_linear(k, n, seed, bias):
    qw = oracle.words((k // 8, n), seed)
    s = oracle.from_f32(oracle.uniform((k // CFG["group"], n), seed + 1, 0.005, 0.03), oracle.F16)
    z = oracle.from_f32(oracle.uniform((k // CFG["group"], n), seed + 2, 4.0, 11.0), oracle.F16)
    b = oracle.from_f32(oracle.normal((n,), seed + 3, 0.1), oracle.F16) if bias else None
    return qw, s, z, b


def main():
    from transformers import GPTJConfig, GPTJForCausalLM
    d, dff, V = CFG["d_model"], CFG["d_ff"], CFG["vocab"]
    hf_cfg = GPTJConfig(vocab_size=V, n_positions=64, n_embd=d, n_layer=CFG["n_layer"], n_head=CFG["n_head"],
                        rotary_dim=CFG["rotary_dim"], n_inner=dff, activation_function="gelu_new",
                        resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0, layer_norm_epsilon=CFG["ln_eps"])
    hf_cfg._attn_implementation = "eager"
    model = GPTJForCausalLM(hf_cfg).float().eval()
    arrays = {}
    sd = model.state_dict()

    def put_linear(prefix, name, lin, has_bias):
        qw, s, z, b = lin
        w = og.dequant_f32(qw, s, z, CFG["group"])  # [k, n]; torch Linear stores [n, k]
        sd[prefix + ".weight"] = torch.from_numpy(np.ascontiguousarray(w.T))
        if has_bias:
            sd[prefix + ".bias"] = torch.from_numpy(oracle.to_f32(b, oracle.F16))
        arrays[name + ".qweight"], arrays[name + ".scales"], arrays[name + ".zeros"] = qw, s, z
        if has_bias:
            arrays[name + ".bias"] = b

    for l in range(CFG["n_layer"]):
        pre = f"transformer.h.{l}."
        g = oracle.from_f32(1.0 + oracle.normal((d,), 100 + l, 0.1), oracle.F16)
        bta = oracle.from_f32(oracle.normal((d,), 200 + l, 0.1), oracle.F16)
        sd[pre + "ln_1.weight"] = torch.from_numpy(oracle.to_f32(g, oracle.F16))
        sd[pre + "ln_1.bias"] = torch.from_numpy(oracle.to_f32(bta, oracle.F16))
        arrays[f"l{l}.ln_gamma"], arrays[f"l{l}.ln_beta"] = g, bta
        qkv = rand_linear(d, 3 * d, 1000 + 100 * l, False)
        w = og.dequant_f32(*qkv[:3], CFG["group"])
        for i, nm in enumerate(("q_proj", "k_proj", "v_proj")):
            sd[pre + f"attn.{nm}.weight"] = torch.from_numpy(np.ascontiguousarray(w[:, i * d:(i + 1) * d].T))
        arrays[f"l{l}.qkv.qweight"], arrays[f"l{l}.qkv.scales"], arrays[f"l{l}.qkv.zeros"] = qkv[:3]
        put_linear(pre + "attn.out_proj", f"l{l}.out_proj", rand_linear(d, d, 1010 + 100 * l, False), False)
        put_linear(pre + "mlp.fc_in", f"l{l}.fc_in", rand_linear(d, dff, 1020 + 100 * l, True), True)
        put_linear(pre + "mlp.fc_out", f"l{l}.fc_out", rand_linear(dff, d, 1030 + 100 * l, True), True)
    g = oracle.from_f32(1.0 + oracle.normal((d,), 300, 0.1), oracle.F16)
    bta = oracle.from_f32(oracle.normal((d,), 301, 0.1), oracle.F16)
    sd["transformer.ln_f.weight"] = torch.from_numpy(oracle.to_f32(g, oracle.F16))
    sd["transformer.ln_f.bias"] = torch.from_numpy(oracle.to_f32(bta, oracle.F16))
    arrays["lnf_gamma"], arrays["lnf_beta"] = g, bta
    put_linear("lm_head", "lm_head", rand_linear(d, V, 2000, True), True)
    model.load_state_dict(sd)

    hidden = oracle.from_f32(oracle.normal((2, T, d), 7), oracle.F16)  # [B, T, d] input embeddings
    arrays["hidden"] = hidden
    with torch.no_grad():
        out = model(inputs_embeds=torch.from_numpy(oracle.to_f32(hidden, oracle.F16)), use_cache=False)
    arrays["logits_all"] = out.logits.numpy().astype(np.float32)  # [B, T, V]
    arrays["cfg_keys"] = np.array(list(CFG.keys()))
    arrays["cfg_vals"] = np.array([float(v) for v in CFG.values()])
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "gptj_tiny_step.npz"), **arrays)
    print("wrote gptj_tiny_step.npz; logits", arrays["logits_all"].shape)


if __name__ == "__main__":
    main()
