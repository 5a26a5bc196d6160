"""Pins the oracle's GPT-J decode step against the `transformers` library's GPT-J (fixture)."""
import numpy as np

from gptj_util import as_oracle_layers, load_fixture


def test_decode_step_matches_transformers(oracle):
    from oracle import gptj as og
    cfg, layers, lnf, lm_head, hidden, logits_all = load_fixture(oracle)
    ol = as_oracle_layers(oracle, layers)
    lnf64 = tuple(oracle.to_f32(x, oracle.F16).astype(np.float64) for x in lnf)
    B, T, d = hidden.shape
    N, H = cfg["n_head"], cfg["head_dim"]
    hid = oracle.to_f32(hidden, oracle.F16).astype(np.float64)
    for rounding, tol in ((False, 2e-4), (True, 3e-2)):
        kc = [np.zeros((B, N, T, H)) for _ in layers]
        vc = [np.zeros((B, N, T, H)) for _ in layers]
        for pos in range(T):  # token by token through the KV cache == the full causal forward
            logits, _ = og.decode_step(cfg, ol, lnf64, lm_head, hid[:, pos], kc, vc, pos,
                                       round_intermediates=rounding)
            err = np.abs(logits - logits_all[:, pos]).max() / np.abs(logits_all[:, pos]).max()
            assert err < tol, (rounding, pos, err)


def test_rotary_is_a_rotation(oracle):
    from oracle import gptj as og
    x = oracle.normal((2, 3, 32), 5).astype(np.float64)
    y = og.rotary(x, 17, 16)
    assert np.allclose(np.linalg.norm(y, axis=-1), np.linalg.norm(x, axis=-1))  # norm preserved
    assert np.array_equal(y[..., 16:], x[..., 16:])                            # pass-through dims
    assert np.allclose(og.rotary(x, 0, 16), x)                                 # position 0 = identity
    # relative-position property: <R_m q, R_n k> depends on m - n only
    q, k = x[0, 0], x[0, 1]
    a = og.rotary(q, 9, 32) @ og.rotary(k, 4, 32)
    b = og.rotary(q, 25, 32) @ og.rotary(k, 20, 32)
    assert np.allclose(a, b)
