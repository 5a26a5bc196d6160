"""Pins the oracle's codecs and generators against torch's CPU casts and closed forms."""
import numpy as np
import torch


def test_bf16_decode_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.to_f32(bits, oracle.BF16)
    ref = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).float().numpy()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_f16_decode_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.to_f32(bits, oracle.F16)
    ref = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_e4m3fn_decode_exhaustive(oracle):
    bits = np.arange(256, dtype=np.uint8)
    got = oracle.to_f32(bits, oracle.F8E4M3FN)
    ref = torch.from_numpy(bits).view(torch.float8_e4m3fn).float().numpy()
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan], ref[~nan])
    assert got[0x7E] == 448.0 and got[0x01] == 2.0 ** -9  # closed form: max and min subnormal


def _encode_samples():
    rng = np.random.default_rng(7)
    parts = [
        rng.standard_normal(200000).astype(np.float32),
        (rng.standard_normal(200000) * 1e-3).astype(np.float32),
        (rng.standard_normal(100000) * 300).astype(np.float32),
        rng.integers(0, 2 ** 32, 400000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        np.array([0.0, -0.0, 448.0, 464.0, 465.0, 479.9, 480.0, 500.0, 65504.0, 65519.9, 65520.0,
                  2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -14, 2.0 ** -9, 2.0 ** -10,
                  1.5 * 2.0 ** -10, 2.0 ** -6, 0.3, 1e-3, np.inf, -np.inf], dtype=np.float32),
    ]
    # every midpoint between adjacent fp16 / e4m3 values (ties-to-even cases)
    h = np.arange(0, 0x7BFF, dtype=np.uint16).view(np.float16).astype(np.float64)
    parts.append(((h[:-1] + h[1:]) / 2).astype(np.float32))
    e = torch.arange(0, 0x7E, dtype=torch.uint8).view(torch.float8_e4m3fn).double().numpy()
    parts.append(((e[:-1] + e[1:]) / 2).astype(np.float32))
    x = np.concatenate(parts)
    return np.concatenate([x, -x])


def test_bf16_encode(oracle):
    x = _encode_samples()
    x = x[~np.isnan(x)]
    got = oracle.from_f32(x, oracle.BF16)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, ref)


def test_f16_encode(oracle):
    x = _encode_samples()
    x = x[~np.isnan(x)]
    got = oracle.from_f32(x, oracle.F16)
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, ref)


def test_e4m3fn_encode(oracle):
    x = _encode_samples()
    x = x[~np.isnan(x)]
    got = oracle.from_f32(x, oracle.F8E4M3FN)
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    # NaN patterns: compare as "is NaN", everything else bit for bit
    gn, rn = (got & 0x7F) == 0x7F, (ref & 0x7F) == 0x7F
    assert np.array_equal(gn, rn)
    assert np.array_equal(got[~gn], ref[~rn])
    # three known values of torch's cast (0.3, 448, 1e-3)
    probe = oracle.to_f32(oracle.from_f32(np.array([0.3, 448.0, 1e-3], np.float32),
                                          oracle.F8E4M3FN), oracle.F8E4M3FN)
    assert probe.tolist() == [0.3125, 448.0, 0.001953125]


def test_generators(oracle):
    a = oracle.normal((1 << 20,), seed=3)
    assert abs(a.mean()) < 5e-3 and abs(a.std() - 1.0) < 5e-3
    # counter based: a slice is reproducible, a different seed differs
    assert np.array_equal(a, oracle.normal((1 << 20,), seed=3))
    assert not np.array_equal(a[:100], oracle.normal((100,), seed=4))
    assert np.array_equal(a[:100], oracle.normal((100,), seed=3))
    u = oracle.uniform((1 << 18,), seed=5, lo=0.001, hi=0.02)
    assert u.min() >= 0.001 and u.max() <= 0.02 and abs(u.mean() - 0.0105) < 1e-4
    w = oracle.words((1 << 16,), seed=9)
    nib = np.stack([(w >> (4 * j)) & 0xF for j in range(8)])
    counts = np.bincount(nib.ravel(), minlength=16)
    assert counts.min() > 0.9 * nib.size / 16 and counts.max() < 1.1 * nib.size / 16
    # scale argument is a plain multiply
    assert np.allclose(oracle.normal((64,), 3, scale=0.25), a[:64] * 0.25, rtol=1e-6)
