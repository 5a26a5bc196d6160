"""bench.py draws its inputs from a restatement (in torch) of the parity tests' seeded generator:
same seed and shape must give the same bits.  Checked here on the CPU by handing the generator a
torch proxy that drops the device argument."""
import numpy as np
import torch

import bench


class _CpuTorch:
    def __getattr__(self, name):
        f = getattr(torch, name)
        if callable(f) and name in ("tensor", "arange", "empty"):
            def on_cpu(*a, **kw):
                kw.pop("device", None)
                return f(*a, **kw)
            return on_cpu
        return f


def test_bench_generator_equals_the_tests_generator(oracle):
    g = bench.Seeded(_CpuTorch())
    g.CHUNK = 1000  # several chunks
    assert np.array_equal(g.normal((37, 91), 11, 0.5).numpy(), oracle.normal((37, 91), 11, 0.5))
    assert np.array_equal(g.uniform((50, 33), 12, 0.001, 0.02).numpy(), oracle.uniform((50, 33), 12, 0.001, 0.02))
    assert np.array_equal(g.words((64, 17), 13).numpy().view(np.uint32), oracle.words((64, 17), 13))
    bf = g.normal((50, 33), 14, dtype=torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(bf, oracle.from_f32(oracle.normal((50, 33), 14), oracle.BF16))
    f16 = g.uniform((50, 33), 15, 0.0, 15.0, dtype=torch.float16).numpy().view(np.uint16)
    assert np.array_equal(f16, oracle.from_f32(oracle.uniform((50, 33), 15, 0.0, 15.0), oracle.F16))
