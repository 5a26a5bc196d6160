"""GPU: the entry point that allocates nothing (xmk_fmha_decode_static) against xmk_fmha_decode, through
the C ABI: same kernels, so the outputs must be equal bit for bit.  Two calls in a row share the
library's built-in scratch array; the second is smaller, so stale partial results of the first lie
behind the ones it writes."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(xmk, B, N, T, H, cap, dtype, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    q = torch.randn((B, N, 1, H), device="cuda", generator=g).to(dtype)
    kc = torch.randn((B, N, cap, H), device="cuda", generator=g).to(dtype)
    vc = torch.randn((B, N, cap, H), device="cuda", generator=g).to(dtype)
    ws = torch.empty((xmk.fmha_decode_workspace_bytes(B, N, H, T),), dtype=torch.uint8, device="cuda")
    ref = torch.full((B, N, 1, H), float("nan"), device="cuda", dtype=dtype)
    got = torch.full((B, N, 1, H), float("nan"), device="cuda", dtype=dtype)
    xmk.fmha_decode(q, kc, vc, ref, ws, num_keys=T)
    return q, kc, vc, ref, got


def test_static_scratch_equals_workspace_path_twice(xmk):
    # first call: benchmark configuration 5's attention (64 units, 2048 keys: 16 splits of head size 256)
    q1, k1, v1, ref1, got1 = _both(xmk, 4, 16, 2048, 256, 2048, torch.float16, 1)
    # second call: fewer units, fewer keys, a smaller head, a ragged cache fill
    q2, k2, v2, ref2, got2 = _both(xmk, 2, 3, 333, 64, 400, torch.bfloat16, 2)
    xmk.fmha_decode_static(q1, k1, v1, got1, num_keys=2048)
    xmk.fmha_decode_static(q2, k2, v2, got2, num_keys=333)
    torch.cuda.synchronize()
    assert torch.isfinite(ref1.float()).all() and torch.isfinite(ref2.float()).all()
    assert torch.equal(got1.view(torch.int16), ref1.view(torch.int16))
    assert torch.equal(got2.view(torch.int16), ref2.view(torch.int16))
    # and the first shape again, after the smaller one
    got1.fill_(float("nan"))
    xmk.fmha_decode_static(q1, k1, v1, got1, num_keys=2048)
    torch.cuda.synchronize()
    assert torch.equal(got1.view(torch.int16), ref1.view(torch.int16))


def test_static_scratch_rejects_what_does_not_fit(xmk):
    B, N, H, T = 64, 64, 256, 4096  # 4096 units x 1 split x 258 floats > 4 MiB
    assert xmk.fmha_decode_workspace_bytes(B, N, H, T) > xmk.fmha_decode_static_max_bytes()
    q = torch.zeros((B, N, 1, H), device="cuda", dtype=torch.float16)
    kv = torch.zeros((B, N, 8, H), device="cuda", dtype=torch.float16)
    with pytest.raises(xmk.XmkError) as e:
        xmk.fmha_decode_static(q, kv, kv, torch.empty_like(q), num_keys=T, kv_head_stride=T * H)
    assert e.value.code == xmk.INVALID_ARGUMENT and "built-in array" in e.value.message


def test_static_calls_in_a_graph_allocate_nothing(xmk):
    """After xmk_fmha_decode_static_init (the address lookup, not to be done under capture): device memory
    is the same before and after eager calls, and two calls captured into a HIP graph replay to the
    workspace path's result every time, with eager work and synchronisations between the replays."""
    xmk.fmha_decode_static_init()
    q1, k1, v1, ref1, got1 = _both(xmk, 4, 16, 2048, 256, 2048, torch.float16, 3)
    q2, k2, v2, ref2, got2 = _both(xmk, 2, 3, 333, 64, 400, torch.bfloat16, 4)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        xmk.fmha_decode_static(q1, k1, v1, got1, num_keys=2048)
        xmk.fmha_decode_static(q2, k2, v2, got2, num_keys=333)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    assert torch.equal(got1.view(torch.int16), ref1.view(torch.int16))
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            xmk.fmha_decode_static(q1, k1, v1, got1, num_keys=2048, stream=side)
            xmk.fmha_decode_static(q2, k2, v2, got2, num_keys=333, stream=side)
    torch.cuda.current_stream().wait_stream(side)
    scratch = torch.zeros((1 << 20,), device="cuda")
    for i in range(4):
        got1.fill_(float("nan"))
        got2.fill_(float("nan"))
        scratch.add_(1.0)  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got1.view(torch.int16), ref1.view(torch.int16)), i
        assert torch.equal(got2.view(torch.int16), ref2.view(torch.int16)), i
