#!/usr/bin/env python3
"""Roofline benchmark of the custom-call kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-also] [--no-cpu] [--ramp S] [--observe S]

One JSON line on stdout.  A "step" is one launch of the workload's kernel on synthetic inputs that
are already resident in HBM.  The headline workload is benchmark configuration 2 (fused causal MHA forward,
bf16 [8,32,2048,128]); the other configs are timed the same way and reported under "also".
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0}  # dense MFMA TFLOP/s, MI355X
HBM_PEAK = 8000.0                                        # GB/s
RAMP_SECONDS = 0.25                                      # untimed launches before the warmup steps (clock ramp)

# HBM bytes per launch of each workload's dominant kernel, measured with rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE (KiB per dispatch), FETCH_SIZE scaled by 2.0 and WRITE_SIZE by 1.0: the factors a
# 1 GiB device copy (--workload copy) gives on this machine.  Counter figures of an earlier run of the same
# kernels (profiles/hbm_traffic_pmc.txt says which build and when), not of the run that prints them: they are
# to be measured again whenever one of these kernels changes.  A workload without a measurement reports null.
TRAFFIC_BYTES = {
    "fmha_causal": (204930 * 2.0 + 131070) * 1024,
    "gemm_8192": (790500 * 2.0 + 131070) * 1024,
    "int4_m1": (17490 * 2.0 + 32) * 1024,
    "gemv_f16_m4_vocab": (203210 * 2.0 + 394) * 1024,
    "gemv_f16_m1_rhsT": (65646 * 2.0 + 32) * 1024,
    "fp8_8192": (393620 * 2.0 + 131070) * 1024,
}


class Seeded:
    """The deterministic input generator of the parity tests, restated on the GPU: a splitmix64 counter
    hash (seed, element index) -> 64 bits; N(0,1) by Box-Muller in double on counters 2i, 2i+1;
    U(lo,hi) and 32-bit words from counter i.  Same seed and shape give the values the tests' host
    generator gives (up to the last bit of the device's log / cos before the cast to float)."""
    CHUNK = 1 << 24

    def __init__(self, torch):
        self.t = torch
        s = lambda v: torch.tensor(v - (1 << 64) if v >= (1 << 63) else v, dtype=torch.int64, device="cuda")
        self.c1, self.c2, self.c3 = s(0x9e3779b97f4a7c15), s(0xbf58476d1ce4e5b9), s(0x94d049bb133111eb)
        self.m, self.a = s(0xd1342543de82ef95), s(0x632be59bd9b4e019)

    @staticmethod
    def _lsr(x, k):  # logical shift right of the 64-bit pattern held in an int64
        return (x >> k) & ((1 << (64 - k)) - 1)

    def _mix(self, x):
        x = x + self.c1
        x = (x ^ self._lsr(x, 30)) * self.c2
        x = (x ^ self._lsr(x, 27)) * self.c3
        return x ^ self._lsr(x, 31)

    def _draw(self, seed, ctr):
        key = self._mix(self.t.tensor(seed, dtype=self.t.int64, device="cuda"))
        return self._mix(key ^ (ctr * self.m + self.a))

    def _unit(self, r):  # (0, 1)
        return (self._lsr(r, 11).double() + 0.5) * (1.0 / 9007199254740992.0)

    def _chunks(self, n):
        for lo in range(0, n, self.CHUNK):
            yield lo, self.t.arange(lo, min(n, lo + self.CHUNK), dtype=self.t.int64, device="cuda")

    def normal(self, shape, seed, scale=1.0, dtype=None):
        t = self.t
        n = 1
        for d in shape:
            n *= d
        out = t.empty((n,), dtype=dtype or t.float32, device="cuda")
        for lo, i in self._chunks(n):
            u1, u2 = self._unit(self._draw(seed, 2 * i)), self._unit(self._draw(seed, 2 * i + 1))
            z = t.sqrt(-2.0 * t.log(u1)) * t.cos(6.283185307179586476925 * u2)
            out[lo:lo + i.numel()] = (z * float(scale)).float().to(out.dtype)  # double -> float -> storage type
        return out.view(shape)

    def uniform(self, shape, seed, lo_v, hi_v, dtype=None):
        t = self.t
        n = 1
        for d in shape:
            n *= d
        out = t.empty((n,), dtype=dtype or t.float32, device="cuda")
        lo_f, hi_f = (t.tensor(v, dtype=t.float32).item() for v in (lo_v, hi_v))  # the bounds are floats, widened
        for lo, i in self._chunks(n):
            u = self._unit(self._draw(seed, i))
            out[lo:lo + i.numel()] = (lo_f + u * (hi_f - lo_f)).float().to(out.dtype)
        return out.view(shape)

    def words(self, shape, seed):
        t = self.t
        n = 1
        for d in shape:
            n *= d
        out = t.empty((n,), dtype=t.int32, device="cuda")
        for lo, i in self._chunks(n):
            out[lo:lo + i.numel()] = self._lsr(self._draw(seed, i), 32).to(t.int32)  # low 32 bits kept: wraps to signed
        return out.view(shape)


class Constant:
    """--data constant: every operand element the same value.  Not a benchmark input: with nothing toggling in
    the operand paths the same kernels draw 150-300 W less and the device holds its full clock, so the run
    shows what the schedule alone sustains, beside what the power limit leaves of it on the seeded data."""

    def __init__(self, torch):
        self.t = torch

    def normal(self, shape, seed, scale=1.0, dtype=None):
        return self.t.full(shape, 0.03125 * float(scale), dtype=dtype or self.t.float32, device="cuda")

    def uniform(self, shape, seed, lo_v, hi_v, dtype=None):
        return self.t.full(shape, 0.5 * (lo_v + hi_v), dtype=dtype or self.t.float32, device="cuda")

    def words(self, shape, seed):
        return self.t.full(shape, 0x11111111, dtype=self.t.int32, device="cuda")


_GEN = None
DATA = "seeded"


def gen(torch):
    global _GEN
    if _GEN is None:
        _GEN = Constant(torch) if DATA == "constant" else Seeded(torch)
    return _GEN


class ClockSampler:
    """Core clock (per XCD), socket power and throttler residencies as the SMI library reports them, read by
    a host thread while a workload runs untimed: what the device held under that load, and which
    limiter (package power tracking, thermal) held it there, next to the published peak (which
    assumes 2400 MHz).  Never running during a timed region."""

    def __init__(self):
        self.smi = self.handle = None
        self.source = "unavailable"
        try:
            sys.path.insert(0, "/opt/rocm/share/amd_smi")
            import amdsmi
            amdsmi.amdsmi_init()
            self.handle = amdsmi.amdsmi_get_processor_handles()[0]
            self.smi = amdsmi
            self.source = "amdsmi gpu_metrics (current_gfxclks, current_socket_power)"
            if not self._read():
                self.source = "amdsmi clock_info / power_info"
                self.metrics = False
                if not self._read():
                    self.smi, self.source = None, "unavailable"
        except Exception as e:  # no SMI library, or no permission: the bench line says so
            self.smi, self.source = None, f"unavailable ({type(e).__name__})"

    metrics = True

    def _read(self):
        try:
            if self.metrics:
                m = self.smi.amdsmi_get_gpu_metrics_info(self.handle)
                clks = [c for c in m.get("current_gfxclks", []) if isinstance(c, (int, float)) and 0 < c < 10000]
                pw = m.get("current_socket_power")
                if not clks:
                    return None
                return clks, (pw if isinstance(pw, (int, float)) and pw < 10000 else None)
            c = self.smi.amdsmi_get_clock_info(self.handle, self.smi.AmdSmiClkType.GFX)["clk"]
            pw = self.smi.amdsmi_get_power_info(self.handle).get("current_socket_power")
            return [c], (pw if isinstance(pw, (int, float)) else None)
        except Exception:
            return None

    THROTTLERS = ("ppt_residency_acc", "socket_thm_residency_acc", "vr_thm_residency_acc", "hbm_thm_residency_acc",
                  "prochot_residency_acc")

    def _residency(self):
        """The firmware's accumulated throttler residencies and its sample counter (gpu_metrics)."""
        for _ in range(3):  # the call fails now and then while the device is busy
            try:
                m = self.smi.amdsmi_get_gpu_metrics_info(self.handle)
                out = {k: m.get(k) for k in self.THROTTLERS + ("accumulation_counter",)}
                if all(isinstance(v, int) for v in out.values()):
                    return out
            except Exception:
                pass
            time.sleep(0.002)
        return None

    def observe(self, torch, fn, seconds):
        """Runs fn back to back for `seconds` (longer when the firmware's counters have not ticked twice by
        then) and samples the clocks every ~10 ms; returns the summary dict."""
        if self.smi is None or seconds <= 0:
            return {"source": self.source}
        import threading
        samples, stop = [], threading.Event()

        def loop():
            while not stop.is_set():
                r = self._read()
                if r:
                    samples.append(r)
                time.sleep(0.01)
        th = threading.Thread(target=loop, daemon=True)
        # The firmware publishes its throttler residencies about once a second, 1000 samples at a time: a
        # difference between two publications that both fall inside this run covers this workload only.
        ticks = []
        last = self._residency() if self.metrics else None
        t0 = time.perf_counter()
        started = False
        burst = 8
        while True:
            tb = time.perf_counter()
            for _ in range(burst):
                fn()
            torch.cuda.synchronize()
            el = time.perf_counter() - t0
            # bursts of about 25 ms, so that the host's reads between them leave the device busy
            burst = max(8, min(4096, int(burst * 0.025 / max(time.perf_counter() - tb, 1e-5))))
            if last is not None:
                r = self._residency()
                if r and r["accumulation_counter"] != last["accumulation_counter"]:
                    ticks.append(r)
                    last = r
            if not started and el > 0.5 * seconds:  # clocks: the settled part only
                th.start()
                started = True
            if el >= seconds and (last is None or len(ticks) >= 2 or el >= seconds + 1.5):
                break
        stop.set()
        if started:
            th.join()
        if not samples:
            return {"source": self.source, "samples": 0}
        means = [sum(c) / len(c) for c, _ in samples]
        pws = [p for _, p in samples if p is not None]
        out = {"source": self.source, "samples": len(samples), "mean_mhz": round(sum(means) / len(means)),
               "min_mhz": round(min(min(c) for c, _ in samples)), "max_mhz": round(max(max(c) for c, _ in samples)),
               "xcds": len(samples[0][0])}
        if pws:
            out["socket_power_w_mean"] = round(sum(pws) / len(pws))
        if len(ticks) >= 2:
            # share of the firmware's samples between two publications during which a throttler held the clock down
            n = ticks[-1]["accumulation_counter"] - ticks[0]["accumulation_counter"]
            if n > 0:
                out["throttled"] = {k[:-len("_residency_acc")]: round((ticks[-1][k] - ticks[0][k]) / n, 3)
                                    for k in self.THROTTLERS}
                out["firmware_samples"] = n
        return out


CLOCKS = None
OBSERVE_SECONDS = 1.0


def _events(torch, fn, steps, warmup, graph=False):
    """Average duration (ms) of fn over `steps` launches, HIP events on torch's current stream
    (the stream every xmk call below is launched on).  graph=True replays the launches from one
    captured HIP graph, so that kernels of a few microseconds are not timed at the rate the host
    can enqueue them from Python."""
    # Bring the device to its sustained clocks first: from idle it takes about 50 ms of continuous
    # work before the kernels run at their steady rate (the first 10 ms run at little more than half of
    # it).  These launches are neither warmup steps nor timed steps.
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < RAMP_SECONDS:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    if graph:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(steps):
                fn()
        launches = fn
        fn, steps_in = (lambda: g.replay()), steps
        fn()  # one untimed replay
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        wall0 = time.perf_counter()
        start.record()
        fn()
        stop.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - wall0) * 1e3 / steps_in
        return start.elapsed_time(stop) / steps_in, wall
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    wall0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - wall0) * 1e3 / steps
    return start.elapsed_time(stop) / steps, wall


# ---------------------------------------------------------------- workloads
def wl_fmha(torch, xmk, causal=True, B=8, N=32, S=2048, H=128):
    q, k, v = (gen(torch).normal((B, N, S, H), 201 + i, dtype=torch.bfloat16) for i in range(3))
    out = torch.empty_like(q)
    flops = 4.0 * B * N * S * S * H * (0.5 if causal else 1.0)
    nbytes = 4.0 * B * N * S * H * 2
    name = f"fmha_fwd_{'causal_' if causal else ''}bf16_b{B}_h{N}_s{S}_d{H}"
    return dict(name=name, fn=lambda: xmk.fmha_forward(q, k, v, out, causal=causal), flops=flops,
                bytes=nbytes, bound="mfma", dtype="bf16", kernel="fmha_fwd_kernel",
                note="causal FLOPs counted as 2*B*N*S^2*D (half of the dense 4*B*N*S^2*D)")


def wl_fmha_bwd(torch, xmk, causal=True, B=8, N=32, S=2048, H=128):
    """Gradients of the headline attention shape.  Flops counted as the 5 products of the textbook
    backward (2.5x the forward's), although the kernels recompute S per pass."""
    q, k, v, d_o = (gen(torch).normal((B, N, S, H), 201 + i, dtype=torch.bfloat16) for i in range(4))
    out = torch.empty_like(q)
    lse = torch.empty((B * N, S), dtype=torch.float32, device="cuda")
    xmk.fmha_forward(q, k, v, out, lse=lse, causal=causal)
    flops = 10.0 * B * N * S * S * H * (0.5 if causal else 1.0)
    return dict(name=f"fmha_bwd_{'causal_' if causal else ''}bf16_b{B}_h{N}_s{S}_d{H}",
                fn=lambda: xmk.fmha_backward(q, k, v, out, d_o, lse, causal=causal), flops=flops,
                bytes=10.0 * B * N * S * H * 2, bound="mfma", dtype="bf16", kernel="fmha_bwd_kernel (3 launches: dK, dV, dQ)",
                note="flops counted as 5 matrix products (2.5x forward)")


def wl_gemm(torch, xmk, m, n, k, bias=False, rhs_t=False):
    a = gen(torch).normal((m, k), 101, k ** -0.5, dtype=torch.bfloat16)
    b = gen(torch).normal((n, k) if rhs_t else (k, n), 102, k ** -0.5, dtype=torch.bfloat16)
    bv = gen(torch).normal((n,), 103, k ** -0.5, dtype=torch.bfloat16) if bias else None
    out = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    epi = xmk.EPI_BIAS if bias else xmk.EPI_DEFAULT
    return dict(name=f"gemm_bf16_{m}x{n}x{k}{'_bias' if bias else ''}{'_rhsT' if rhs_t else ''}",
                fn=lambda: xmk.run_gemm(a, b, out, rhs_transpose=rhs_t, bias=bv, epilogue=epi),
                flops=2.0 * m * n * k, bytes=2.0 * (m * k + k * n + m * n) + (2 * n if bias else 0),
                bound="mfma", dtype="bf16", kernel="gemm_mfma_kernel")


def wl_fp8(torch, xmk, m, n, k, rhs_t=True):
    a = gen(torch).normal((m, k), 401)
    b = gen(torch).normal((n, k) if rhs_t else (k, n), 402)
    sa, sb = a.abs().max() / 448.0, b.abs().max() / 448.0
    qa, qb = (a / sa).to(torch.float8_e4m3fn), (b / sb).to(torch.float8_e4m3fn)
    sa, sb = sa.reshape(1).float(), sb.reshape(1).float()
    out = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    return dict(name=f"gemm_fp8_e4m3_{m}x{n}x{k}{'_rhsT' if rhs_t else '_rhs_kn'}",
                fn=lambda: xmk.fp8_gemm(qa, qb, sa, sb, out, rhs_transpose=rhs_t),
                flops=2.0 * m * n * k, bytes=1.0 * (m * k + k * n) + 2.0 * m * n, bound="mfma", dtype="fp8",
                kernel="fp8_gemm_kernel")


def wl_int4(torch, xmk, m, k=4096, n=16384, group=128, copies=12):
    # Rotate through `copies` weight sets (12 x 35.7 MB > the 256 MB last-level cache) so that
    # every launch streams its weights from HBM.
    G = gen(torch)
    qws = [G.words((k // 8, n), 300 + 10 * c) for c in range(copies)]
    sc = [G.uniform((k // group, n), 301 + 10 * c, 0.001, 0.02, dtype=torch.float16) for c in range(copies)]
    zp = [G.uniform((k // group, n), 302 + 10 * c, 0.0, 15.0, dtype=torch.float16) for c in range(copies)]
    act = G.normal((m, k), 299, dtype=torch.float16)
    out = torch.empty((m, n), dtype=torch.float16, device="cuda")
    state = [0]

    def fn():
        i = state[0] % copies
        state[0] += 1
        xmk.int4_gemm(act, qws[i], sc[i], zp[i], out, group=group)
    nbytes = k * n / 2 + 2 * (k // group) * n * 2 + 2 * m * k + 2 * m * n
    return dict(name=f"int4_gemm_m{m}_k{k}_n{n}_g{group}", fn=fn, flops=2.0 * m * k * n, bytes=nbytes,
                bound="hbm", dtype="f16", kernel="int4_gemm_kernel", graph=True)


def wl_gemv_f16(torch, xmk, m=1, n=16384, k=4096, copies=4, rhs_t=False):
    """Dense fp16 small-row GEMM, the shape class the reference's own tile table is mostly made of
    (`1_16384_4096`, xla/service/gpu/xetla/gemm/gemm.cc:33): weight-bandwidth bound, so reported as
    HBM GB/s.  K-split through xmk_gemm_ws with caller scratch when the planner asks for one.  The
    launches rotate through `copies` weight sets (4 x 134 MB > the 256 MB last-level cache)."""
    G = gen(torch)
    a = G.normal((m, k), 601, dtype=torch.float16)
    bs = [G.normal((n, k) if rhs_t else (k, n), 602 + c, k ** -0.5, dtype=torch.float16) for c in range(copies)]
    out = torch.empty((m, n), dtype=torch.float16, device="cuda")
    need = xmk.gemm_workspace_bytes(a, bs[0], out, rhs_transpose=rhs_t)
    ws = torch.empty((max(need, 16),), dtype=torch.uint8, device="cuda") if need else None
    state = [0]

    def fn():
        b = bs[state[0] % copies]
        state[0] += 1
        xmk.run_gemm(a, b, out, rhs_transpose=rhs_t, workspace=ws)
    return dict(name=f"gemm_f16_m{m}_n{n}_k{k}{'_rhsT' if rhs_t else ''}", fn=fn, flops=2.0 * m * n * k, bytes=2.0 * (m * k + k * n + m * n),
                bound="hbm", dtype="f16", graph=True,
                kernel=xmk.gemm_policy_name(m, n, k, rhs_t, xmk.F16, xmk.F16) + (" + splitk_reduce_kernel" if need else ""),
                note=f"xmk_gemm_ws, {need} bytes of K-split scratch" if need else "xmk_gemm, unsplit")


def wl_gptj_decode(torch, xmk, n_layer=28, batch=4, cache_len=2047):
    """benchmark configuration 5: GPT-J-6B-shaped decode step, int4 group-128 weights, fp16 KV cache filled to
    `cache_len`, one new token per sequence.  The whole step (about 8 launches per block) is replayed
    from one HIP graph."""
    d, heads, hd, dff, vocab, g = 4096, 16, 256, 16384, 50400, 128
    cap = cache_len + 1

    G, seed = gen(torch), [500]

    def nxt():
        seed[0] += 1
        return seed[0]

    def lin(k, n, bias):
        qw = G.words((k // 8, n), nxt())
        sc = G.uniform((k // g, n), nxt(), 0.001, 0.02, dtype=torch.float16)
        zp = G.uniform((k // g, n), nxt(), 0.0, 15.0, dtype=torch.float16)
        b = G.normal((n,), nxt(), 0.02, dtype=torch.float16) if bias else None
        return qw, sc, zp, b

    layers = []
    for _ in range(n_layer):
        layers.append(dict(ln_gamma=torch.ones((d,), device="cuda").half(), ln_beta=torch.zeros((d,), device="cuda").half(),
                           qkv=lin(d, 3 * d, False), out_proj=lin(d, d, False), fc_in=lin(d, dff, True),
                           fc_out=lin(dff, d, True),
                           k_cache=G.normal((batch, heads, cap, hd), nxt(), dtype=torch.float16),
                           v_cache=G.normal((batch, heads, cap, hd), nxt(), dtype=torch.float16)))
    cfg = xmk.GptjConfig(n_layer, heads, hd, 64, d, dff, vocab, g, batch, cap, 1e-5)
    dec = xmk.GptjDecoder(cfg, layers, torch.ones((d,), device="cuda").half(), torch.zeros((d,), device="cuda").half(),
                          lin(d, vocab, True))
    hidden = G.normal((batch, d), nxt(), dtype=torch.float16)
    logits = torch.empty((batch, vocab), dtype=torch.float16, device="cuda")
    wbytes = n_layer * ((4 * d * d + 2 * d * dff) / 2 + (4 * d * d + 2 * d * dff) / g * 4) \
        + d * vocab / 2 + d * vocab / g * 4
    kvbytes = n_layer * 2.0 * batch * heads * cap * hd * 2
    return dict(name=f"gptj6b_decode_step_int4_l{n_layer}_b{batch}_kv{cache_len}", fn=lambda: dec.step(hidden, cache_len, logits),
                flops=0.0, bytes=wbytes + kvbytes, bound="hbm", dtype="f16", kernel="int4_gemm_kernel + fmha_decode_split_kernel",
                graph=True, graph_steps=3)


def wl_lib_gemm(torch, xmk, m=8192, n=8192, k=8192):
    """torch.matmul (hipBLASLt / rocBLAS behind it) on the 8192^3 shape: what the vendor library reaches on
    the same device in the same run, to read the GEMM kernel's fraction of the published peak against."""
    a = gen(torch).normal((m, k), 101, k ** -0.5, dtype=torch.bfloat16)
    b = gen(torch).normal((k, n), 102, k ** -0.5, dtype=torch.bfloat16)
    out = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    return dict(name=f"library_torch_matmul_bf16_{m}x{n}x{k}", fn=lambda: torch.matmul(a, b, out=out), flops=2.0 * m * n * k,
                bytes=2.0 * (m * k + k * n + m * n), bound="mfma", dtype="bf16", kernel="vendor library GEMM (not this library)")


def wl_copy(torch, xmk, nbytes=1 << 30):
    """A plain device copy of known size: the calibration point for the HBM byte counters."""
    src = torch.empty((nbytes,), dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    return dict(name=f"copy_{nbytes >> 20}MiB", fn=lambda: dst.copy_(src), flops=0.0, bytes=2.0 * nbytes,
                bound="hbm", dtype="u8", kernel="torch copy kernel")


WORKLOADS = {
    "copy": lambda t, x: wl_copy(t, x),
    "fmha_causal": lambda t, x: wl_fmha(t, x, True),
    "fmha": lambda t, x: wl_fmha(t, x, False),
    "fmha_bwd_causal": lambda t, x: wl_fmha_bwd(t, x, True),
    "fmha_bwd": lambda t, x: wl_fmha_bwd(t, x, False),
    "gemm_8192": lambda t, x: wl_gemm(t, x, 8192, 8192, 8192),
    "gemm_8192_rhsT": lambda t, x: wl_gemm(t, x, 8192, 8192, 8192, rhs_t=True),
    "gemm_c1": lambda t, x: wl_gemm(t, x, 512, 4096, 4096, bias=True),
    "lib_gemm_8192": lambda t, x: wl_lib_gemm(t, x),
    "gemv_f16_m1": lambda t, x: wl_gemv_f16(t, x, 1),
    "gemv_f16_m1_rhsT": lambda t, x: wl_gemv_f16(t, x, 1, rhs_t=True),
    "gemv_f16_m4_vocab": lambda t, x: wl_gemv_f16(t, x, 4, 50400, 4096, copies=2),
    "int4_m1": lambda t, x: wl_int4(t, x, 1),
    "int4_m8": lambda t, x: wl_int4(t, x, 8),
    "int4_m32": lambda t, x: wl_int4(t, x, 32),
    "fp8_8192": lambda t, x: wl_fp8(t, x, 8192, 8192, 8192),
    "fp8_8192_kn": lambda t, x: wl_fp8(t, x, 8192, 8192, 8192, rhs_t=False),
    "gptj_decode": lambda t, x: wl_gptj_decode(t, x),
}
ALSO = ["fmha", "fmha_bwd_causal", "gemm_8192", "gemm_8192_rhsT", "lib_gemm_8192", "gemm_c1", "gemv_f16_m1", "gemv_f16_m1_rhsT", "gemv_f16_m4_vocab", "int4_m1", "int4_m8", "int4_m32", "fp8_8192", "fp8_8192_kn", "gptj_decode"]


def measure(torch, xmk, key, steps, warmup):
    w = WORKLOADS[key](torch, xmk)
    if "graph_steps" in w:
        steps, warmup = min(steps, w["graph_steps"]), min(warmup, 1)
    ms, wall_ms = _events(torch, w["fn"], steps, warmup, graph=w.get("graph", False))
    if w["bound"] == "mfma":
        achieved, peak, unit = w["flops"] / ms / 1e9, PEAK["fp8" if w["dtype"] == "fp8" else "bf16"], "TFLOP/s"
    else:
        achieved, peak, unit = w["bytes"] / ms / 1e6, HBM_PEAK, "GB/s"
    roof = {"bound": w["bound"], "achieved": round(achieved, 2), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": TRAFFIC_BYTES.get(key), "kernel": w["kernel"],
            "kernel_ms": round(ms, 5), "algorithmic_flops": w["flops"], "algorithmic_bytes": w["bytes"]}
    if CLOCKS is not None:
        # after the timed region: the same launches back to back while a host thread reads the SMI clocks
        roof["clock_mhz_observed"] = CLOCKS.observe(torch, w["fn"], OBSERVE_SECONDS)
    return w, ms, wall_ms, roof


def _cpu_time(fn, warm, timed):
    for _ in range(warm):
        fn()
    t0 = time.perf_counter()
    for _ in range(timed):
        fn()
    return (time.perf_counter() - t0) / timed


def cpu_baseline(torch):
    """The reference's CPU path for each benchmark configuration, as torch-CPU formulas (jax / jaxlib,
    whose XLA-CPU backend the reference would use, is not installed): a bounded sample of each workload,
    fp32 arithmetic on the rounded inputs, all host threads torch uses.  A reported baseline, not a
    target.  The headline entry is configuration 2; the others are listed under "also"."""
    try:
        import jax  # noqa: F401
        backend = "jax is importable but the harness times torch-CPU formulas"
    except Exception:
        backend = "torch-CPU formulas (jax not installed)"
    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)
    out = {}
    # C2: softmax(mask(Q K^T scale)) V on `units` of the 256 (batch, head) units
    units, S, H = 64, 2048, 128
    q, k, v = (torch.randn((units, S, H), generator=g).bfloat16().float() for _ in range(3))
    mask = torch.ones((S, S), dtype=torch.bool).tril()

    def attn():
        s = torch.baddbmm(torch.zeros(()), q, k.transpose(1, 2), beta=0.0, alpha=H ** -0.5)
        s.masked_fill_(~mask, float("-inf"))
        return torch.softmax(s, -1) @ v
    dt = _cpu_time(attn, 1, 3)
    head = {"value": round(2.0 * units * S * S * H / dt / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "seconds": round(dt, 3), "backend": backend, "os_cpu_count": os.cpu_count(), "torch_num_threads": threads,
            "sample": f"{units} of 256 (batch, head) units of the causal S=2048 D=128 workload, fp32 softmax(mask(QK^T/sqrt(D)))V "
                      f"with causal FLOPs counted as 2*S^2*D per unit"}
    # C1: a @ b + bias, whole problem
    m, n, kk = 512, 4096, 4096
    a, b, bias = torch.randn((m, kk), generator=g), torch.randn((kk, n), generator=g), torch.randn((n,), generator=g)
    dt = _cpu_time(lambda: torch.addmm(bias, a, b), 3, 5)
    out["gemm_bf16_512x4096x4096_bias"] = {"value": round(2.0 * m * n * kk / dt / 1e12, 4), "unit": "TFLOP/s",
                                           "sample": "whole problem, fp32 addmm, 3 warm + 5 timed", "seconds": round(dt, 4)}
    # C1b / C4: 8192^3 is sampled as 1024 rows of A against the whole B (the fp8 one upcasts e4m3 first)
    m, n, kk = 1024, 8192, 8192
    a, b = torch.randn((m, kk), generator=g), torch.randn((kk, n), generator=g)
    dt = _cpu_time(lambda: a @ b, 1, 1)
    out["gemm_bf16_8192x8192x8192"] = {"value": round(2.0 * m * n * kk / dt / 1e12, 4), "unit": "TFLOP/s",
                                       "sample": "1024 of 8192 rows of A against the whole B, fp32 matmul, 1 warm + 1 timed",
                                       "seconds": round(dt, 3)}
    a8, b8 = a.to(torch.float8_e4m3fn), b.to(torch.float8_e4m3fn)
    dt = _cpu_time(lambda: ((a8.float() @ b8.float()) * 0.5).bfloat16(), 1, 1)
    out["gemm_fp8_e4m3_8192x8192x8192"] = {"value": round(2.0 * m * n * kk / dt / 1e12, 4), "unit": "TFLOP/s",
                                           "sample": "1024 of 8192 rows of A: upcast e4m3 -> fp32, matmul, scale, round to bf16",
                                           "seconds": round(dt, 3)}
    # C3: unpack -> dequant -> dot, whole problem
    kk, n, grp = 4096, 16384, 128
    qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (kk // 8, n), dtype=torch.int32, generator=g)
    sc = (torch.rand((kk // grp, n), generator=g) * 0.019 + 0.001).half().float()
    zp = (torch.rand((kk // grp, n), generator=g) * 15).half().float()
    shifts = (torch.arange(8, dtype=torch.int32) * 4).view(1, 8, 1)

    def int4(act):
        qv = ((qw.unsqueeze(1) >> shifts) & 15).reshape(kk, n).float()
        w = (qv - zp.repeat_interleave(grp, 0)) * sc.repeat_interleave(grp, 0)
        return act @ w
    for mm in (1, 8, 32):
        act = torch.randn((mm, kk), generator=g).half().float()
        dt = _cpu_time(lambda: int4(act), 1, 2)
        nbytes = kk * n / 2 + 2 * (kk // grp) * n * 2 + 2 * mm * kk + 2 * mm * n
        out[f"int4_gemm_m{mm}_k4096_n16384_g128"] = {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s",
                                                    "sample": "whole problem: unpack, dequantise, fp32 matmul; 1 warm + 2 timed",
                                                    "seconds": round(dt, 3)}
    # C5: one decoder block of the 28 (its four int4 linears at batch 4 + attention over 2048 cached keys)
    d, dff, heads, hd, B, T = 4096, 16384, 16, 256, 4, 2048
    lin = {}
    for name, (ki, ni) in {"qkv": (d, 3 * d), "out": (d, d), "fc_in": (d, dff), "fc_out": (dff, d)}.items():
        lin[name] = (torch.randint(-2 ** 31, 2 ** 31 - 1, (ki // 8, ni), dtype=torch.int32, generator=g),
                     (torch.rand((ki // grp, ni), generator=g) * 0.019 + 0.001).half().float(),
                     (torch.rand((ki // grp, ni), generator=g) * 15).half().float())
    kc, vc = torch.randn((B, heads, T, hd), generator=g), torch.randn((B, heads, T, hd), generator=g)
    x = torch.randn((B, d), generator=g)

    def dq(name):
        qw_, sc_, zp_ = lin[name]
        qv = ((qw_.unsqueeze(1) >> shifts) & 15).reshape(qw_.shape[0] * 8, qw_.shape[1]).float()
        return (qv - zp_.repeat_interleave(grp, 0)) * sc_.repeat_interleave(grp, 0)

    def block():
        h = torch.nn.functional.layer_norm(x, (d,))
        qkv = h @ dq("qkv")
        qh = qkv[:, :d].view(B, heads, 1, hd)
        p = torch.softmax((qh @ kc.transpose(-1, -2)) * hd ** -0.5, -1)
        att = (p @ vc).reshape(B, d)
        return x + att @ dq("out") + torch.nn.functional.gelu(h @ dq("fc_in"), approximate="tanh") @ dq("fc_out")
    dt = _cpu_time(block, 0, 1)
    out["gptj6b_decode_step_int4_l28_b4_kv2047"] = {"value": round(dt * 28 * 1e3, 1), "unit": "ms per step (28 x the one block timed)",
                                                    "sample": "1 of 28 decoder blocks (lm_head left out): dequantise + fp32 matmul per "
                                                              "linear, attention over 2048 cached keys; 1 timed",
                                                    "seconds": round(dt, 3)}
    head["also"] = out
    return head


def cpu_baseline_oracle(units=32, S=2048, H=128):
    """The C oracle (double accumulation, OpenMP) on a sample of the headline workload, for comparison."""
    import oracle
    q, k, v = (oracle.from_f32(oracle.normal((1, units, S, H), 5 + i), oracle.BF16) for i in range(3))
    t0 = time.perf_counter()
    oracle.fmha_fwd(q, k, v, oracle.BF16, H ** -0.5, causal=True)
    dt = time.perf_counter() - t0
    return {"value": round(2.0 * units * S * S * H / dt / 1e12, 5), "unit": "TFLOP/s", "cores": oracle.num_threads(),
            "kind": "port", "seconds": round(dt, 2),
            "sample": f"{units} of 256 units, oracle/xmk_oracle.c xo_fmha_fwd (OpenMP, double accumulation)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="fmha_causal", choices=sorted(WORKLOADS))
    ap.add_argument("--no-also", action="store_true", help="time only the headline workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--ramp", type=float, default=RAMP_SECONDS,
                    help="seconds of untimed launches before the warmup steps (0 for profiler runs)")
    ap.add_argument("--observe", type=float, default=1.0,
                    help="seconds each workload runs untimed, after its timed steps, while the SMI clocks are sampled "
                         "(0: no sampling, for profiler runs)")
    ap.add_argument("--data", default="seeded", choices=["seeded", "constant"],
                    help="seeded: the parity tests' generator (the benchmark); constant: every operand element equal "
                         "(a power experiment: see class Constant)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no sharding, no collectives); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    globals()["RAMP_SECONDS"] = args.ramp
    globals()["DATA"] = args.data
    import torch
    xmk = importlib.import_module("intel-extension-for-openxla_amd")
    xmk.lib()  # fails loudly if libxmk.so is missing: there is no fallback path
    torch.cuda.set_device(0)

    if args.observe > 0:
        globals()["CLOCKS"] = ClockSampler()
        globals()["OBSERVE_SECONDS"] = args.observe
    w, ms, wall_ms, roof = measure(torch, xmk, args.workload, args.steps, args.warmup)
    line = {
        "metric": "TFLOP/s & %MFMA peak (GEMM/MHA); int4 GEMV HBM GB/s & %peak; 1 GPU",
        "value": roof["achieved"], "unit": roof["unit"], "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall_ms, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": w["dtype"],
        "data": "synthetic" if args.data == "seeded" else "synthetic, constant operands (power experiment, not a benchmark figure)",
        "config": {"workload": w["name"], "note": w.get("note", "")},
        "roofline": roof,
    }
    if not args.no_also:
        also = {}
        for key in ALSO:
            if key == args.workload:
                continue
            torch.cuda.empty_cache()
            w2, ms2, _, roof2 = measure(torch, xmk, key, max(10, args.steps // 2), max(3, args.warmup // 2))
            also[w2["name"]] = roof2
        line["also"] = also
    if CLOCKS is not None and not args.no_also:
        # The headline ran first, from an idle device, and the SMI figures lag by about a second: read its
        # clocks again now that the device has been busy throughout.
        roof["clock_mhz_observed"] = CLOCKS.observe(torch, w["fn"], 2 * OBSERVE_SECONDS)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(torch)
        line["cpu_baseline"]["also"]["oracle_fmha_fwd_causal"] = cpu_baseline_oracle()
    try:
        props = torch.cuda.get_device_properties(0)
        line["device"] = {"name": props.name, "cus": props.multi_processor_count,
                          "clock_mhz_assumed_by_peak": 2400,
                          "clock_mhz_observed": roof.get("clock_mhz_observed", {"source": "not sampled (--observe 0)"}),
                          "note": "the published peaks assume 2400 MHz; each workload's roofline entry carries the clock the "
                                  "SMI library reported while that workload ran"}
    except Exception:  # device query is informational only
        pass
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
