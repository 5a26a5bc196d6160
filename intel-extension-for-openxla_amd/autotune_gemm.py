"""Offline GEMM tile autotuner: times every tile policy on a list of (m, n, k) shapes and writes
csrc/gemm_policy_table.h with the shapes where the heuristic's choice is not the fastest.

    python autotune_gemm.py [--shapes m,n,k ...] [--dry-run]
    python autotune_gemm.py --small [--shapes m,n,k ...] [--dry-run]

--small tunes the decode-sized row counts (m = 1 .. 32) of the same list over tile policy x number of K
slices (xmk_gemm_ws with scratch; XMK_GEMM_SPLITK forces the slices) and merges the winners into the table.

The counterpart of the reference's tuned table (xetla/gemm/gemm.cc:31-285) and of its
GemmAlgorithmPicker measurement loop (gemm_impl_picker.cc:124-185).  The measurements run in worker
processes (XMK_GEMM_POLICY / XMK_GEMM_SPLITK force a choice); the parent never touches the GPU.
Rebuild the library afterwards (python build.py) for the table to take effect.
"""
import argparse
import importlib
import json
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
TABLE = os.path.join(HERE, "csrc", "gemm_policy_table.h")
POLICIES = ["mfma_256x256x32_w2x2_s4", "mfma_128x128x64_w2x2_s3", "mfma_128x64x64_w2x2_s4", "mfma_64x64x64_w2x2_s4",
            "mfma_256x128x64_w2x2_s3", "stream_rows_8x512_w8"]
TILES = [(256, 256), (128, 128), (128, 64), (64, 64), (256, 128)]  # the matrix-core policies (the heuristic's candidates)
# The last policy is the streaming kernel for up to eight rows: forced on a shape it cannot take, the library
# falls back to its own choice, so such a candidate simply repeats the default's time.
MFMA_POLICIES = len(TILES)

# (n, k) pairs of the reference's LLM shape list (gemm.cc:31-285) that fit the medium/large-M tiles,
# plus the benchmark shapes.
NK = [(4096, 4096), (11008, 4096), (4096, 11008), (16384, 4096), (4096, 16384), (5120, 5120), (13824, 5120),
      (5120, 13824), (8192, 8192), (7168, 8192), (8192, 7168), (14336, 7168), (7168, 14336), (12288, 4096)]
MS = [64, 128, 256, 512, 1024, 2048, 4096]
DEFAULT_SHAPES = [(m, n, k) for m in MS for (n, k) in NK] + [(8192, 8192, 8192)]
# Decode-sized shapes: the m = 1, 4, 32 rows of gemm.cc:33-47 and the row counts between, on the GPT-J
# projections (4096 x 4096, 4096 -> 16384, 16384 -> 4096, the stacked q/k/v 4096 -> 12288).
SMALL_NK = [(4096, 16384), (16384, 4096), (4096, 4096), (12288, 4096)]
SMALL_MS = [1, 4, 8, 16, 32]
# The vocabulary projections that fill the reference's table for m = 1, 4 (gemm.cc:77-80, 92-93, 112-113);
# 50400 = 787.5 x 64 is ragged in every tile width.
VOCAB_NK = [(50400, 4096), (50272, 4096), (32000, 4096), (65024, 4096)]
VOCAB_MS = [1, 4, 32]
SMALL_SHAPES = [(m, n, k) for m in SMALL_MS for (n, k) in SMALL_NK] + [(m, n, k) for m in VOCAB_MS for (n, k) in VOCAB_NK]
SPLITS = [1, 2, 4, 8, 16]


TILE_RATE = [1.0, 0.75, 0.60, 0.55, 0.90]


def heuristic(m, n, k):
    """select_policy's heuristic (csrc/gemm_kernel.h), restated."""
    best, best_score = len(TILES) - 1, -1.0
    for i, (bm, bn) in enumerate(TILES):
        tiles = -(-m // bm) * -(-n // bn)
        waves = -(-tiles // 256)
        score = TILE_RATE[i] * (tiles / (waves * 256)) * (m * n / (tiles * bm * bn))
        if score > best_score:
            best, best_score = i, score
    return best


def worker_small(shapes):
    """Times xmk_gemm_ws (scratch for up to 16 slices) from a HIP graph of 20 launches per replay, for the
    library's own choice and for every tile policy x number of K slices (XMK_GEMM_POLICY / XMK_GEMM_SPLITK
    are read at every call, so one process walks them all)."""
    sys.path.insert(0, os.path.dirname(HERE))
    import torch
    xmk = importlib.import_module(os.path.basename(HERE))
    cands = [None] + [(pol, ks) for pol in range(len(POLICIES)) for ks in SPLITS]
    out = {("default" if c is None else f"{c[0]}x{c[1]}"): {} for c in cands}
    for (m, n, k) in shapes:
        a = (torch.randn((m, k), device="cuda") * k ** -0.5).bfloat16()
        copies = max(2, min(4, int(6e8 // (2 * n * k)) + 1))  # rotate past the 256 MB cache
        bs = [(torch.randn((k, n), device="cuda") * k ** -0.5).bfloat16() for _ in range(copies)]
        c = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        ws = torch.empty((16 * m * n,), dtype=torch.float32, device="cuda")
        for cand in cands:
            for var in ("XMK_GEMM_POLICY", "XMK_GEMM_SPLITK"):
                os.environ.pop(var, None)
            if cand is not None:
                os.environ["XMK_GEMM_POLICY"], os.environ["XMK_GEMM_SPLITK"] = str(cand[0]), str(cand[1])
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                for b in bs:
                    xmk.run_gemm(a, b, c, workspace=ws)
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=st):
                    for i in range(20):
                        xmk.run_gemm(a, bs[i % copies], c, workspace=ws)
            torch.cuda.synchronize()
            g.replay()
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            best = 1e30
            for _ in range(5):
                s.record()
                g.replay()
                e.record()
                torch.cuda.synchronize()
                best = min(best, s.elapsed_time(e) / 20)
            out["default" if cand is None else f"{cand[0]}x{cand[1]}"][f"{m},{n},{k}"] = best
            del g
        print(f"shape {m},{n},{k} measured", file=sys.stderr, flush=True)
    print("RESULT " + json.dumps(out), flush=True)


def run_worker(shapes, env_extra, flag):
    env = dict(os.environ, **env_extra)
    cmd = [sys.executable, os.path.abspath(__file__), flag, "--shapes"] + [f"{m},{n},{k}" for m, n, k in shapes]
    r = subprocess.run(cmd, env=env, stdout=subprocess.PIPE, text=True, timeout=1100)
    line = [l for l in r.stdout.splitlines() if l.startswith("RESULT ")]
    if r.returncode != 0 or not line:
        sys.exit(f"worker {env_extra} failed:\n{r.stdout[-2000:]}")
    return json.loads(line[0][7:])


def load_table():
    """(m, n, k) -> (policy, ksplit, comment) of the table as it stands."""
    rows = {}
    if os.path.exists(TABLE):
        for l in open(TABLE):
            m = re.match(r"\s*\{(\d+), (\d+), (\d+), (\d+), (\d+)\},\s*//\s*(.*)", l)
            if m and int(m.group(1)) > 0:
                rows[(int(m.group(1)), int(m.group(2)), int(m.group(3)))] = (int(m.group(4)), int(m.group(5)), m.group(6))
    return rows


def write_table(rows):
    with open(TABLE, "w") as f:
        f.write("// Tuned (m, n, k) -> {policy index, K slices} table.  GENERATED by autotune_gemm.py; do not edit by hand.\n")
        f.write("// Shapes where a choice other than the heuristic's was measured faster on an MI355X (bf16, row-major\n")
        f.write("// operands).  K slices 0: tile policy only (TFLOP/s heuristic -> chosen); K slices >= 1: the number of\n")
        f.write("// slices and their tile for xmk_gemm_ws (microseconds default -> chosen).\n")
        f.write("constexpr TunedShape kTunedShapes[] = {\n")
        for (m, n, k) in sorted(rows):
            pol, ks, note = rows[(m, n, k)]
            f.write(f"    {{{m}, {n}, {k}, {pol}, {ks}}},  // {note}\n")
        f.write("    {0, 0, 0, 0, 0},\n};\n")
    print(f"wrote {TABLE}: {len(rows)} shapes")


def tune_small(shapes, args):
    res = run_worker(shapes, {}, "--worker-small")
    base = res.pop("default")
    cand = {tuple(int(x) for x in key.split("x")): v for key, v in res.items()}
    rows = load_table()
    for (m, n, k) in shapes:
        key = f"{m},{n},{k}"
        # (the streaming kernel takes at most eight rows: with more, that candidate only repeats the default)
        usable = [c for c in cand if c[0] < MFMA_POLICIES or m <= 8]
        best = min(usable, key=lambda c: cand[c][key])
        t0, t1 = base[key] * 1e3, cand[best][key] * 1e3
        gbs = 2.0 * (m * k + k * n + m * n) / t0 / 1e3
        print(f"{key:>18}: default {t0:7.2f} us ({gbs:5.0f} GB/s)  best {t1:7.2f} us  = {POLICIES[best[0]]} x {best[1]} slices")
        rows.pop((m, n, k), None)
        if t1 < t0 * (1.0 - args.margin):
            rows[(m, n, k)] = (best[0], best[1], f"{t0:.1f} -> {t1:.1f} us")
    if not args.dry_run:
        write_table(rows)


def worker(shapes):
    sys.path.insert(0, os.path.dirname(HERE))
    import torch
    xmk = importlib.import_module(os.path.basename(HERE))
    out = {}
    for (m, n, k) in shapes:
        a = (torch.randn((m, k), device="cuda") * k ** -0.5).bfloat16()
        b = (torch.randn((k, n), device="cuda") * k ** -0.5).bfloat16()
        c = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        for _ in range(3):
            xmk.run_gemm(a, b, c)
        iters = max(5, min(50, int(2e12 / (2.0 * m * n * k))))
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        best = 1e30
        for _ in range(3):
            s.record()
            for _ in range(iters):
                xmk.run_gemm(a, b, c)
            e.record()
            torch.cuda.synchronize()
            best = min(best, s.elapsed_time(e) / iters)
        out[f"{m},{n},{k}"] = best
    print("RESULT " + json.dumps(out), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--shapes", nargs="*", help="m,n,k triples (default: the built-in LLM shape list)")
    ap.add_argument("--worker", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--worker-small", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--small", action="store_true", help="tune m = 1 .. 32 over tile policy x K slices")
    ap.add_argument("--dry-run", action="store_true", help="measure and print, do not write the table")
    ap.add_argument("--margin", type=float, default=0.03, help="ignore wins smaller than this fraction")
    args = ap.parse_args()
    default = SMALL_SHAPES if (args.small or args.worker_small) else DEFAULT_SHAPES
    shapes = [tuple(int(x) for x in s.split(",")) for s in args.shapes] if args.shapes else default
    if args.worker:
        worker(shapes)
        return
    if args.worker_small:
        worker_small(shapes)
        return
    if args.small:
        tune_small(shapes, args)
        return
    times = []
    for pol in range(MFMA_POLICIES):
        times.append(run_worker(shapes, {"XMK_GEMM_POLICY": str(pol)}, "--worker"))
        print(f"policy {pol} ({POLICIES[pol]}) measured", flush=True)
    rows = []
    for (m, n, k) in shapes:
        key = f"{m},{n},{k}"
        t = [times[p][key] for p in range(MFMA_POLICIES)]
        best, h = min(range(len(t)), key=lambda i: t[i]), heuristic(m, n, k)
        tf = [2.0 * m * n * k / x / 1e9 for x in t]
        print(f"{key:>18}: " + " ".join(f"{x:7.1f}" for x in tf) + f"  TFLOP/s  heuristic {h} best {best}")
        if best != h and t[best] < t[h] * (1.0 - args.margin):
            rows.append((m, n, k, best, tf[h], tf[best]))
    if args.dry_run:
        return
    table = {key: v for key, v in load_table().items() if v[1] != 0 or key not in set(shapes)}
    for (m, n, k, best, a, b) in rows:
        table[(m, n, k)] = (best, 0, f"{a:.0f} -> {b:.0f}")
    write_table(table)


if __name__ == "__main__":
    main()
