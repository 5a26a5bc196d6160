"""Builds libxmk.so (the C-ABI kernel library) for gfx950 with hipcc, in-tree.

Usage: python build.py [-j N] [--force]   (without --force: incremental)
Each translation unit under csrc/ is compiled to an object file and the objects
are linked into one shared library next to this file.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libxmk.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I", INCLUDE, "-I", CSRC,
         # packed-fp32 VALU forms are kept out of generated code on purpose
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes"] + os.environ.get("XMK_CXXFLAGS", "").split()


# Per-file flags.  fmha_fwd.hip: matrix instructions write VGPRs, so that the softmax reads the
# scores where they were produced (the whole register budget is then one file of 256 per wave).
EXTRA = {"fmha_fwd.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".cc")))


def _deps_mtime():
    hdrs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hdrs += [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE)]
    return max(os.path.getmtime(h) for h in hdrs)


def _compile(args):
    src, force = args
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    spath = os.path.join(CSRC, src)
    if (not force and os.path.exists(obj)
            and os.path.getmtime(obj) > max(os.path.getmtime(spath), _deps_mtime())):
        return src, obj, 0, ""
    cmd = [HIPCC] + FLAGS + EXTRA.get(src, []) + (["-x", "hip"] if src.endswith(".cc") else []) + \
          ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    return src, obj, r.returncode, out


def build(jobs=None, verbose=False, force=True):
    """force=False recompiles only sources newer than their object file."""
    os.makedirs(OBJ, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for src, obj, rc, out in pool.map(_compile, [(s, force) for s in sources()]):
            if out and (verbose or rc != 0):
                print(f"--- {src}\n{out}", file=sys.stderr)
            if rc != 0:
                raise RuntimeError(f"hipcc failed on {src}")
            objs.append(obj)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    j = int(sys.argv[sys.argv.index("-j") + 1]) if "-j" in sys.argv else None
    print(build(j, verbose=True, force="--force" in sys.argv))
