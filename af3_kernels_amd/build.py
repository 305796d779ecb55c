"""Builds libaf3_dpa.so (hand-written HIP for gfx950) in-tree with hipcc.

    python -m af3_kernels_amd.build [--force]

The library is linked from one object per source file so that an edit recompiles one file.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJDIR = os.path.join(CSRC, "_obj")
LIB = os.path.join(HERE, "libaf3_dpa.so")
SOURCES = ["api.hip", "dpa_generic.hip", "dpa_mfma.hip", "dpa_mfma_rows.hip", "dpa_mfma_f32.hip", "dpa_mfma_fp8.hip", "elementwise.hip", "pair_bias.hip", "glu.hip"]
HEADERS = [os.path.join(CSRC, "common.hpp"), os.path.join(CSRC, "mfma_helpers.hpp"), os.path.join(HERE, "..", "include", "af3_dpa.h")]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed-fp32 ops are switched off for device code; the host pass warns that it does not know
# the feature, which is harmless.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, force):
    obj = os.path.join(OBJDIR, src + ".o")
    path = os.path.join(CSRC, src)
    if force or _stale(obj, [path] + HEADERS):
        r = subprocess.run([HIPCC] + FLAGS + ["-c", path, "-o", obj], capture_output=True, text=True)
        msgs = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if "packed-fp32-ops" not in l and l.strip())
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{msgs}")
        if msgs:
            print(msgs, file=sys.stderr)
    return obj


def build(force=False, verbose=False):
    os.makedirs(OBJDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES) + 1)) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), SOURCES))
    if force or _stale(LIB, objs):
        r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv, verbose=True)
