"""Builds libq8_hip.so (gfx950) from q8_kernels_amd/csrc/*.hip with hipcc.

Usage:  python -m q8_kernels_amd.build        (always recompiles)
The shared library is written next to this file; nothing is installed.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libq8_hip.so")
SOURCES = ["api.hip", "rows.hip", "fused.hip", "elementwise.hip", "gemm.hip", "attn.hip"]
# packed fp32 VALU forms are disabled on purpose (they have miscomputed on this hardware pool)
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src):
    obj = os.path.join(HERE, "build", os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(verbose=True):
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = [o for o, _ in results]
    if verbose:
        for (_, err), src in zip(results, SOURCES):
            if err.strip():
                print("[%s]\n%s" % (src, err), file=sys.stderr)
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
