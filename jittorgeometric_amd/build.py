"""Compiles the HIP sources under csrc/ into libjgamd.so (gfx950 only).

hipcc cross-compiles without a GPU.  The library is built in-tree, next to
this file, and is what `jittorgeometric_amd._lib` loads.
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libjgamd.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # packed fp32 VALU forms are switched off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _compile(src):
    obj = os.path.join(CSRC, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    p = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in p.stderr.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
    return obj, err


def build(verbose=False):
    """Always recompiles every source, then links."""
    srcs = sources()
    if not srcs:
        raise RuntimeError("no HIP sources under " + CSRC)
    # a library from older sources must not survive a failed build: the ctypes signatures follow
    # the sources, and a call through a stale entry point would pass the wrong arguments
    if os.path.exists(LIB):
        os.remove(LIB)
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        results = list(ex.map(_compile, srcs))
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            if err.strip():
                print(err, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0:
        raise RuntimeError("link failed:\n" + p.stderr)
    for o in objs:
        os.remove(o)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
