"""Build recipe of libfgnn_hip.so: every csrc/*.hip compiled for gfx950 with hipcc and linked
into one shared library next to this file (in-tree, so it travels with the source tree)."""
from __future__ import annotations

import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libfgnn_hip.so")
OBJ_DIR = os.path.join(HERE, "csrc", "_obj")

HIPCC_FLAGS = [
    "-std=c++20", "-O3", "--offload-arch=gfx950", "-fPIC", "-fvisibility=hidden",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    # packed fp32 VALU ops are kept off for every device function of the library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _compile(src: str, extra) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [_hipcc()] + HIPCC_FLAGS + list(extra) + ["-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 target feature; drop that noise
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err:
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = False, extra_flags=()) -> str:
    """Compile and link unconditionally; returns the library path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    if verbose:
        print("hipcc: %d sources -> %s" % (len(srcs), LIB_PATH))
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(lambda s: _compile(s, extra_flags), srcs))
    cmd = [_hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
