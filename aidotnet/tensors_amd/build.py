"""Builds ``libaidotnet_mi355.so`` (gfx950 only) in-tree with hipcc.

Run as ``python -m aidotnet.tensors_amd.build``; ``__graft_entry__.build()`` calls
:func:`build_library`.  hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libaidotnet_mi355.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["gemm.hip", "attention.hip", "decode.hip", "convert.hip", "api.hip"]
# -packed-fp32-ops off: packed fp32 VALU forms are kept out of all device code.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src: str, obj: str) -> None:
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stderr[-4000:]))


def build_library(verbose: bool = False, jobs: int = 5) -> str:
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    pairs = [(os.path.join(CSRC, s), os.path.join(objdir, s.replace(".hip", ".o"))) for s in SOURCES]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda p: _compile(*p), pairs))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + [o for _, o in pairs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s" % r.stderr[-4000:])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print("built", LIB_PATH, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
