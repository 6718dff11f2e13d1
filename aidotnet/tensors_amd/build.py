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
# (source, object name, extra flags): gemm.hip is compiled in three parts so that its template instances build in parallel
SOURCES = [("gemm.hip", "gemm.o", ["-DAIDN_GEMM_PART=0"]), ("gemm.hip", "gemm_f16.o", ["-DAIDN_GEMM_PART=1"]),
           ("gemm.hip", "gemm_bf16.o", ["-DAIDN_GEMM_PART=2"]), ("attention.hip", "attention.o", []), ("attention_prefill.hip", "attention_prefill.o", []),
           ("decode.hip", "decode.o", []),
           ("convert.hip", "convert.o", []), ("api.hip", "api.o", [])]
# -packed-fp32-ops off: packed fp32 VALU forms are kept out of all device code.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src: str, obj: str, extra=()) -> None:
    # the resource-usage remarks name every kernel with its register and scratch use: a kernel that needs scratch memory has
    # spilled registers (for the GEMM kernels that means accumulators in memory and a 30-fold slowdown), so the build refuses it
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-Rpass-analysis=kernel-resource-usage", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stderr[-4000:]))
    spilled = kernels_with_scratch(r.stderr)
    if spilled:
        raise RuntimeError("%s: kernels that spill registers to scratch memory:\n  %s"
                           % (src, "\n  ".join("%s (%d bytes/lane)" % kv for kv in spilled)))


def kernels_with_scratch(remarks: str):
    """(kernel name, scratch bytes per lane) of every kernel in hipcc's kernel-resource-usage remarks that uses scratch."""
    out, name = [], None
    for line in remarks.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line and name is not None:
            n = int(line.split("ScratchSize [bytes/lane]:")[1].split("[")[0].strip())
            if n > 0:
                out.append((name, n))
    return out


def _stale(src: str, obj: str) -> bool:
    """True when `obj` is older than its source or than any header the sources share."""
    if not os.path.exists(obj):
        return True
    deps = [src] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hpp", ".h", ".inc"))]
    deps.append(os.path.join(os.path.dirname(os.path.dirname(HERE)), "include", "aidotnet_mi355.h"))
    return any(os.path.getmtime(d) > os.path.getmtime(obj) for d in deps if os.path.exists(d))


def build_library(verbose: bool = False, jobs: int = 8, incremental: bool = False) -> str:
    """Compiles every source (always, unless `incremental`: then only those newer than their object file) and links."""
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    pairs = [(os.path.join(CSRC, s), os.path.join(objdir, o), x) for s, o, x in SOURCES]
    todo = [p for p in pairs if not incremental or _stale(p[0], p[1])]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda p: _compile(*p), todo))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + [o for _, o, _ in pairs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s" % r.stderr[-4000:])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print("built", LIB_PATH, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True, incremental="--incremental" in sys.argv[1:]))
