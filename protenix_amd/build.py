"""Builds protenix_amd/libprotenix_amd.so from csrc/*.hip with hipcc for gfx950.

Run as ``python -m protenix_amd.build``.  hipcc cross-compiles, so no GPU is
needed; the library is left in-tree next to this file.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libprotenix_amd.so")
SOURCES = ["api.hip", "layernorm.hip", "rowgemm.hip", "triattn.hip", "attnpack.hip", "attnbwd.hip", "attnout.hip", "ntgemm.hip", "transition.hip", "single.hip", "stream.hip"]
# per-source extra flags (none: the attention core's redo checks of the form !(x < limit) are
# what catches a NaN logit, so it is built with NaNs honoured like everything else)
EXTRA_FLAGS = {}
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; cannot build libprotenix_amd.so")
    return exe


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), err))
    return err


def build(verbose: bool = False) -> str:
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    jobs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        for src in SOURCES:
            obj = os.path.join(objdir, src.replace(".hip", ".o"))
            objs.append(obj)
            cmd = [hipcc, *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
            jobs.append(pool.submit(_run, cmd))
        for j in jobs:
            msg = j.result()
            if verbose and msg:
                print(msg, file=sys.stderr)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
