"""Compile the HIP sources in csrc/ into libmlora_hip.so (gfx950), in-tree, with hipcc.

Usage: python build.py [--force]
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmlora_hip.so")
SOURCES = ["api.hip", "gather_mm.hip", "gather_mm_batch.hip", "gemv.hip", "gemm.hip", "rowops.hip", "attention.hip", "decode_step.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-mllvm", "-amdgpu-kernarg-preload-count=16",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _run(cmd):
    p = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass prints a harmless "not a recognized feature" line for the packed-fp32 switch
    err = "\n".join(l for l in p.stderr.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build(force: bool = True, jobs: int = 6) -> str:
    """Compile every source to an object and link the shared library; returns its path."""
    objs = []
    todo = []
    hdr_m = max(os.path.getmtime(os.path.join(CSRC, "common.h")), os.path.getmtime(os.path.join(CSRC, "lora_device.h")),
                os.path.getmtime(os.path.join(CSRC, "gather_mm_batch.h")),
                os.path.getmtime(os.path.join(HERE, "..", "include", "mlora.h")))
    for src in SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(CSRC, src.replace(".hip", ".o"))
        objs.append(o)
        if force or not os.path.exists(o) or os.path.getmtime(o) < max(os.path.getmtime(s), hdr_m):
            todo.append([_hipcc(), *FLAGS, "-c", s, "-o", o])
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(_run, todo))
    if todo or not os.path.exists(LIB):
        _run([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB])
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
