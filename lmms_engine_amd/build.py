"""Builds lmms_engine_amd/libmuon_hip.so from csrc/ with hipcc for gfx950.

Run as `python -m lmms_engine_amd.build` or call build_library().  The library is built
in-tree, next to this file, so it travels with the source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmuon_hip.so")
SOURCES = ["gemm_nt.hip", "elementwise.hip", "multi_tensor.hip", "api.hip"]
# Measurement kernels (MFMA-only loops) for the benchmark's operand-power legs: a library of their own, no part of the product.
PROBE_LIB = os.path.join(HERE, "libmuon_probe.so")
PROBE_SOURCES = ["probe.hip"]
# Packed-fp32 VALU forms stay off for every device function.
HIP_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-fPIC",
    "-std=c++17",
    "-fvisibility=hidden",  # the libraries export their extern "C" entry points and nothing else
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _compile_and_link(sources, lib, hipcc, verbose):
    objdir = os.path.join(CSRC, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    for src in sources:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIP_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    objs = []
    for src, obj, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "not a recognized feature" not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and out.strip():
            print(out)
        objs.append(obj)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", lib]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}")
    return lib


def build_library(verbose: bool = False) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError("hipcc not found; cannot build libmuon_hip.so")
    _compile_and_link(PROBE_SOURCES, PROBE_LIB, hipcc, verbose)
    return _compile_and_link(SOURCES, LIB, hipcc, verbose)


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
