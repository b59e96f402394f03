"""Build recipe for the gfx950 shared library (liblarql_hip.so, in-tree).

hipcc cross-compiles for gfx950 without a GPU.  The packed-FP32 target feature
is switched off for all device code.
"""
from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "liblarql_hip.so")
SOURCES = ["gemv.hip", "topk.hip", "quantize.hip", "moe.hip", "gemm.hip", "api.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-Wall",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(verbose: bool = False) -> str:
    objs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd))
        r = subprocess.run(cmd, capture_output=True, text=True)
        # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err)
        objs.append(obj)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
