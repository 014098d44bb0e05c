"""Builds libnatten_amd.so in-tree with hipcc for gfx950:  python -m natten_amd.build"""

from __future__ import annotations

import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = [os.path.join(_HERE, "csrc", "natten_amd.hip")]
OUTPUT = os.path.join(_HERE, "libnatten_amd.so")

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-shared",
    "-fPIC",
    # keep the compiler from forming packed-fp32 VALU instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # matrix instructions accumulate in ordinary vector registers: kernels that run one wave per
    # SIMD otherwise shuttle their accumulators to and from the accumulation registers every iteration
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
]


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, *SOURCES, "-o", OUTPUT]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed building libnatten_amd.so")
    return OUTPUT


if __name__ == "__main__":
    print(build(verbose=True))
