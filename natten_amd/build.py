"""Builds libnatten_amd.so in-tree with hipcc for gfx950:  python -m natten_amd.build

  python -m natten_amd.build --ablate N --output PATH
builds a timing-only library instead (NATTEN_AMD_ABLATE = N leaves parts of the forward kernel's
tile loop out, see csrc/fna_fwd.hpp; its results are wrong by design).  NATTEN_AMD_LIBRARY=PATH makes
the package load such a library in place of the shipped one."""

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


def build(verbose: bool = False, ablate: int = 0, output: str = OUTPUT) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if ablate and os.path.abspath(output) == OUTPUT:
        raise ValueError("a timing-only build must not replace the shipped library: give --output")
    defines = [f"-DNATTEN_AMD_ABLATE={int(ablate)}"] if ablate else []
    cmd = [hipcc, *HIPCC_FLAGS, *defines, *SOURCES, "-o", output]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed building libnatten_amd.so")
    return output


if __name__ == "__main__":
    import argparse

    ap = argparse.ArgumentParser()
    ap.add_argument("--ablate", type=int, default=0, help="NATTEN_AMD_ABLATE mask of a timing-only build")
    ap.add_argument("--output", default=OUTPUT)
    a = ap.parse_args()
    print(build(verbose=True, ablate=a.ablate, output=a.output))
