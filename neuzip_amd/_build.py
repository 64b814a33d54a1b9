"""Compile libneuzip_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
from __future__ import annotations

import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libneuzip_hip.so")

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # no packed-FP32 VALU forms (v_pk_add/mul/fma_f32) in the gfx950 code object:
    # the device pass honours the feature; the x86 host pass of the same command
    # does not know it and prints "not a recognized feature for this target
    # (ignoring feature)" once per pass, which is harmless
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # float arithmetic as written, whatever the compiler's defaults are: IEEE
    # division where the code divides (the coder's reciprocal table), gradual
    # underflow (the block normalizers scale bf16 subnormals), no contraction
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-fno-gpu-flush-denormals-to-zero",
    "-ffp-contract=off",
]


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, os.path.join(CSRC, "nz_api.hip"), "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd, cwd=CSRC)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
