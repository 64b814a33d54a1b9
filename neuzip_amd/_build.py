"""Compile libneuzip_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Nine translation units: nz_launch.hip twice per precision (the encode kernels
and the decode kernels of one kept-mantissa setting) and nz_api.hip (the C ABI
and the kernels all precisions share); they compile side by side and are linked
into one library.
"""
from __future__ import annotations

import os
import shlex
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libneuzip_hip.so")
PRECISIONS = (7, 3, 1, 0)

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-fPIC",
    # no packed-FP32 VALU forms (v_pk_add/mul/fma_f32) in the gfx950 code object:
    # the device pass honours the feature; the x86 host pass of the same command
    # does not know it and says so once ("not a recognized feature for this
    # target"), which run() below leaves out of what it prints
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # float arithmetic as written, whatever the compiler's defaults are: IEEE
    # division where the code divides, gradual underflow (the block normalizers
    # scale bf16 subnormals), no contraction
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-fno-gpu-flush-denormals-to-zero",
    "-ffp-contract=off",
]


def units(objdir: str):
    """(source, extra flags, object file) of every translation unit."""
    out = [(os.path.join(CSRC, "nz_api.hip"), [], os.path.join(objdir, "nz_api.o"))]
    # the lossless precision first: its halves take longest, the pool starts them first
    for s in PRECISIONS:
        for part, tag in ((0, "enc"), (12, "dec")):
            out.append((os.path.join(CSRC, "nz_launch.hip"), [f"-DNZ_S={s}", f"-DNZ_PART={part}"],
                        os.path.join(objdir, f"nz_launch_s{s}_{tag}.o")))
    return out


def run(cmd, verbose: bool) -> None:
    """Run a compiler command; its messages are passed on, the host pass's note
    about the device-only feature aside."""
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, cwd=CSRC, capture_output=True, text=True)
    lines = (res.stdout + res.stderr).splitlines()
    # the note is one line, or two with the count of warnings it caused
    keep = [ln for ln in lines if "-packed-fp32-ops' is not a recognized feature" not in ln
            and ln.strip() != "1 warning generated when compiling for host."]
    if keep:
        print("\n".join(keep), flush=True)
    if res.returncode != 0:
        raise subprocess.CalledProcessError(res.returncode, cmd)


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    with tempfile.TemporaryDirectory(prefix="nz_build_") as objdir:
        tus = units(objdir)

        def compile_one(tu):
            src, extra, obj = tu
            # NZ_HIPCC_EXTRA: more flags for a measurement build (e.g. -DNZ_PROBE_EXTRA_SLOTS)
            more = shlex.split(os.environ.get("NZ_HIPCC_EXTRA", ""))
            run([hipcc, *HIPCC_FLAGS, *extra, *more, "-c", src, "-o", obj], verbose)
            return obj

        with ThreadPoolExecutor(max_workers=min(len(tus), os.cpu_count() or 4)) as pool:
            objs = list(pool.map(compile_one, tus))
        run([hipcc, "--offload-arch=gfx950", "-fPIC", "-shared", *objs, "-o", LIB_PATH], verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
