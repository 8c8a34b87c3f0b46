"""Builds ao_amd/lib/libao_amd.so from the HIP sources in ao_amd/csrc with hipcc for gfx950.

hipcc cross-compiles, so this runs on a machine without a GPU.  The library links against the HIP
runtime only (no torch), which keeps the C ABI independent of the PyTorch build.
"""
import glob
import os
import shutil
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libao_amd.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # every fp32 op must round on its own: the quantize kernels restate a chain of separate torch ops
    "-ffp-contract=off",
    # hipcc may not form packed fp32 math on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose: bool = False) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(LIB_DIR, exist_ok=True)
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc, *HIPCC_FLAGS, "-I", os.path.join(_HERE, "..", "include"), "-o", tmp, *sources()]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
