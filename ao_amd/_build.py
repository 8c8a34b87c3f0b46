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
    # every fp32 op must round on its own: the quantize kernels restate a chain of separate torch ops
    "-ffp-contract=off",
    # hipcc may not form packed fp32 math on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose: bool = False, obj_dir: str = None, only_stale: bool = False) -> str:
    """Compiles every source to an object file (in parallel, one hipcc per source) and links the shared library.
    `obj_dir` keeps the objects (default: a temporary directory); with `only_stale` a source whose object is newer
    than the source and every header is not compiled again (development aid, never used by the build check)."""
    import concurrent.futures
    import tempfile

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(LIB_DIR, exist_ok=True)
    include = os.path.join(_HERE, "..", "include")
    tmp_dir = None
    if obj_dir is None:
        tmp_dir = tempfile.mkdtemp(prefix="ao_amd_build_")
        obj_dir = tmp_dir
    os.makedirs(obj_dir, exist_ok=True)
    headers = glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(CSRC, "*.inc")) + glob.glob(os.path.join(include, "*.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)

    def compile_one(src):
        obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
        if only_stale and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header):
            return obj
        cmd = [hipcc, *HIPCC_FLAGS, "-c", "-I", include, "-o", obj, src]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
        return obj

    try:
        with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
            objs = list(pool.map(compile_one, sources()))
        tmp = LIB_PATH + ".tmp"
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
        os.replace(tmp, LIB_PATH)
    finally:
        if tmp_dir:
            shutil.rmtree(tmp_dir, ignore_errors=True)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
