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


TORCH_BINDING_PATH = os.path.join(LIB_DIR, "libao_amd_torch.so")


def build_torch_binding(verbose: bool = False) -> str:
    """Compiles csrc/torch_binding/*.cpp (the C++ torch.library registration a torchao maintainer would add) against
    the installed libtorch and links it to libao_amd.so.  Host code only: hipcc is used as the C++ compiler so that the
    HIP headers of ATen resolve, no device code is generated.  The Python package does not load the result (it
    registers the same operators itself); tests load it in a process of its own."""
    import torch

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    tdir = os.path.dirname(torch.__file__)
    srcs = sorted(glob.glob(os.path.join(CSRC, "torch_binding", "*.cpp")))
    tmp = TORCH_BINDING_PATH + ".tmp"
    cmd = [hipcc, "-O2", "-std=c++17", "-fPIC", "-shared", "-w", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DHIPBLAS_V2",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-I", os.path.join(tdir, "include"), "-I", os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
           "-I", os.path.join(_HERE, "..", "include"), "-I", os.path.join(os.path.dirname(os.path.dirname(os.path.realpath(hipcc))), "include"),
           "-x", "c++", *srcs, "-o", tmp,
           "-L", os.path.join(tdir, "lib"), "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
           "-L", LIB_DIR, "-lao_amd", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    os.replace(tmp, TORCH_BINDING_PATH)
    return TORCH_BINDING_PATH


CEILINGS_PATH = os.path.join(LIB_DIR, "ao_amd_ceilings")


def build_ubench(verbose: bool = False) -> str:
    """Compiles csrc/ubench/ceilings.hip, the standalone program that measures the fixed costs the kernels are bounded
    by (empty kernel, load-only stream, the GEMV's tile loop on cached weights, LDS reads, grid barriers).  Nothing in
    the package loads it."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(LIB_DIR, exist_ok=True)
    tmp = CEILINGS_PATH + ".tmp"
    cmd = [hipcc, *[f for f in HIPCC_FLAGS if f != "-fPIC"], "-I", os.path.join(_HERE, "..", "include"), "-o", tmp,
           os.path.join(CSRC, "ubench", "ceilings.hip")]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    os.replace(tmp, CEILINGS_PATH)
    return CEILINGS_PATH


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_torch_binding(verbose=True))
    print(build_ubench(verbose=True))
