"""The C++ torch.library binding (ao_amd/csrc/torch_binding, built as ao_amd/lib/libao_amd_torch.so): what
torchao/csrc would hold for this path.  It registers torchao::quant_llm_linear with the reference's schema
(torchao/csrc/fp6_llm.cpp:7) for the CUDA dispatch key on top of the C ABI.  The Python package registers the same
operator itself, so the library is loaded in a process that never imports ao_amd.ops; inputs are made through ctypes."""
import os
import subprocess
import sys

import pytest

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_BINDING = os.path.join(_ROOT, "ao_amd", "lib", "libao_amd_torch.so")

_SCRIPT = r'''
import ctypes, importlib.util, os, sys, torch
root = sys.argv[1]
spec = importlib.util.spec_from_file_location("ao_amd_lib_only", os.path.join(root, "ao_amd", "_lib.py"))
_lib = importlib.util.module_from_spec(spec); spec.loader.exec_module(_lib)
L = _lib.lib()
ctypes.CDLL(_lib.LIB_PATH, mode=ctypes.RTLD_GLOBAL)
torch.ops.load_library(os.path.join(root, "ao_amd", "lib", "libao_amd_torch.so"))
assert "ao_amd.ops" not in sys.modules
dev = torch.device("cuda:0"); st = torch.cuda.current_stream().cuda_stream
for (e, m, M, N, K) in [(3, 2, 1, 512, 1024), (2, 3, 5, 256, 512), (3, 2, 64, 1024, 4096)]:
    g = torch.Generator().manual_seed(N + K + M)
    w = (torch.randn(N, K, generator=g) * 0.05).half().to(dev)
    x = torch.randn(M, K, generator=g).half().to(dev)
    nbits = 1 + e + m
    tc = torch.empty(N, K * nbits // 8, dtype=torch.uint8, device=dev)
    scale = torch.empty(N, dtype=torch.float16, device=dev)
    _lib.check(L.ao_amd_fp6_quantize_pack(w.data_ptr(), _lib.F16, N, K, e, m, tc.data_ptr(), scale.data_ptr(), st))
    wd = torch.empty(N, K, dtype=torch.float32, device=dev)
    _lib.check(L.ao_amd_fp6_dequantize(tc.data_ptr(), scale.data_ptr(), N, K, e, m, wd.data_ptr(), st))
    y = torch.ops.torchao.quant_llm_linear(e, m, x, tc, scale, 1)
    ref = x.float() @ wd.half().float().t()   # the kernel multiplies fp16(value * scale)
    err = float((y.float() - ref).norm() / ref.norm())
    print(f"case e{e}m{m} M={M} N={N} K={K}: rel_l2 {err:.2e}", flush=True)
    assert y.dtype is torch.float16 and tuple(y.shape) == (M, N) and err <= 1e-3, err
try:
    torch.ops.torchao.quant_llm_linear(3, 2, x.float(), tc, scale, 1)
    raise SystemExit("a float32 activation was accepted")
except RuntimeError as ex:
    assert "float16" in str(ex)
print("binding ok")
'''


def test_binding_library_is_built_and_links_the_c_abi():
    """CPU: the library exists after build(), depends on libao_amd.so and exports nothing but the registration"""
    assert os.path.exists(_BINDING), "run __graft_entry__.build()"
    out = subprocess.run(["ldd", _BINDING], capture_output=True, text=True).stdout
    assert "libao_amd.so" in out and "libtorch" in out, out


@pytest.mark.gpu
def test_cpp_binding_runs_quant_llm_linear_through_the_dispatcher():
    print("case C++ torch binding in a process of its own", flush=True)
    r = subprocess.run([sys.executable, "-c", _SCRIPT, _ROOT], capture_output=True, text=True, timeout=300)
    print(r.stdout[-2000:], r.stderr[-2000:], flush=True)
    assert r.returncode == 0 and "binding ok" in r.stdout
