"""The C++ torch.library binding (ao_amd/csrc/torch_binding, built as ao_amd/lib/libao_amd_torch.so): what
torchao/csrc would hold for this path.  It registers torchao::quant_llm_linear with the reference's schema
(torchao/csrc/fp6_llm.cpp:7), torchao::int4wo_quantize_pack and torchao::int4wo_linear for the CUDA and Meta dispatch
keys on top of the C ABI.  The Python package registers the same operators itself, so the library is loaded in a process
that never imports ao_amd.ops; inputs are made through ctypes.  The operators go through torch.library.opcheck as the
reference's own do (test/test_ops.py:35-45)."""
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
def refused(fn, text):
    try:
        fn()
    except RuntimeError as ex:
        assert text in str(ex), str(ex)
        return
    raise SystemExit("accepted: " + text)
refused(lambda: torch.ops.torchao.quant_llm_linear(3, 2, x.float(), tc, scale, 1), "FP16")
refused(lambda: torch.ops.torchao.quant_llm_linear(3, 2, x, tc.view(torch.int8), scale, 1), "UINT8")
refused(lambda: torch.ops.torchao.quant_llm_linear(3, 2, x, tc[:, :-8].contiguous(), scale, 1), "Dimensions mismatched")
refused(lambda: torch.ops.torchao.quant_llm_linear(3, 2, x, tc, scale[:-1], 1), "Dimensions mismatched")
# the re-tiled weight is kept per weight tensor: same answer on the second call, a new one after an in-place write
y1 = torch.ops.torchao.quant_llm_linear(e, m, x, tc, scale, 1)
assert torch.equal(y1, y)
tc2 = tc.clone(); tc.zero_()          # version bump: all codes +0
y0 = torch.ops.torchao.quant_llm_linear(e, m, x, tc, scale, 1)
assert float(y0.float().abs().max()) == 0.0
tc.copy_(tc2)
assert torch.equal(torch.ops.torchao.quant_llm_linear(e, m, x, tc, scale, 1), y)
# the int4 operators through the dispatcher
for (M, N, K, g) in [(1, 512, 1024, 64), (5, 300, 512, 128), (70, 1024, 4096, 64)]:
    gen = torch.Generator().manual_seed(N + K + M)
    w = (torch.randn(N, K, generator=gen) * 0.02).bfloat16().to(dev)
    xb = torch.randn(M, K, generator=gen).bfloat16().to(dev)
    packed, qp = torch.ops.torchao.int4wo_quantize_pack(w, g)
    p_ref = torch.empty_like(packed); q_ref = torch.empty_like(qp)
    _lib.check(L.ao_amd_int4wo_quantize_pack(w.data_ptr(), N, K, K, g, p_ref.data_ptr(), q_ref.data_ptr(), st))
    assert torch.equal(packed, p_ref) and torch.equal(qp, q_ref)
    dq = torch.empty(N, K, dtype=torch.bfloat16, device=dev)
    _lib.check(L.ao_amd_int4wo_dequantize(packed.data_ptr(), qp.data_ptr(), N, K, g, dq.data_ptr(), st))
    b = torch.randn(N, generator=gen).bfloat16().to(dev)
    y32 = torch.ops.torchao.int4wo_linear(xb, packed, qp, g, N, b, True)
    ref = xb.float() @ dq.float().t() + b.float()
    err = float((y32 - ref).norm() / ref.norm())
    y16 = torch.ops.torchao.int4wo_linear(xb, packed, qp, g, N, None, False)
    ref16 = (xb.float() @ dq.float().t()).bfloat16().float()
    err16 = float((y16.float() - ref16).norm() / ref16.norm())
    print(f"case int4 M={M} N={N} K={K} g={g}: rel_l2 {err:.2e} / {err16:.2e}", flush=True)
    assert y32.dtype is torch.float32 and err <= 2e-5 and y16.dtype is torch.bfloat16 and err16 <= 1e-3
    # meta device: shapes and dtypes without a launch
    pm, qm = torch.ops.torchao.int4wo_quantize_pack(w.to("meta"), g)
    assert pm.shape == packed.shape and qm.shape == qp.shape and pm.dtype is torch.int32 and pm.device.type == "meta"
    ym = torch.ops.torchao.int4wo_linear(xb.to("meta"), pm, qm, g, N, None, False)
    assert ym.shape == y16.shape and ym.dtype is torch.bfloat16
refused(lambda: torch.ops.torchao.int4wo_linear(xb.float(), packed, qp, g, N, None, False), "bfloat16")
refused(lambda: torch.ops.torchao.int4wo_linear(xb, packed[:-1], qp, g, N, None, False), "packed weight must be")
# torch.library.opcheck, as the reference's test/test_ops.py:35-45 runs it on its operator
utils = ["test_schema", "test_autograd_registration", "test_faketensor", "test_aot_dispatch_dynamic"]
torch.library.opcheck(torch.ops.torchao.quant_llm_linear.default, (e, m, x, tc, scale, 1), test_utils=utils)
torch.library.opcheck(torch.ops.torchao.int4wo_quantize_pack.default, (w, g), test_utils=utils)
torch.library.opcheck(torch.ops.torchao.int4wo_linear.default, (xb, packed, qp, g, N, b, False), test_utils=utils)
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
    first_error = r.stderr.find("Error")
    print(r.stdout[-2000:], r.stderr[max(0, first_error - 300):first_error + 1500] if first_error >= 0 else r.stderr[-1500:], flush=True)
    assert r.returncode == 0 and "binding ok" in r.stdout
