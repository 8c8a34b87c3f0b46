"""Every kernel instantiation the FPx linear dispatch can select is reached by a GPU test, as for the int4 linear
(tests/test_dispatch_gpu.py): `ao_amd_fp6_linear_plan` answers on the host which instantiation a problem runs, the CPU
test walks a grid of problems and pins the families, the GPU test takes the smallest problem of the grid that reaches
each instantiation and checks it: one-hot activation rows must return columns of fp16(value * scale) bit for bit (the
kernel's conversion and its single fp16 rounding, torchao/csrc/cuda/fp6_llm/utils_parallel_dequant.cuh:47-59), random rows
must agree with an fp32 matmul on the dequantized weight to 1e-3 relative L2 and to the reference test's mean relative
error < 1e-3 (test/test_ops.py:47-62).  The batch buckets of the reference's launcher (fp6_linear.cu:72-93: up to 8, 16,
32, 64 rows, then tiles of 128) all appear in the row counts walked."""
import functools
import itertools

import pytest
import torch

SHAPES = [(256, 512), (1024, 1024), (2048, 4096), (4096, 4096), (6144, 4096), (14336, 4096), (4096, 14336), (28672, 4096),
          (128256, 4096)]   # (N, K)
MS = [1, 2, 3, 4, 8, 16, 17, 24, 32, 33, 64, 65, 128, 256, 512, 1024]
FORMATS = [(3, 2), (2, 3)]   # the two conversion paths; e2m2 / e3m1 are stored as the 6-bit code of the same value


@functools.lru_cache(maxsize=None)
def _walk():
    """plan name -> smallest problem (M, K, N, ebits, mbits, norm, dual) of the grid that reaches it"""
    from ao_amd import _lib

    best = {}
    for (N, K), M, (e, m), fused in itertools.product(SHAPES, MS, FORMATS, ("", "norm", "dual")):
        if fused and (M > 16 or K > 8192):
            continue
        if N * M > (1 << 25):
            continue
        try:
            name = _lib.fp6_linear_plan(M, K, N, e, m, norm=bool(fused), dual=fused == "dual")
        except _lib.AoAmdError:
            continue
        cost = N * K * (1 + M // 64)
        if name not in best or cost < best[name][0]:
            best[name] = (cost, (M, K, N, e, m, bool(fused), fused == "dual"))
    return {k: v[1] for k, v in best.items()}


def test_dispatch_walk_finds_every_kernel_family():
    from ao_amd import _lib

    plans = _walk()
    assert {n.split("<")[0] for n in plans} == {"fp6_gemv_kernel", "fp6_linear_kernel", "fp6_linear_mb_kernel", "fp6_gemm_kernel"}
    for e3 in (0, 1):
        for tile in ("2,8,2,1", "1,4,4,4", "1,2,8,8"):
            assert "fp6_gemm_kernel<%d,%s>" % (e3, tile) in plans
        for w in (4, 8):
            assert "fp6_linear_mb_kernel<%d,%d,2>" % (w, e3) in plans
        for w in (1, 2, 4, 8, 16):
            assert "fp6_gemv_kernel<%d,%d,0>" % (w, e3) in plans, (w, e3)
        assert any(n.startswith("fp6_gemv_kernel<") and n.endswith(",%d,1>" % e3) for n in plans)   # two weights + SwiGLU
        for rbw in (1, 2, 4):
            assert any(n.startswith("fp6_linear_kernel<") and n.endswith(",%d,%d>" % (e3, rbw)) for n in plans), (e3, rbw)
    # the benchmark's own rows (M in 1, 16, 128 on the Llama-3-8B shapes)
    assert _lib.fp6_linear_plan(1, 4096, 14336) == "fp6_gemv_kernel<4,1,0>"
    assert _lib.fp6_linear_plan(16, 4096, 14336) == "fp6_linear_kernel<8,1,4>"
    assert _lib.fp6_linear_plan(128, 4096, 14336) == "fp6_gemm_kernel<1,1,4,4,4>"
    assert _lib.fp6_linear_plan(128, 14336, 4096) == "fp6_gemm_kernel<1,1,2,8,8>"
    assert _lib.fp6_linear_plan(128, 4096, 4096) == "fp6_gemm_kernel<1,1,2,8,8>"
    assert _lib.fp6_linear_plan(24, 4096, 14336) == "fp6_linear_mb_kernel<8,1,2>"
    assert len(plans) >= 34


def _cases():
    try:
        return sorted(_walk().items())
    except Exception:  # library not built: the CPU suite reports that elsewhere
        return []


@pytest.mark.gpu
@pytest.mark.parametrize("name,problem", _cases(), ids=[n for n, _ in _cases()])
def test_every_instantiation_is_correct(cabi, name, problem):
    from ao_amd import ops

    M, K, N, e, m, norm, dual = problem
    print(f"case fp6 dispatch {name}: M={M} K={K} N={N} e{e}m{m} norm={norm} dual={dual}", flush=True)
    assert cabi.fp6_linear_plan(M, K, N, e, m, norm=norm, dual=dual) == name
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(N + K + M + e)
    w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).half()
    tc, scale = ops.fp6_quantize_pack(w, e, m)
    native = ops.fp6_repack(tc, 1 + e + m)
    dq = ops.fp6_dequantize(tc, scale, e, m)            # fp32 values * fp16 scale
    w16 = dq.half().float()                             # the single fp16 rounding of the kernels
    x = torch.randn(M, K, device=dev, generator=gen).half()
    nw = (1.0 + 0.1 * torch.randn(K, device=dev, generator=gen)).half()

    def run(xx):
        if dual:
            return ops.fp6_swiglu(e, m, xx, native, scale, native_u, scale_u, nw, 1e-5)
        if norm:
            return ops.fp6_rmsnorm_linear(e, m, xx, nw, 1e-5, native, scale)
        return ops.fp6_linear_native(e, m, xx, native, scale)

    xn = ops.rmsnorm(x, nw, 1e-5) if norm else x
    if dual:
        wu = (torch.randn(N, K, device=dev, generator=gen) * 0.02).half()
        tcu, scale_u = ops.fp6_quantize_pack(wu, e, m)
        native_u = ops.fp6_repack(tcu, 1 + e + m)
        wu16 = ops.fp6_dequantize(tcu, scale_u, e, m).half().float()
        gate = (xn.float() @ w16.t()).half().float()
        up = (xn.float() @ wu16.t()).half().float()
        ref = torch.nn.functional.silu(gate).half().float() * up
    else:
        ref = xn.float() @ w16.t()
    y = run(x).float()
    torch.cuda.synchronize()
    err = float((y - ref).norm() / ref.norm())
    print(f"  rel_l2 = {err:.3e}", flush=True)
    assert bool(torch.isfinite(y).all()) and err <= (2e-3 if norm else 1e-3)
    if not norm:
        # the reference test's criterion on the same data
        mre = float(((y - ref).abs().mean() / ref.abs().mean()))
        assert mre < 1e-3
        # one-hot rows: columns of fp16(value * scale), bit for bit
        ks = torch.randint(0, K, (M,), device=dev, generator=gen)
        ks[0] = 0
        ks[-1] = K - 1
        xh = torch.zeros(M, K, dtype=torch.float16, device=dev)
        xh[torch.arange(M, device=dev), ks] = 1.0
        yh = run(xh)
        assert torch.equal(yh, dq.half().t()[ks])
