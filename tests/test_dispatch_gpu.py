"""Every kernel instantiation the int4 linear dispatch can select is reached by a GPU test.

`ao_amd_int4wo_linear_plan` answers, on the host, which instantiation a problem runs.  The CPU test walks a grid of
problems and pins the set of instantiations that exist; the GPU test takes, for every one of them, the smallest problem
of the grid that reaches it and checks the result: rows of one-hot activations must return single dequantized weights
bit for bit (the in-register dequantization of that kernel), random activations must agree with an fp32 matmul on the
bit-exact dequantized weight to 2e-5 relative L2 with fp32 output (accumulation order is the only difference) and to
1e-3 with bf16 output.  A new instantiation therefore cannot ship without a shape that exercises it: it appears in the
walk, and with it in the GPU parametrisation.
"""
import functools
import itertools

import numpy as np
import pytest
import torch

SHAPES = [(48, 192), (64, 512), (256, 1024), (512, 2048), (1024, 4096), (4096, 4096), (3072, 8192), (14336, 4096),
          (4096, 14336), (1024, 16384), (128256, 4096), (28672, 4096), (8192, 16384), (16384, 16384), (4096, 16384),
          (16384, 4096), (36864, 4096)]   # (N, K)
MS = [1, 2, 4, 16, 17, 32, 33, 64, 65, 128, 256, 512, 1024]
GROUPS = [32, 64, 128, 256]


@functools.lru_cache(maxsize=None)
def _walk():
    """plan name -> smallest problem (M, K, N, g, norm) of the grid that reaches it"""
    from ao_amd import _lib

    best = {}
    for (N, K), M, g, norm in itertools.product(SHAPES, MS, GROUPS, (False, True)):
        if norm and (M > 16 or K % max(128, g) or K > 16384):
            continue
        if N * M > (1 << 26):
            continue
        try:
            name = _lib.int4wo_linear_plan(M, K, N, g, aligned=K % max(128, g) == 0, norm=norm)
        except _lib.AoAmdError:
            continue   # combinations the entry point rejects (e.g. the fused norm on a shape that does not fit LDS)
        cost = N * K * (1 + M // 64)
        if name not in best or cost < best[name][0]:
            best[name] = (cost, (M, K, N, g, norm))
    return {k: v[1] for k, v in best.items()}


def test_dispatch_walk_finds_every_kernel_family():
    plans = _walk()
    families = {n.split("<")[0] for n in plans}
    assert families == {"int4wo_gemv1_kernel", "int4wo_gemv2_kernel", "int4wo_gemv_kernel", "int4wo_linear_kernel", "int4wo_gemm_kernel",
                        "int4wo_gemm_ksplit_kernel", "int4wo_gemm_lds_kernel", "int4wo_gemm_kwave_kernel",
                        "int4wo_linear_rb4_kernel"}
    # the tile variants of the matrix-core kernels and both K-split forms
    for g in GROUPS:
        for tile in ("int4wo_gemm_kernel<%d,2,8>", "int4wo_gemm_kernel<%d,1,4>", "int4wo_gemm_kernel<%d,1,2>",
                     "int4wo_gemm_ksplit_kernel<%d,4,4>", "int4wo_gemm_ksplit_kernel<%d,2,4>",
                     "int4wo_gemm_lds_kernel<%d,1>", "int4wo_gemm_lds_kernel<%d,2>", "int4wo_gemm_kwave_kernel<%d>",
                     "int4wo_linear_rb4_kernel<%d,4>", "int4wo_linear_rb4_kernel<%d,8>", "int4wo_linear_rb4_kernel<%d,4,2>",
                     "int4wo_linear_rb4_kernel<%d,8,2>", "int4wo_linear_rb4_kernel<%d,4,4>", "int4wo_linear_rb4_kernel<%d,8,4>"):
            assert tile % g in plans, tile % g
    # the single-row kernel: exactly the instantiations that int4wo_gemv1.hip compiles (waves, chunks per lane, norm)
    gemv1 = {n.split(" ")[0] for n in plans if n.startswith("int4wo_gemv1_kernel<")}
    want = {"int4wo_gemv1_kernel<%d,2,%d>" % (w, nm) for w in (4, 8, 16) for nm in (0, 1)}
    want |= {"int4wo_gemv1_kernel<4,4,0>", "int4wo_gemv1_kernel<4,4,1>", "int4wo_gemv1_kernel<8,4,0>", "int4wo_gemv1_kernel<4,8,0>"}
    assert gemv1 == want, sorted(gemv1 ^ want)
    # the single-row kernel with one workgroup per CU: exactly the instantiations that int4wo_gemv2.hip compiles (activation
    # chunks per thread, qparam chunks per lane); it takes fused-norm launches whose row blocks spread evenly over the CUs
    gemv2 = {n.split(" ")[0] for n in plans if n.startswith("int4wo_gemv2_kernel<")}
    assert gemv2 == {"int4wo_gemv2_kernel<%d,%d>" % (xc, ql) for xc in (1, 2) for ql in (1, 2, 4)}, sorted(gemv2)
    from ao_amd import _lib

    assert _lib.int4wo_linear_plan(1, 4096, 28672, 64, norm=True) == "int4wo_gemv2_kernel<1,2> upw=7 run=14"
    assert _lib.int4wo_linear_plan(1, 4096, 28672, 64).startswith("int4wo_gemv1_kernel")          # no norm
    assert _lib.int4wo_linear_plan(1, 4096, 14336, 64, norm=True).startswith("int4wo_gemv1_kernel")   # 224 workgroups
    assert _lib.int4wo_linear_plan(1, 4096, 128256, 64, norm=True).startswith("int4wo_gemv1_kernel")  # 32 units per workgroup
    # the prefill kernel takes a problem only when its 256-row tiles fill most of the chip

    assert _lib.int4wo_linear_plan(2048, 4096, 14336, 64).startswith("int4wo_gemm_lds_kernel<64,2>")
    assert _lib.int4wo_linear_plan(512, 4096, 14336, 64).startswith("int4wo_gemm_lds_kernel<64,1>")
    assert _lib.int4wo_linear_plan(2048, 14336, 4096, 64).startswith("int4wo_gemm_lds_kernel<64,1>")
    assert not _lib.int4wo_linear_plan(512, 14336, 4096, 64).startswith("int4wo_gemm_lds_kernel")   # 64 tiles
    assert _lib.int4wo_linear_plan(300, 4096, 14336, 64).startswith("int4wo_gemm_lds_kernel<64,1>")
    assert not _lib.int4wo_linear_plan(128, 4096, 28672, 64).startswith("int4wo_gemm_lds_kernel")   # half of the tile rows empty
    # 256 x 128 tiles where 256 x 256 ones would not fill the chip (168) or would need more time for their rounds
    assert _lib.int4wo_linear_plan(768, 4096, 14336, 64).startswith("int4wo_gemm_lds_kernel<64,1>")
    assert _lib.int4wo_linear_plan(2048, 4096, 28672, 64).startswith("int4wo_gemm_lds_kernel<64,1>")
    # ... and the 128-row tiles with K split over the waves where those do not, from 65 rows, when at least 192
    # of them exist
    assert _lib.int4wo_linear_plan(128, 4096, 14336, 64) == "int4wo_gemm_kwave_kernel<64>"
    assert _lib.int4wo_linear_plan(512, 14336, 4096, 64) == "int4wo_gemm_kwave_kernel<64>"
    assert not _lib.int4wo_linear_plan(128, 4096, 4096, 64).startswith("int4wo_gemm_kwave_kernel")   # 64 tiles
    assert _lib.int4wo_linear_plan(65, 1024, 14336, 64) == "int4wo_gemm_kwave_kernel<64>"
    assert not _lib.int4wo_linear_plan(64, 1024, 14336, 64).startswith("int4wo_gemm_kwave_kernel")
    # 4 to 16 rows on weights with 768 or more 16-row blocks: four row blocks per workgroup share the activation loads
    assert _lib.int4wo_linear_plan(16, 4096, 14336, 64) == "int4wo_linear_rb4_kernel<64,8>"
    assert _lib.int4wo_linear_plan(4, 4096, 128256, 64) == "int4wo_linear_rb4_kernel<64,4>"
    assert not _lib.int4wo_linear_plan(16, 14336, 4096, 64).startswith("int4wo_linear_rb4_kernel")   # 64 workgroups
    assert not _lib.int4wo_linear_plan(3, 4096, 14336, 64).startswith("int4wo_linear_rb4_kernel")
    # ... and 17 to 32 rows there take it with two activation blocks per workgroup instead of the 64-row tiles
    assert _lib.int4wo_linear_plan(24, 4096, 14336, 64) == "int4wo_linear_rb4_kernel<64,8,2>"
    # ... 33 to 48 rows (64 on the widest weights) with four
    assert _lib.int4wo_linear_plan(40, 4096, 14336, 64) == "int4wo_linear_rb4_kernel<64,8,4>"
    assert _lib.int4wo_linear_plan(64, 4096, 128256, 64) == "int4wo_linear_rb4_kernel<64,4,4>"
    assert not _lib.int4wo_linear_plan(49, 4096, 14336, 64).startswith("int4wo_linear_rb4_kernel")
    assert len(plans) >= 88


def _cases():
    try:
        return sorted(_walk().items())
    except Exception:  # library not built: the CPU suite reports that elsewhere
        return []


@pytest.mark.gpu
@pytest.mark.parametrize("name,problem", _cases(), ids=[n.replace(" ", "_") for n, _ in _cases()])
def test_every_instantiation_is_correct(cabi, name, problem):
    M, K, N, g, norm = problem
    print(f"case dispatch {name}: M={M} K={K} N={N} g={g} norm={norm}", flush=True)
    dev = torch.device("cuda:0")
    L = cabi.lib()
    st = torch.cuda.current_stream().cuda_stream
    assert cabi.int4wo_linear_plan(M, K, N, g, aligned=K % max(128, g) == 0, norm=norm) == name
    gen = torch.Generator(device=dev).manual_seed(N + K + M + g)
    w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).bfloat16()
    _, _, pb, qb = cabi.packed_shape(N, K, g)
    packed = torch.empty(pb // 4, dtype=torch.int32, device=dev)
    qp = torch.empty(qb // 4, dtype=torch.int32, device=dev)
    cabi.check(L.ao_amd_int4wo_quantize_pack(w.data_ptr(), N, K, K, g, packed.data_ptr(), qp.data_ptr(), st))
    dq = torch.empty(N, K, dtype=torch.bfloat16, device=dev)
    cabi.check(L.ao_amd_int4wo_dequantize(packed.data_ptr(), qp.data_ptr(), N, K, g, dq.data_ptr(), st))

    def run(x, fp32):
        y = torch.empty(x.shape[0], N, dtype=torch.float32 if fp32 else torch.bfloat16, device=dev)
        dt = cabi.F32 if fp32 else cabi.BF16
        if norm:
            cabi.check(L.ao_amd_int4wo_rmsnorm_linear(x.data_ptr(), x.shape[0], K, K, nw.data_ptr(), 1e-5, packed.data_ptr(),
                                                      qp.data_ptr(), N, g, None, y.data_ptr(), dt, N, st))
        else:
            cabi.check(L.ao_amd_int4wo_linear(x.data_ptr(), x.shape[0], K, K, packed.data_ptr(), qp.data_ptr(), N, g, None,
                                              y.data_ptr(), dt, N, st))
        torch.cuda.synchronize()
        return y

    nw = (1.0 + 0.1 * torch.randn(K, device=dev, generator=gen)).bfloat16()
    x = torch.randn(M, K, device=dev, generator=gen).bfloat16()
    if norm:
        # RMSNorm as the module computes it (torchao/_models/llama/model.py:232-244): bf16(bf16(x * rsqrt(mean x^2 + eps)) * w)
        xf = x.float()
        xn = ((xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).bfloat16().float() * nw.float()).bfloat16()
    else:
        xn = x
    y_ref = xn.float() @ dq.float().t()
    y32 = run(x, True)
    err = float((y32 - y_ref).norm() / y_ref.norm())
    print(f"  rel_l2 fp32-out = {err:.3e}", flush=True)
    # with the fused norm a 1-ulp difference of the row statistic can move single activations by one bf16 step
    assert err <= (1e-3 if norm else 2e-5)
    y16 = run(x, False)
    err16 = float((y16.float() - y_ref.bfloat16().float()).norm() / y_ref.norm())
    assert err16 <= 1e-3
    if not norm:
        # one-hot rows: the kernel's dequantization, bit for bit
        ks = torch.randint(0, K, (M,), device=dev, generator=gen)
        ks[0] = 0
        ks[-1] = K - 1
        xh = torch.zeros(M, K, dtype=torch.bfloat16, device=dev)
        xh[torch.arange(M, device=dev), ks] = 1.0
        yh = run(xh, True)
        exact = bool(torch.equal(yh, dq.float().t()[ks]))
        assert exact
