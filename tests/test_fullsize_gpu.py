"""GPU tests at the full Llama-3-8B sizes, where the scalar CPU oracle would take minutes: size-independent
properties of the path instead of element-by-element comparison with the oracle.

  * codes stay in [0, 15]; pack / unpack round-trip bit for bit
  * quantize_affine(dequantized weight, same scale / zero) returns the same codes (the idempotence the reference
    checks with `check_idempotent`, test/quantization/test_quant_primitives.py:42-47)
  * the linear with a one-hot activation row returns a column of the dequantized weight, bit for bit
  * linearity of the fp32-output linear: y(x1) + y(x2) vs y(x1 + x2) with exactly representable sums
  * the M = 1 kernel, the M <= 16 kernel and the M > 16 kernel agree on the same activation row
  * FP6: quantize(dequantize(codes)) returns the same bytes; one-hot rows of the linear return weight columns
"""
import numpy as np
import pytest
import torch

from _util import rel_l2

pytestmark = pytest.mark.gpu

SHAPES = [(14336, 4096), (4096, 14336), (128256, 4096)]   # (N, K) of w1/w3, w2 and the vocabulary head


def _dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def _weight(N, K, seed):
    g = torch.Generator(device=_dev()).manual_seed(seed)
    return (torch.randn(N, K, device=_dev(), generator=g) * 0.02).bfloat16()


@pytest.mark.parametrize("g", [64, 128])
@pytest.mark.parametrize("shape", SHAPES)
def test_int4_quantize_properties(shape, g):
    from ao_amd import ops

    N, K = shape
    print(f"case int4 full-size N={N} K={K} g={g}", flush=True)
    w = _weight(N, K, seed=N + g)
    packed, qp = ops.int4wo_quantize_pack(w, g)
    codes, scale, zero = ops.int4wo_unpack(packed, qp, N, K, g)
    assert codes.shape == (N, K) and scale.shape == (N, K // g)
    assert int(codes.min()) >= 0 and int(codes.max()) <= 15
    # every group reaches both ends of the range on random data (group min -> 0, group max -> 15)
    cg = codes.view(N, K // g, g)
    assert bool((cg.amin(dim=2) == 0).all()) and bool((cg.amax(dim=2) == 15).all())
    # pack(unpack(.)) reproduces the packed words
    packed2, qp2 = ops.int4wo_pack(codes, scale, zero, g)
    assert torch.equal(packed2, packed) and torch.equal(qp2, qp)
    del packed2, qp2, cg
    # reconstruction error within half a step (+ bf16 rounding of the result)
    dq = ops.int4wo_dequantize(packed, qp, N, K, g)
    step = scale.float().repeat_interleave(g, dim=1)
    err = (dq.float() - w.float()).abs()
    assert bool((err <= 0.75 * step + w.float().abs() * 2.0 ** -6 + 1e-6).all())
    del err, step
    # dequantized values quantize back to their own codes under the same (scale, zero), and the generic
    # dequantize_affine primitive agrees with the fused kernel
    from ao_amd.quantization.quant_primitives import ZeroPointDomain, dequantize_affine, quantize_affine

    codes2 = quantize_affine(dq, (1, g), scale, zero, torch.int32, 0, 15, ZeroPointDomain.FLOAT)
    assert torch.equal(codes2, codes)
    del codes2
    dq2 = dequantize_affine(codes, (1, g), scale, zero, torch.int32, 0, 15, ZeroPointDomain.FLOAT,
                            output_dtype=torch.bfloat16)
    assert torch.equal(dq2, dq)


@pytest.mark.parametrize("shape", SHAPES)
def test_int4_linear_properties(shape):
    from ao_amd import ops

    N, K = shape
    g = 64
    print(f"case int4 linear full-size N={N} K={K}", flush=True)
    dev = _dev()
    w = _weight(N, K, seed=7 + N)
    packed, qp = ops.int4wo_quantize_pack(w, g)
    dq = ops.int4wo_dequantize(packed, qp, N, K, g)
    del w
    # one-hot rows: M = 1 (GEMV), M = 5 (GEMV, several rows), M = 20 (GEMM kernel)
    ks = [0, 1, 63, 64, 127, 128, K // 2 + 3, K - 129, K - 2, K - 1, 1000, 2049, 77, 4000, 31, 32, 33, 500, 900, 1300]
    for M in (1, 5, 20):
        x = torch.zeros(M, K, dtype=torch.bfloat16, device=dev)
        for m in range(M):
            x[m, ks[m]] = 1.0
        y = ops.int4wo_linear(x, packed, qp, g, N, None, True)
        for m in range(M):
            assert torch.equal(y[m], dq[:, ks[m]].float()), (M, m, ks[m])
    # linearity on values whose sums and products are exact in the kernel's arithmetic: small integers
    gen = torch.Generator(device=dev).manual_seed(11)
    x1 = torch.randint(-4, 5, (1, K), device=dev, generator=gen).bfloat16()
    x2 = torch.randint(-4, 5, (1, K), device=dev, generator=gen).bfloat16()
    y1 = ops.int4wo_linear(x1, packed, qp, g, N, None, True)
    y2 = ops.int4wo_linear(x2, packed, qp, g, N, None, True)
    y12 = ops.int4wo_linear(x1 + x2, packed, qp, g, N, None, True)
    assert rel_l2((y1 + y2).cpu().numpy(), y12.cpu().numpy()) <= 1e-5
    # the three kernels on the same row: fp32 outputs agree to accumulation-order noise
    xr = torch.randn(1, K, device=dev, generator=gen).bfloat16()
    ya = ops.int4wo_linear(xr, packed, qp, g, N, None, True)
    yb = ops.int4wo_linear(xr.repeat(4, 1), packed, qp, g, N, None, True)
    yc = ops.int4wo_linear(xr.repeat(40, 1), packed, qp, g, N, None, True)
    assert rel_l2(yb[3:4].cpu().numpy(), ya.cpu().numpy()) <= 1e-5
    assert rel_l2(yc[39:40].cpu().numpy(), ya.cpu().numpy()) <= 1e-5
    # and against torch's fp32 matmul on the dequantized weight (tolerance of the path: 1e-3)
    ref = xr.float() @ dq.float().t()
    assert rel_l2(ya.cpu().numpy(), ref.cpu().numpy()) <= 1e-3


@pytest.mark.parametrize("shape", [(14336, 4096), (4096, 14336)])
def test_fp6_properties(shape):
    from ao_amd import ops

    N, K = shape
    print(f"case fp6 full-size N={N} K={K}", flush=True)
    dev = _dev()
    gen = torch.Generator(device=dev).manual_seed(N)
    w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).half()
    tc, scale = ops.fp6_quantize_pack(w, 3, 2)
    assert tc.shape == (N, K * 6 // 8) and scale.shape == (N,)
    # row scale = amax / 28 (largest e3m2 normal), computed in fp32 and rounded to fp16
    expect = (w.float().abs().amax(dim=1).clamp(min=1e-12) / 28.0).half()
    assert torch.equal(scale, expect)
    # codes -> values -> codes is the identity (unit scale: every e3m2 value is exactly representable)
    vals = ops.fp6_dequantize(tc, None, 3, 2)
    assert bool((vals.abs().amax(dim=1) == 28.0).all())   # the row maximum lands on the largest normal
    tc2, scale2 = ops.fp6_quantize_pack(vals, 3, 2)
    assert torch.equal(tc2, tc) and bool((scale2 == 1.0).all())
    # one-hot activation rows return columns of the scaled dequantized weight, rounded once to fp16
    dq = ops.fp6_dequantize(tc, scale, 3, 2)
    ks = [0, 1, 31, 32, 127, 128, K - 1, K // 2, 777, 4001, 15, 16, 17, 2048, 63, 64, 65, 300]
    for M in (1, 18):
        x = torch.zeros(M, K, dtype=torch.float16, device=dev)
        for m in range(M):
            x[m, ks[m]] = 1.0
        y = ops.quant_llm_linear(3, 2, x, tc, scale)
        for m in range(M):
            assert rel_l2(y[m].float().cpu().numpy(), dq[:, ks[m]].cpu().numpy()) <= 1e-3, (M, m)


@pytest.mark.parametrize("M", [16, 128])
@pytest.mark.parametrize("shape", [(4096, 4096), (14336, 4096), (4096, 14336)])
def test_fp6_linear_full_size(shape, M):
    """The FP6 configuration's many-row cases at the real Llama-3-8B shapes (the tile variants these shapes select are
    not the ones small shapes select): one-hot activation rows return columns of fp16(value * scale) bit for bit, random
    rows agree with an fp32 matmul on that weight to 1e-3 relative L2 and to the reference test's mean relative error
    (test/test_ops.py:47-62)."""
    from ao_amd import _lib, ops

    N, K = shape
    print(f"case fp6 linear full-size N={N} K={K} M={M}: {_lib.fp6_linear_plan(M, K, N)}", flush=True)
    dev = _dev()
    gen = torch.Generator(device=dev).manual_seed(N + M)
    w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).half()
    tc, scale = ops.fp6_quantize_pack(w, 3, 2)
    w16 = ops.fp6_dequantize(tc, scale, 3, 2).half()
    ks = torch.randint(0, K, (M,), device=dev, generator=gen)
    ks[0], ks[-1] = 0, K - 1
    xh = torch.zeros(M, K, dtype=torch.float16, device=dev)
    xh[torch.arange(M, device=dev), ks] = 1.0
    yh = ops.quant_llm_linear(3, 2, xh, tc, scale)
    assert torch.equal(yh, w16.t()[ks])
    x = torch.randn(M, K, device=dev, generator=gen).half()
    y = ops.quant_llm_linear(3, 2, x, tc, scale).float()
    ref = x.float() @ w16.float().t()
    assert rel_l2(y.cpu().numpy(), ref.cpu().numpy()) <= 1e-3
    assert float((y - ref).abs().mean() / ref.abs().mean()) < 1e-3


@pytest.mark.parametrize("M", [128, 512, 2048])
@pytest.mark.parametrize("shape", SHAPES)
def test_int4_prefill_gemm_full_size(shape, M):
    """The prefill configuration (M in {128, 512, 2048}, g = 64) at the real Llama-3-8B shapes, through the C ABI's
    fused kernel (whatever tile variant the dispatch picks there): one-hot rows bit for bit, random rows against an
    fp32 matmul on the bit-exact dequantized weight (2e-5 with fp32 output, 1e-3 with bf16 output)."""
    from ao_amd import _lib, ops

    N, K = shape
    g = 64
    if N * M > (1 << 28):
        pytest.skip("output larger than the launch allows")
    plan = _lib.int4wo_linear_plan(M, K, N, g)
    print(f"case int4 prefill full-size N={N} K={K} M={M}: {plan}", flush=True)
    assert plan.startswith("int4wo_gemm")
    dev = _dev()
    w = _weight(N, K, seed=3 + N + M)
    packed, qp = ops.int4wo_quantize_pack(w, g)
    dq = ops.int4wo_dequantize(packed, qp, N, K, g)
    del w
    L = _lib.lib()
    st = torch.cuda.current_stream().cuda_stream

    def run(x, fp32):
        y = torch.empty(M, N, dtype=torch.float32 if fp32 else torch.bfloat16, device=dev)
        _lib.check(L.ao_amd_int4wo_linear(x.data_ptr(), M, K, K, packed.data_ptr(), qp.data_ptr(), N, g, None, y.data_ptr(),
                                          _lib.F32 if fp32 else _lib.BF16, N, st))
        torch.cuda.synchronize()
        return y

    gen = torch.Generator(device=dev).manual_seed(M)
    ks = torch.randint(0, K, (M,), device=dev, generator=gen)
    ks[0], ks[1] = 0, K - 1
    xh = torch.zeros(M, K, dtype=torch.bfloat16, device=dev)
    xh[torch.arange(M, device=dev), ks] = 1.0
    yh = run(xh, True)
    exact = bool(torch.equal(yh, dq.float().t()[ks]))
    assert exact
    del yh, xh
    x = torch.randn(M, K, device=dev, generator=gen).bfloat16()
    ref = x.float() @ dq.float().t()
    y32 = run(x, True)
    assert float((y32 - ref).norm() / ref.norm()) <= 2e-5
    del y32
    y16 = run(x, False)
    assert float((y16.float() - ref.bfloat16().float()).norm() / ref.norm()) <= 1e-3


def test_config1_output_tolerance(oracle):
    """The CPU-runnable configuration: one bf16 weight [4096, 4096] ~N(0, 0.02), group 128, x [1, 4096] ~N(0, 1): the
    linear's output against the oracle's dequantize-then-linear with fp32 accumulation, rel-L2 <= 1e-3 (codes, scales
    and zeros of this configuration are compared bit for bit in test_int4wo_gpu.py)."""
    from _util import bits16, make_act, make_weight
    from ao_amd import ops

    N = K = 4096
    g = 128
    w = make_weight(N, K, seed=1234, special=False)
    x = make_act(1, K, seed=4321)
    codes, scale, zero = oracle.int4wo_quantize(bits16(w), oracle.BF16, g, N, K)
    dq = oracle.dequantize_affine(codes, oracle.I32, (1, g), scale, oracle.BF16, zero, oracle.BF16, 0, 15, 1, oracle.BF16)
    y_ref = oracle.linear(bits16(x), oracle.BF16, dq, oracle.BF16)
    packed, qp = ops.int4wo_quantize_pack(w.to(_dev()), g)
    y32 = ops.int4wo_linear(x.to(_dev()), packed, qp, g, N, None, True)
    err = rel_l2(y32.cpu().numpy(), y_ref)
    print(f"config 1 output rel-L2 = {err:.3e}", flush=True)
    assert err <= 1e-3
    y16 = ops.int4wo_linear(x.to(_dev()), packed, qp, g, N, None, False)
    y_ref16 = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(y_ref))
    assert rel_l2(y16.float().cpu().numpy(), y_ref16) <= 1e-3


@pytest.mark.parametrize("M,N,K,g,bias,fp32,kernel", [
    (2048, 14336, 4096, 64, False, False, "lds"), (1000, 14336, 4096, 128, True, False, "lds"),
    (2048, 6100, 1024, 64, True, False, "lds"), (1792, 4096, 2048, 32, False, True, "lds"),
    (2048, 4096, 14336, 256, True, False, "lds"),
    (128, 14336, 4096, 64, False, False, "kwave"), (200, 12352, 1024, 128, True, False, "kwave"),
    (512, 4096, 14336, 256, False, True, "kwave"), (333, 6100, 2048, 32, True, False, "kwave"),
    (1000, 4098, 4096, 64, True, True, "kwave"), (130, 14336, 1152, 64, False, False, "kwave"),
    (213, 6144, 1920, 128, True, False, "kwave")])
def test_prefill_gemm_tiles_edges_and_repeated_launches(cabi, M, N, K, g, bias, fp32, kernel):
    """The prefill kernels (activations through LDS-direct loads, weights dequantized between the matrix instructions;
    256-row tiles, and 128-row tiles whose waves split K, with step counts per wave that differ when K / 64 is not a
    multiple of 4): every output element is written (the output starts as NaN), ragged M and N, bias, both output
    types, and the same launch three times in a row with LDS of every CU overwritten in between by another kernel, so
    that a read that runs ahead of its data cannot find the previous launch's identical bytes there."""
    print(f"case prefill gemm M={M} N={N} K={K} g={g} bias={bias} fp32={fp32} {kernel}", flush=True)
    dev = torch.device("cuda:0")
    L = cabi.lib()
    st = torch.cuda.current_stream().cuda_stream
    assert cabi.int4wo_linear_plan(M, K, N, g).startswith(f"int4wo_gemm_{kernel}_kernel")
    gen = torch.Generator(device=dev).manual_seed(M + N + K)
    w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).bfloat16()
    _, _, pb, qb = cabi.packed_shape(N, K, g)
    packed = torch.empty(pb // 4, dtype=torch.int32, device=dev)
    qp = torch.empty(qb // 4, dtype=torch.int32, device=dev)
    cabi.check(L.ao_amd_int4wo_quantize_pack(w.data_ptr(), N, K, K, g, packed.data_ptr(), qp.data_ptr(), st))
    dq = torch.empty(N, K, dtype=torch.bfloat16, device=dev)
    cabi.check(L.ao_amd_int4wo_dequantize(packed.data_ptr(), qp.data_ptr(), N, K, g, dq.data_ptr(), st))
    del w
    b = (torch.randn(N, device=dev, generator=gen) * 0.1).bfloat16() if bias else None
    x = torch.randn(M, K, device=dev, generator=gen).bfloat16()
    ref = x.float() @ dq.float().t()
    if bias:
        ref += b.float()
    y = torch.empty(M, N, dtype=torch.float32 if fp32 else torch.bfloat16, device=dev)
    for rep in range(3):
        y.fill_(float("nan"))
        # a kernel that fills LDS with other data: the fp16 RMSNorm over many rows uses every CU
        junk = torch.randn(4096, 4096, device=dev).half()
        torch.nn.functional.layer_norm(junk, (4096,))
        cabi.check(L.ao_amd_int4wo_linear(x.data_ptr(), M, K, K, packed.data_ptr(), qp.data_ptr(), N, g,
                                          None if b is None else b.data_ptr(), y.data_ptr(), cabi.F32 if fp32 else cabi.BF16, N, st))
        torch.cuda.synchronize()
        finite = bool(torch.isfinite(y.float()).all())
        want = ref if fp32 else ref.bfloat16().float()
        err = float((y.float() - want).norm() / ref.norm())
        print(f"  launch {rep}: finite {finite} rel_l2 {err:.2e}", flush=True)
        assert finite and err <= (2e-5 if fp32 else 1e-3)
    # one-hot rows: the kernel's dequantization, bit for bit
    ks = torch.randint(0, K, (M,), device=dev, generator=gen)
    xh = torch.zeros(M, K, dtype=torch.bfloat16, device=dev)
    xh[torch.arange(M, device=dev), ks] = 1.0
    yh = torch.empty(M, N, dtype=torch.float32, device=dev)
    cabi.check(L.ao_amd_int4wo_linear(xh.data_ptr(), M, K, K, packed.data_ptr(), qp.data_ptr(), N, g, None, yh.data_ptr(),
                                      cabi.F32, N, st))
    torch.cuda.synchronize()
    exact = bool(torch.equal(yh, dq.float().t()[ks]))
    assert exact


@pytest.mark.parametrize("M,N,K,g", [(2048, 14336, 4096, 64), (512, 14336, 4096, 128), (512, 4096, 14336, 256),
                                     (128, 14336, 4096, 64), (213, 6144, 1920, 128), (150, 12288, 1152, 64)])
def test_prefill_gemm_launches_repeat_bit_for_bit(cabi, M, N, K, g):
    """The prefill kernels sum in a fixed order, so 40 launches on the same operands must give the same fp32 bits; a
    result read before its matrix instruction has finished (their latency is the kernels' own business: the
    instructions are asm statements) shows up as a launch that differs in a few elements.  K = 1920 and 1152 give the
    four waves of the 128-row kernel different step counts: the waves that leave the loop after an even-numbered step
    still have that step's look-ahead requests in flight, into registers the epilogue must not use before they landed
    (it did, for its store addresses: one wave's partial tile went to the wrong place in a few launches of a hundred)."""
    plan = cabi.int4wo_linear_plan(M, K, N, g)
    print(f"case prefill gemm repeat M={M} N={N} K={K} g={g}: {plan}", flush=True)
    assert plan.startswith(("int4wo_gemm_lds_kernel", "int4wo_gemm_kwave_kernel"))
    dev = torch.device("cuda:0")
    L = cabi.lib()
    st = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device=dev).manual_seed(M + N + K + g)
    w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).bfloat16()
    _, _, pb, qb = cabi.packed_shape(N, K, g)
    packed = torch.empty(pb // 4, dtype=torch.int32, device=dev)
    qp = torch.empty(qb // 4, dtype=torch.int32, device=dev)
    cabi.check(L.ao_amd_int4wo_quantize_pack(w.data_ptr(), N, K, K, g, packed.data_ptr(), qp.data_ptr(), st))
    del w
    x = torch.randn(M, K, device=dev, generator=gen).bfloat16()
    first = torch.empty(M, N, dtype=torch.float32, device=dev)
    y = torch.empty_like(first)
    differing = []
    for rep in range(40):
        out = first if rep == 0 else y
        out.fill_(float("nan"))
        cabi.check(L.ao_amd_int4wo_linear(x.data_ptr(), M, K, K, packed.data_ptr(), qp.data_ptr(), N, g, None, out.data_ptr(),
                                          cabi.F32, N, st))
        torch.cuda.synchronize()
        if rep and not torch.equal(y, first):
            differing.append((rep, int((y != first).sum())))
    finite = bool(torch.isfinite(first).all())
    assert finite and differing == []


@pytest.mark.parametrize("M,N,K,g,bias,residual,fp32", [(13, 14400, 1024, 128, True, False, False), (16, 14336, 4096, 64, False, True, False),
                                                        (4, 16384, 2048, 32, True, True, False), (9, 14336, 4096, 256, True, False, True),
                                                        (17, 14336, 4096, 64, True, False, False), (29, 14400, 1024, 128, True, True, False),
                                                        (32, 16384, 2048, 256, False, False, True), (11, 14330, 1024, 64, True, False, False),
                                                        (23, 12346, 1024, 64, False, True, False), (33, 14336, 4096, 64, True, False, False),
                                                        (48, 14400, 1024, 128, False, True, False), (41, 16384, 2048, 32, True, False, True),
                                                        (64, 65536, 512, 256, True, True, False)])
def test_four_row_blocks_per_workgroup_kernel_epilogues(cabi, M, N, K, g, bias, residual, fp32):
    """int4wo_linear_rb4_kernel (4 to 48 or 64 activation rows, four 16-row weight blocks per workgroup sharing the
    activation loads, two activation blocks from 17 rows, four from 33): bias, residual (y = bf16(bf16(acc + bias) + residual), the order of the unfused modules), fp32 output and
    ragged M, against an fp32 matmul on the bit-exact dequantized weight."""
    plan = cabi.int4wo_linear_plan(M, K, N, g, residual=residual)
    print(f"case rb4 M={M} N={N} K={K} g={g} bias={bias} residual={residual} fp32={fp32}: {plan}", flush=True)
    assert plan.startswith("int4wo_linear_rb4_kernel")
    dev = torch.device("cuda:0")
    L = cabi.lib()
    st = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device=dev).manual_seed(M + N + K)
    w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).bfloat16()
    _, _, pb, qb = cabi.packed_shape(N, K, g)
    packed = torch.empty(pb // 4, dtype=torch.int32, device=dev)
    qp = torch.empty(qb // 4, dtype=torch.int32, device=dev)
    cabi.check(L.ao_amd_int4wo_quantize_pack(w.data_ptr(), N, K, K, g, packed.data_ptr(), qp.data_ptr(), st))
    dq = torch.empty(N, K, dtype=torch.bfloat16, device=dev)
    cabi.check(L.ao_amd_int4wo_dequantize(packed.data_ptr(), qp.data_ptr(), N, K, g, dq.data_ptr(), st))
    b = (torch.randn(N, device=dev, generator=gen) * 0.1).bfloat16() if bias else None
    res = torch.randn(M, N, device=dev, generator=gen).bfloat16() if residual else None
    x = torch.randn(M, K, device=dev, generator=gen).bfloat16()
    ref = x.float() @ dq.float().t()
    if bias:
        ref = ref + b.float()
    y = torch.full((M, N), float("nan"), dtype=torch.float32 if fp32 else torch.bfloat16, device=dev)
    if residual:
        ref = ref.bfloat16().float() + res.float()
        cabi.check(L.ao_amd_int4wo_linear_residual(x.data_ptr(), M, K, K, packed.data_ptr(), qp.data_ptr(), N, g,
                                                   None if b is None else b.data_ptr(), res.data_ptr(), N, y.data_ptr(), N, st))
    else:
        cabi.check(L.ao_amd_int4wo_linear(x.data_ptr(), M, K, K, packed.data_ptr(), qp.data_ptr(), N, g,
                                          None if b is None else b.data_ptr(), y.data_ptr(), cabi.F32 if fp32 else cabi.BF16, N, st))
    torch.cuda.synchronize()
    finite = bool(torch.isfinite(y.float()).all())
    want = ref if fp32 else ref.bfloat16().float()
    err = float((y.float() - want).norm() / ref.norm())
    assert finite and err <= (2e-5 if fp32 else 1.5e-3)
