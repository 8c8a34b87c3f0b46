"""Seeded random shapes through the linear entry points, each compared with the matrix product of the library's own
dequantized weight, and the fused quantize + pack kernels compared bit for bit with the step-by-step primitives.

The kernel a call runs is chosen from (M, N, K, group) by a dispatch with a dozen branches per format; the hand-picked
shapes of the other tests reach every branch, these reach the combinations nobody thought of (a 128-row tile kernel
whose waves take different numbers of K steps was found wrong this way, at 213 x 6144 x 1920).  Every case prints its
shape first.
"""
import random

import pytest
import torch

pytestmark = pytest.mark.gpu


def _rel_l2(y, ref):
    return float((y.float() - ref.float()).norm() / ref.float().norm().clamp_min(1e-30))


def _rows(rng):
    r = rng.random()
    if r < 0.3:
        return rng.randint(1, 16)
    if r < 0.6:
        return rng.randint(17, 64)
    if r < 0.85:
        return rng.randint(65, 300)
    return rng.choice([384, 512, 777, 1024])


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_linear_entry_points_on_random_shapes(seed):
    from ao_amd import ops

    dev = torch.device("cuda:0")
    rng = random.Random(seed)
    torch.manual_seed(seed)
    for i in range(60):
        kind = rng.choice(["int4", "int4", "int4", "int8", "fp6"])
        M = _rows(rng)
        if kind == "int4":
            g = rng.choice([32, 64, 128, 256])
            N = rng.choice([rng.randint(1, 600), 16 * rng.randint(1, 400), 64 * rng.randint(1, 230),
                            rng.choice([4096, 6144, 14336, 12288, 1024])])
            K = g * rng.randint(1, max(1, 4096 // g)) if rng.random() < 0.7 else rng.choice([4096, 8192, 14336, 1024, 2048])
            if N * K > 14336 * 8192:
                N = 4096
            bias, resid = rng.random() < 0.4, rng.random() < 0.25
            f32 = rng.random() < 0.3 and not resid
            print(f"case random {seed}/{i} int4 M={M} N={N} K={K} g={g} bias={bias} residual={resid} fp32={f32}", flush=True)
            w = (torch.randn(N, K, device=dev) * 0.02).bfloat16()
            x = torch.randn(M, K, device=dev).bfloat16()
            packed, qparams = ops.int4wo_quantize_pack(w, g)
            dq = ops.int4wo_dequantize(packed, qparams, N, K, g)
            b = torch.randn(N, device=dev).bfloat16() if bias else None
            ref = x.float() @ dq.float().t()
            if bias:
                ref = ref + b.float()
            if resid:
                r = torch.randn(M, N, device=dev).bfloat16()
                y = ops.int4wo_linear_residual(x, packed, qparams, g, N, r, b)
                ref = ref.bfloat16().float() + r.float()
            else:
                y = ops.int4wo_linear(x, packed, qparams, g, N, b, f32)
            if not f32:
                ref = ref.bfloat16().float()   # the output's own rounding, as the kernel applies it to its fp32 sum
            tol = 2e-5 if f32 else 1e-3   # summation order only; with a bf16 output an element at a rounding boundary may flip
        elif kind == "int8":
            N = rng.choice([rng.randint(1, 600), 16 * rng.randint(1, 400), rng.choice([4096, 6144, 14336, 1024])])
            K = rng.choice([128 * rng.randint(1, 32), 128 * rng.randint(1, 112), 4096, 14336])
            if N * K > 14336 * 8192:
                N = 4096
            bias = rng.random() < 0.4
            print(f"case random {seed}/{i} int8 M={M} N={N} K={K} bias={bias}", flush=True)
            wq = torch.randint(-128, 128, (N, K), device=dev, dtype=torch.int8)
            s = (torch.rand(N, device=dev) * 0.01 + 0.001).bfloat16()
            x = torch.randn(M, K, device=dev).bfloat16()
            b = torch.randn(N, device=dev).bfloat16() if bias else None
            y = ops.int8wo_linear(x, wq, s, b)
            ref = (x.float() @ wq.float().t()).bfloat16().float() * s.float()
            if bias:
                ref = ref.bfloat16().float() + b.float()
            tol = 6e-3   # three bf16 roundings
        else:
            eb, mb = rng.choice([(3, 2), (2, 3), (2, 2)])
            N = 64 * rng.randint(1, 230) if rng.random() < 0.7 else rng.choice([4096, 14336, 6144, 1024])
            K = 64 * rng.randint(1, 128) if rng.random() < 0.7 else rng.choice([4096, 14336, 8192])
            if N * K > 14336 * 8192:
                N = 4096
            print(f"case random {seed}/{i} fp e{eb}m{mb} M={M} N={N} K={K}", flush=True)
            w = (torch.randn(N, K, device=dev) * 0.02).half()
            x = torch.randn(M, K, device=dev).half()
            data, s = ops.fp6_quantize_pack(w, eb, mb)
            dq = ops.fp6_dequantize(data, s, eb, mb)
            y = ops.quant_llm_linear(eb, mb, x, data, s, 1)
            ref = x.float() @ dq.float().t()
            tol = 2e-3   # fp16 output rounding (2^-12) and the fp16 rounding of weight * scale
        err = _rel_l2(y, ref)
        assert bool(torch.isfinite(y.float()).all()) and err <= tol, (seed, i, kind, M, N, K, err)


@pytest.mark.parametrize("seed", [1, 2])
def test_fused_quantize_pack_kernels_on_random_shapes_bit_exact(seed):
    from ao_amd import ops
    from ao_amd.quantization.utils import get_groupwise_affine_qparams, groupwise_affine_quantize_tensor_from_qparams

    dev = torch.device("cuda:0")
    rng = random.Random(100 + seed)
    torch.manual_seed(100 + seed)

    def special_values(w):
        for v in (0.0, float("inf"), -float("inf"), float("nan"), 1e-30, -1e-30, 3e38, 65504.0, 6e-8):
            if rng.random() < 0.25:
                idx = torch.randint(0, w.numel(), (max(1, w.numel() // 5000),), device=dev)
                w.view(-1)[idx] = v
        return w

    for i in range(60):
        scale = rng.choice([0.02, 1.0, 100.0, 1e-3])
        if rng.random() < 0.5:
            g = rng.choice([32, 64, 128, 256])
            N = rng.choice([rng.randint(1, 700), 16 * rng.randint(1, 300), rng.choice([4096, 1024])])
            K = g * rng.randint(1, max(1, 6144 // g))
            print(f"case random pack {seed}/{i} int4 N={N} K={K} g={g} scale={scale}", flush=True)
            w = (torch.randn(N, K, device=dev) * scale).bfloat16()
            if rng.random() < 0.3:
                w[:, :g] = 0   # constant groups
            if rng.random() < 0.3:
                w = special_values(w)
            packed, qparams = ops.int4wo_quantize_pack(w, g)
            s, z = get_groupwise_affine_qparams(w, 4, g, torch.bfloat16)
            codes = groupwise_affine_quantize_tensor_from_qparams(w, s, z, 4, g)
            packed2, qparams2 = ops.int4wo_pack(codes, s, z, g)
            assert torch.equal(packed, packed2) and torch.equal(qparams, qparams2), (seed, i, N, K, g)
        else:
            eb, mb = rng.choice([(3, 2), (2, 3), (2, 2)])
            N = 64 * rng.randint(1, 40)
            K = 64 * rng.randint(1, 40) if rng.random() < 0.8 else rng.choice([4096, 1024, 2048])
            dt = rng.choice([torch.bfloat16, torch.float16])
            print(f"case random pack {seed}/{i} fp e{eb}m{mb} N={N} K={K} {dt} scale={scale}", flush=True)
            w = (torch.randn(N, K, device=dev) * scale).to(dt)
            if rng.random() < 0.3:
                w[rng.randrange(N)] = 0
            if rng.random() < 0.3:
                w = special_values(w)
            # 16-bit rows take the one-launch kernel with the hardware conversions, fp32 rows the three-launch path
            data, s = ops.fp6_quantize_pack(w, eb, mb)
            data2, s2 = ops.fp6_quantize_pack(w.float(), eb, mb)
            assert torch.equal(data, data2) and torch.equal(s.view(torch.int16), s2.view(torch.int16)), (seed, i, N, K)


@pytest.mark.parametrize("seed", [1, 2])
def test_module_api_on_random_layers(seed):
    """quantize_(nn.Linear, ...) on random layer shapes, activation dtypes and leading dimensions: the forward returns
    the activation's dtype and shape and agrees with F.linear on the layer's own dequantized weight.  in_features that
    are not a multiple of the group (int4: zero-extended to a whole group) or of 128 (int8: the reference's op
    sequence instead of the HIP kernel) and layers the FPx recipe leaves in floating point are part of the draw."""
    import torch.nn as nn
    import torch.nn.functional as F

    from ao_amd.dtypes import AffineQuantizedTensor
    from ao_amd.prototype.quant_llm import QuantLlmLinearWeight
    from ao_amd.quantization import fp6_llm_weight_only, int4_weight_only, int8_weight_only, quantize_

    dev = torch.device("cuda:0")
    rng = random.Random(200 + seed)
    torch.manual_seed(200 + seed)
    for i in range(60):
        kind = rng.choice(["int4", "int4", "int8", "fpx"])
        N = rng.choice([rng.randint(1, 300), 8 * rng.randint(1, 200), 256 * rng.randint(1, 16), rng.choice([4096, 1024, 11008])])
        K = rng.choice([rng.randint(8, 600), 32 * rng.randint(1, 64), 128 * rng.randint(1, 40), rng.choice([4096, 1024])])
        lead = rng.choice([(1,), (3,), (2, 5), (17,), (40,), (130,), (1, 1, 7)])
        g = rng.choice([32, 64, 128, 256])
        bias = rng.random() < 0.5
        if kind == "fpx":
            K = max(64, K // 64 * 64)
            wdt = torch.float16
            dt = rng.choice([torch.float16, torch.float16, torch.bfloat16, torch.float32])
        else:
            wdt = torch.bfloat16
            dt = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        print(f"case random api {seed}/{i} {kind} N={N} K={K} lead={lead} dtype={dt} bias={bias} g={g}", flush=True)
        lin = nn.Linear(K, N, bias=bias, device=dev, dtype=wdt)
        quantize_(lin, int4_weight_only(group_size=g) if kind == "int4" else int8_weight_only() if kind == "int8" else fp6_llm_weight_only())
        if not isinstance(lin.weight, (AffineQuantizedTensor, QuantLlmLinearWeight)):
            assert kind == "fpx" and (N % 256 or K % 64), (kind, N, K)   # the recipe's own shape rule
            continue
        x = torch.randn(*lead, K, device=dev, dtype=dt)
        with torch.no_grad():
            y = lin(x)
            ref = F.linear(x.float(), lin.weight.dequantize().float(), None if lin.bias is None else lin.bias.float())
        assert y.shape == ref.shape and y.dtype is dt, (kind, N, K, lead, dt)
        err = _rel_l2(y, ref)
        # the 16-bit roundings of the chains (product, scale, bias; fp16 products for FPx) against an fp32 reference
        assert bool(torch.isfinite(y.float()).all()) and err <= 8e-3, (seed, i, kind, N, K, lead, dt, err)


@pytest.mark.parametrize("seed", [11, 12])
def test_hqq_matrix_core_product_on_random_shapes(seed):
    """Both products of the HQQ mixed matmul (1-64 rows) over random shapes, dtypes, signedness and group sizes against
    the float64 product with the dequantized weight, rounded to the output dtype (1.5e-3: one rounding of the result)."""
    from ao_amd import ops
    from ao_amd.prototype.hqq import pack_2xint4

    dev = torch.device("cuda:0")
    rng = random.Random(seed)
    torch.manual_seed(seed)
    for i in range(24):
        transposed = rng.random() < 0.5
        dtype = rng.choice([torch.bfloat16, torch.float16])
        signed = rng.random() < 0.5
        M = rng.randint(1, 64)
        if transposed:
            N, g = 16 * rng.randint(1, 80), 2 * rng.choice([1, 4, 16, 32, 64])
        else:
            N, g = 4 * rng.randint(1, 300), 8 * rng.choice([1, 2, 4, 8, 16])
        K = g * rng.randint(1, 40)
        print(f"case {i} hqq transposed={transposed} {dtype} signed={signed} M={M} N={N} K={K} g={g}", flush=True)
        lo, hi = (-8, 8) if signed else (0, 16)
        W_q = torch.randint(lo, hi, (K, N)).to(torch.int8 if signed else torch.uint8)
        s = (torch.rand(K // g, N) * 0.02 + 1e-3).to(dtype).to(dev)
        z = (torch.rand(K // g, N) * 6 + (-3 if signed else 5)).to(dtype).to(dev)
        packed = pack_2xint4(W_q).to(dev)
        # (q - zero) * scale, each op rounded to the storage dtype (the reference kernel's formula)
        w = ((W_q.to(dev).to(dtype).reshape(K // g, g, N) - z[:, None, :]) * s[:, None, :]).reshape(K, N)
        x = torch.randn(M, N if transposed else K, dtype=dtype, device=dev)
        y = ops.hqq_mixed_mm_mfma(x, packed, s, z, g, transposed)
        ref = (x.double() @ (w.double().t() if transposed else w.double())).to(dtype)
        err = _rel_l2(y, ref)
        assert err <= 1.5e-3, err


@pytest.mark.parametrize("seed", [21, 22])
def test_workspace_linears_on_random_shapes(seed):
    """The operators at 16-256 rows on narrow weights, where they may split K over workgroups through a workspace
    (int4 and the Quant-LLM formats), against the product with the dequantized weight."""
    from ao_amd import _lib, ops

    L = _lib.lib()
    dev = torch.device("cuda:0")
    rng = random.Random(seed)
    torch.manual_seed(seed)
    for i in range(16):
        M = rng.randint(16, 256)
        K = 256 * rng.randint(4, 60)
        if rng.random() < 0.5:
            g = rng.choice([32, 64, 128, 256])
            N = rng.choice([1000, 1024, 2048, 4096, 4100, 6144])
            print(f"case {i} int4 M={M} N={N} K={K} g={g} parts={L.ao_amd_int4wo_linear_ws_parts(M, K, N, g)}", flush=True)
            w = (torch.randn(N, K) * 0.02).bfloat16().to(dev)
            packed, qp = ops.int4wo_quantize_pack(w, g)
            dq = ops.int4wo_dequantize(packed, qp, N, K, g)
            x = torch.randn(M, K).bfloat16().to(dev)
            y = ops.int4wo_linear(x, packed, qp, g, N)
            ref = (x.float() @ dq.float().t()).bfloat16()
        else:
            e, m = rng.choice([(3, 2), (2, 3), (2, 2), (3, 1)])
            N = 64 * rng.randint(4, 100)
            print(f"case {i} fp{1 + e + m} e{e}m{m} M={M} N={N} K={K} parts={L.ao_amd_fp6_linear_ws_parts(M, K, N)}", flush=True)
            w = (torch.randn(N, K) * 0.05).half().to(dev)
            tc, scale = ops.fp6_quantize_pack(w, e, m)
            native = ops.fp6_repack(tc, 1 + e + m)
            wd = ops.fp6_dequantize(tc, scale, e, m).half()
            x = torch.randn(M, K).half().to(dev)
            y = ops.fp6_linear_native(e, m, x, native, scale)
            ref = (x.float() @ wd.float().t()).half()
        err = _rel_l2(y, ref)
        assert err <= 1e-3, err
