"""GPU consistency sweep over random shapes: every linear kernel (decode kernel, tiled kernels with both tile sizes,
general fallback; int4, FP6 / FP5, int8) against an fp32 matmul on the weight that the library's own dequantize kernels
return.  Those dequantize kernels are compared bit for bit with the CPU oracle in the parity tests, so this
sweep extends that parity to many shapes at the price of a GPU matmul: ragged N, K not a multiple of 128, M on
both sides of every dispatch boundary.  fp32 outputs, tolerance 2e-5 relative L2 (accumulation order only)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def _rel(a, b):
    return float((a.double() - b.double()).norm() / b.double().norm().clamp(min=1e-30))


def test_int4_linear_random_shapes():
    from ao_amd import ops

    dev = _dev()
    rng = np.random.default_rng(2024)
    gen = torch.Generator(device=dev).manual_seed(7)
    for case in range(40):
        g = int(rng.choice([32, 64, 128, 256]))
        N = int(rng.integers(1, 700))
        K = int(rng.integers(1, 12)) * 128 if case % 3 else int(rng.integers(1, 1500))
        M = int(rng.choice([1, 2, 3, 15, 16, 17, 33, 64, 65, 130, 300]))
        print(f"case int4 random N={N} K={K} M={M} g={g}", flush=True)
        Kq = -(-K // g) * g
        w = (torch.randn(N, Kq, device=dev, generator=gen) * 0.05).bfloat16()
        w[:, K:] = 0                              # the reference zero-pads K to a group multiple before quantizing
        x = torch.randn(M, K, device=dev, generator=gen).bfloat16()
        packed, qp = ops.int4wo_quantize_pack(w[:, :K].contiguous() if K % g == 0 else w, g)
        Kw = K if K % g == 0 else Kq
        dq = ops.int4wo_dequantize(packed, qp, N, Kw, g).float()[:, :K]
        xin = x if Kw == K else torch.nn.functional.pad(x, (0, Kw - K))
        y = ops.int4wo_linear(xin, packed, qp, g, N, None, True)
        assert _rel(y, x.float() @ dq.t()) <= 2e-5, (N, K, M, g)


def test_fp6_linear_random_shapes():
    from ao_amd import ops

    dev = _dev()
    rng = np.random.default_rng(99)
    gen = torch.Generator(device=dev).manual_seed(8)
    for case in range(24):
        ebits, mbits = [(3, 2), (2, 3), (2, 2), (3, 1)][case % 4]
        N = int(rng.integers(1, 12)) * 64
        K = int(rng.integers(1, 24)) * 64
        M = int(rng.choice([1, 3, 16, 17, 64, 65, 129, 300]))
        print(f"case fpx random e{ebits}m{mbits} N={N} K={K} M={M}", flush=True)
        w = (torch.randn(N, K, device=dev, generator=gen) * 0.05).half()
        x = (torch.rand(M, K, device=dev, generator=gen) - 0.5).half()
        data, scale = ops.fp6_quantize_pack(w, ebits, mbits)
        dq = ops.fp6_dequantize(data, scale, ebits, mbits).half().float()   # the kernel rounds code * scale to fp16
        y = ops.quant_llm_linear(ebits, mbits, x, data, scale)
        ref = (x.float() @ dq.t())
        assert _rel(y.float(), ref.half().float()) <= 1e-3, (N, K, M, ebits, mbits)


def test_int8_linear_random_shapes():
    from ao_amd import ops

    dev = _dev()
    rng = np.random.default_rng(5)
    gen = torch.Generator(device=dev).manual_seed(9)
    for case in range(24):
        N = int(rng.integers(1, 900))
        K = int(rng.integers(1, 20)) * 128
        M = int(rng.choice([1, 2, 16, 17, 40]))
        print(f"case int8 random N={N} K={K} M={M}", flush=True)
        q = torch.randint(-128, 128, (N, K), device=dev, dtype=torch.int8, generator=gen)
        s = (torch.rand(N, device=dev, generator=gen) * 1e-2 + 1e-3).bfloat16()
        x = torch.randn(M, K, device=dev, generator=gen).bfloat16()
        y = ops.int8wo_linear(x, q, s, None, True)                        # bf16(x @ q^T) * s, before the last rounding
        acc = x.float() @ q.float().t()
        ref = acc.bfloat16().float() * s.float()
        # an accumulator on a bf16 rounding boundary may land on the other side: allow a few one-ulp elements
        assert _rel(y, ref) <= 1e-3 and float(((y - ref).abs() > 1e-6 * ref.abs() + 1e-12).float().mean()) <= 0.02
