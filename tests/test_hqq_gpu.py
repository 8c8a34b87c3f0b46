"""GPU tests of the HQQ prototype path: the dequantize kernel bit-exact against the oracle, the mixed matmul (forward and
transposed) at the reference test's shapes against `x @ W_dq` / `x @ W_dq.T` (test/hqq/test_triton_mm.py:18-29, 118-139),
and the HQQ -> int4 weight-only converter module."""
import numpy as np
import pytest
import torch

from _util import bits16, rel_l2

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def _hqq_like(N, K, g, dtype, seed, signed=False):
    """Codes, scales and zeros shaped as HQQ leaves them with axis = 1 grouping of an [N, K] weight: W_q [N, K],
    scale / zero [N, K/g] (meta tensors reshaped as in the reference test)."""
    gen = torch.Generator().manual_seed(seed)
    lo, hi = (-8, 8) if signed else (0, 16)
    W_q = torch.randint(lo, hi, (N, K), generator=gen).to(torch.int8 if signed else torch.uint8)
    scale = (torch.rand(N, K // g, generator=gen) * 0.02 + 1e-3).to(dtype)
    zero = (torch.rand(N, K // g, generator=gen) * 6 + (-3 if signed else 5)).to(dtype)
    return W_q, scale, zero


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(128, 128, 64), (48, 256, 32), (4096, 4096, 128)])
def test_dequantize_bit_exact(oracle, shape, dtype, signed):
    from ao_amd import ops
    from ao_amd.prototype.hqq import pack_2xint4

    N, K, g = shape
    print(f"case hqq dequantize N={N} K={K} g={g} {dtype} signed={signed}", flush=True)
    dev = _dev()
    W_q, scale, zero = _hqq_like(N, K, g, dtype, seed=N + g, signed=signed)
    packed = pack_2xint4(W_q.T.contiguous())
    w = ops.hqq_dequantize(packed.to(dev), scale.T.contiguous().to(dev), zero.T.contiguous().to(dev), g)
    assert w.shape == (K, N) and w.dtype is dtype
    ref = oracle.hqq_dequantize(packed.numpy(), bits16(scale.T.contiguous()), bits16(zero.T.contiguous()), g,
                                oracle.BF16 if dtype is torch.bfloat16 else oracle.F16)
    assert np.array_equal(bits16(w), ref)


@pytest.mark.parametrize("transposed", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("group_size", [64, 128])
@pytest.mark.parametrize("shape", [(16, 128, 128), (16, 4096, 4096), (300, 512, 1024)])
def test_mixed_mm(oracle, shape, group_size, dtype, transposed):
    """Arguments passed as the reference test passes them: packed W_q.T, scales.T and zeros.T as (non-contiguous)
    transposed views of the [N, K/g] parameters."""
    from ao_amd.prototype.hqq import pack_2xint4, triton_mixed_mm

    M, N, K = shape
    print(f"case mixed_mm M={M} N={N} K={K} g={group_size} {dtype} transposed={transposed}", flush=True)
    dev = _dev()
    W_q, scale, zero = _hqq_like(N, K, group_size, dtype, seed=M + N + group_size)
    W_q, scale, zero = W_q.to(dev), scale.to(dev), zero.to(dev)
    # HQQ's dequantize: ((W_q - zero) * scale) on the grouped view, in the compute dtype
    W_dq = ((W_q.to(dtype).reshape(-1, group_size) - zero.reshape(-1, 1)) * scale.reshape(-1, 1)).reshape(N, K)
    packed_w = pack_2xint4(W_q.T)
    gen = torch.Generator(device=dev).manual_seed(7)
    if transposed:
        x = torch.randn(M, N, dtype=dtype, device=dev, generator=gen)
        expect = x @ W_dq
    else:
        x = torch.randn(M, K, dtype=dtype, device=dev, generator=gen)
        expect = x @ W_dq.T
    out = triton_mixed_mm(x, packed_w, scale.T, zero.T, transposed=transposed, group_size=group_size,
                          fp8_fast_accum=False, kernel_type="compute_bound")
    assert out.shape == expect.shape and out.dtype is dtype
    # The reference test asks for atol = rtol = 1e-3 between its kernel and torch's matmul.  Two GEMMs that sum in a
    # different order may round an element to neighbouring values of the output dtype, and one bf16 step is 2^-7
    # relative, so the bound here is one step of the dtype (plus the reference's atol), on few elements.
    step = 2.0 ** -7 if dtype is torch.bfloat16 else 2.0 ** -10
    assert torch.allclose(expect, out, atol=1e-3, rtol=step)
    assert (expect != out).float().mean().item() <= 0.05
    # and against fp32 accumulation on the CPU for the small cases
    if N * K <= 512 * 1024:
        ref = (x.double().cpu() @ (W_dq.double().cpu() if transposed else W_dq.double().cpu().T)).numpy()
        assert rel_l2(out.float().cpu().numpy(), ref) <= 4e-3  # one rounding of the result to bf16 / fp16


def test_mixed_mm_argument_checks():
    from ao_amd.prototype.hqq import mixed_mm, pack_2xint4

    dev = _dev()
    W_q, scale, zero = _hqq_like(64, 128, 64, torch.float16, seed=1)
    b = pack_2xint4(W_q.T.contiguous()).to(dev)
    s, z = scale.T.contiguous().to(dev), zero.T.contiguous().to(dev)
    x = torch.randn(4, 128, dtype=torch.float16, device=dev)
    with pytest.raises(AssertionError, match="incompatible dimensions"):
        mixed_mm(x[:, :64], b, s, z, 64)
    with pytest.raises(AssertionError, match="transpose requires"):
        mixed_mm(x, b, s, z, 64, transposed=True)
    with pytest.raises(AssertionError):
        mixed_mm(x.bfloat16(), b, s, z, 64)
    with pytest.raises(AssertionError, match="int8 or uint8"):
        mixed_mm(x, b.to(torch.int32), s, z, 64)


@pytest.mark.parametrize("g", [64, 128])
def test_converter_module_runs_hqq_weights_on_the_int4_kernels(oracle, g):
    from ao_amd import ops
    from ao_amd.prototype.hqq import HQQLinearTorchWeightOnlyInt4

    dev = _dev()
    N, K = 256, 1024
    W_q, scale, zero = _hqq_like(N, K, g, torch.bfloat16, seed=3 + g)
    meta = {"scale": scale.reshape(-1, 1).to(dev), "zero": zero.reshape(-1, 1).to(dev), "shape": (N, K),
            "packing": None, "nbits": 4, "group_size": g, "axis": 1}
    cfg = {"weight_quant_params": {"nbits": 4, "group_size": g, "axis": 1}}
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(1)) * 0.1).bfloat16().to(dev)
    mod = HQQLinearTorchWeightOnlyInt4(None, cfg, initialize=False).initialize_with_hqq_quants(
        W_q.reshape(-1, g).to(dev).float(), meta, bias=bias)
    assert mod.ready and mod.in_features == K and mod.out_features == N and not mod.padding
    assert mod.scales_and_zeros.shape == (K // g, N, 2) and mod.scales_and_zeros.dtype is torch.bfloat16
    codes, s, z_aff = ops.int4wo_unpack(mod.weight_int4pack, mod._qparams, N, K, g)
    assert torch.equal(codes.cpu(), W_q.to(torch.int32))           # the conversion keeps the codes
    assert torch.equal(s.cpu(), scale)                              # and the scales
    assert torch.equal(mod.scales_and_zeros[:, :, 0].t().cpu(), scale)
    assert torch.equal(mod.scales_and_zeros[:, :, 1].t().cpu(), z_aff.cpu())
    # forward = linear over the affine reconstruction (the int4 kernels' own oracle) ...
    x = torch.randn(2, 5, K, generator=torch.Generator().manual_seed(2)).bfloat16()
    y = mod(x.to(dev))
    assert y.shape == (2, 5, N) and y.dtype is torch.bfloat16
    dq = oracle.dequantize_affine(codes.cpu().numpy(), oracle.I32, (1, g), bits16(s), oracle.BF16, bits16(z_aff),
                                  oracle.BF16, 0, 15, 1, oracle.BF16)
    assert np.array_equal(bits16(mod.dequantize()), dq)
    y_ref = oracle.linear(bits16(x.reshape(-1, K)), oracle.BF16, dq, oracle.BF16)
    y_ref = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(y_ref)) + bias.float().cpu().numpy()
    assert rel_l2(y.float().cpu().numpy().reshape(-1, N), y_ref) <= 4e-3
    # ... which is HQQ's own reconstruction up to the bf16 rounding of the converted zero point
    hqq_w = ((W_q.double().reshape(-1, g) - zero.double().reshape(-1, 1)) * scale.double().reshape(-1, 1)).reshape(N, K)
    y_hqq = x.double().reshape(-1, K) @ hqq_w.T + bias.double().cpu()
    assert rel_l2(y.float().cpu().numpy().reshape(-1, N), y_hqq.numpy()) <= 2e-2

    with pytest.raises(ImportError, match="hqq"):
        HQQLinearTorchWeightOnlyInt4(torch.nn.Linear(K, N, bias=False), cfg, initialize=True)


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,g", [(1, 4096, 4096, 64), (3, 1000, 512, 128), (8, 11008, 4096, 64), (16, 256, 2048, 32), (5, 64, 128, 128)])
def test_fused_small_m_product_matches_the_dequantized_matmul(oracle, M, N, K, g, dtype, signed):
    """The fused forward kernel (1-16 rows): within 1e-3 relative L2 of the fp32-accumulated product with the oracle's
    dequantized weight (rounded to the output dtype), and exactly the dequantized weight on one-hot rows: the kernel
    rounds every weight as ao_amd_hqq_dequantize does.  N = 1000 and 64 leave lanes and whole waves without columns."""
    from ao_amd import ops
    from ao_amd.prototype.hqq import mixed_mm, pack_2xint4

    print(f"case hqq fused M={M} N={N} K={K} g={g} {dtype} signed={signed}", flush=True)
    dev = _dev()
    W_q, scale, zero = _hqq_like(N, K, g, dtype, seed=M + N + g, signed=signed)
    packed = pack_2xint4(W_q.T.contiguous()).to(dev)
    s, z = scale.T.contiguous().to(dev), zero.T.contiguous().to(dev)
    code = oracle.BF16 if dtype is torch.bfloat16 else oracle.F16
    w_ref = oracle.hqq_dequantize(packed.cpu().numpy(), bits16(s.cpu()), bits16(z.cpu()), g, code)   # [K, N] bits
    w_f32 = (oracle.bf16_bits_to_f32(w_ref) if dtype is torch.bfloat16 else w_ref.view(np.float16).astype(np.float32))
    x = torch.randn(M, K, dtype=dtype, generator=torch.Generator().manual_seed(3)).to(dev)
    y = ops.hqq_mixed_mm_small(x, packed, s, z, g)
    assert y.shape == (M, N) and y.dtype is dtype
    ref = x.float().cpu().numpy().astype(np.float64) @ w_f32.astype(np.float64)
    ref_r = torch.from_numpy(ref).to(dtype).float().numpy()
    err = rel_l2(y.float().cpu().numpy(), ref_r)
    assert err <= 1e-3, err
    # the module-level entry point takes the matrix-core kernel for these shapes
    if N % 16 == 0 or K % 8 == 0:
        err2 = rel_l2(mixed_mm(x, packed, s, z, g).float().cpu().numpy(), ref_r)
        assert err2 <= 1e-3, err2
    # one-hot rows read single weights back, bit for bit
    ks = torch.randint(0, K, (M,), generator=torch.Generator().manual_seed(4))
    ks[0], ks[-1] = 0, K - 1
    xh = torch.zeros(M, K, dtype=dtype)
    xh[torch.arange(M), ks] = 1.0
    yh = ops.hqq_mixed_mm_small(xh.to(dev), packed, s, z, g)
    want = torch.from_numpy(w_ref[ks.numpy()].astype(np.int16)).view(dtype)
    exact = bool(torch.equal(yh.cpu(), want))
    assert exact


def test_fused_product_limits():
    from ao_amd import ops
    from ao_amd.prototype.hqq import mixed_mm, pack_2xint4

    dev = _dev()
    W_q, scale, zero = _hqq_like(64, 128, 64, torch.float16, seed=1)
    b = pack_2xint4(W_q.T.contiguous()).to(dev)
    s, z = scale.T.contiguous().to(dev), zero.T.contiguous().to(dev)
    with pytest.raises(RuntimeError, match="1 to 16 rows"):
        ops.hqq_mixed_mm_small(torch.randn(17, 128, dtype=torch.float16, device=dev), b, s, z, 64)
    # 17 rows go the two-pass way through the module-level entry point
    y = mixed_mm(torch.randn(17, 128, dtype=torch.float16, device=dev), b, s, z, 64)
    assert y.shape == (17, 64)


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("transposed", [False, True])
@pytest.mark.parametrize("M,N,K,g", [(1, 4096, 4096, 64), (16, 128, 128, 128), (17, 1008, 520, 8), (33, 4096, 11008, 128),
                                     (64, 11008, 4096, 64), (9, 48, 100, 2), (40, 64, 2048, 32)])
def test_matrix_core_product_matches_the_dequantized_matmul(oracle, M, N, K, g, dtype, transposed, signed):
    """The matrix-core kernel (1-64 rows, forward and transposed): within 1e-3 relative L2 of the float64 product with
    the oracle's dequantized weight (rounded to the output dtype), and exactly the dequantized weight on one-hot rows:
    the kernel rounds every weight as ao_amd_hqq_dequantize does.  N = 1008 and 48 leave lanes of the last tile without
    columns, K = 520 and 100 leave the last reduction step / the last tile of byte rows partly empty; K = 100 and
    group 2 are legal only for the transposed product: the forward one refuses them."""
    from ao_amd import ops
    from ao_amd.prototype.hqq import pack_2xint4

    if not transposed and (K % 8 or g % 8):
        with pytest.raises(RuntimeError, match="multiples of 8"):
            W_q, scale, zero = _hqq_like(N, K, g, dtype, seed=1, signed=signed)
            ops.hqq_mixed_mm_mfma(torch.zeros(M, K, dtype=dtype, device=_dev()), pack_2xint4(W_q.T.contiguous()).to(_dev()),
                                  scale.T.contiguous().to(_dev()), zero.T.contiguous().to(_dev()), g, False)
        return
    print(f"case hqq mfma M={M} N={N} K={K} g={g} {dtype} transposed={transposed} signed={signed}", flush=True)
    dev = _dev()
    W_q, scale, zero = _hqq_like(N, K, g, dtype, seed=M + N + g, signed=signed)
    packed = pack_2xint4(W_q.T.contiguous()).to(dev)
    s, z = scale.T.contiguous().to(dev), zero.T.contiguous().to(dev)
    code = oracle.BF16 if dtype is torch.bfloat16 else oracle.F16
    w_ref = oracle.hqq_dequantize(packed.cpu().numpy(), bits16(s.cpu()), bits16(z.cpu()), g, code)   # [K, N] bits
    w_f64 = (oracle.bf16_bits_to_f32(w_ref) if dtype is torch.bfloat16 else w_ref.view(np.float16)).astype(np.float64)
    R = N if transposed else K          # reduction length
    x = torch.randn(M, R, dtype=dtype, generator=torch.Generator().manual_seed(3)).to(dev)
    y = ops.hqq_mixed_mm_mfma(x, packed, s, z, g, transposed)
    assert y.shape == (M, K if transposed else N) and y.dtype is dtype
    ref = x.float().cpu().numpy().astype(np.float64) @ (w_f64.T if transposed else w_f64)
    ref_r = torch.from_numpy(ref).to(dtype).float().numpy()
    err = rel_l2(y.float().cpu().numpy(), ref_r)
    assert err <= 1e-3, err
    # a second call with a padded, strided activation gives the same bits
    xp = torch.zeros(M, R + 8, dtype=dtype, device=dev)
    xp[:, :R] = x
    same = bool(torch.equal(ops.hqq_mixed_mm_mfma(xp[:, :R], packed, s, z, g, transposed), y))
    assert same
    # one-hot rows read single rows (forward) or columns (transposed) of the weight back, bit for bit
    idx = torch.randint(0, R, (M,), generator=torch.Generator().manual_seed(4))
    idx[0], idx[-1] = 0, R - 1
    xh = torch.zeros(M, R, dtype=dtype)
    xh[torch.arange(M), idx] = 1.0
    yh = ops.hqq_mixed_mm_mfma(xh.to(dev), packed, s, z, g, transposed)
    picked = w_ref[:, idx.numpy()].T if transposed else w_ref[idx.numpy()]
    want = torch.from_numpy(np.ascontiguousarray(picked).astype(np.int16)).view(dtype)
    exact = bool(torch.equal(yh.cpu(), want))
    assert exact


def test_matrix_core_product_limits():
    from ao_amd import ops
    from ao_amd.prototype.hqq import pack_2xint4

    dev = _dev()
    W_q, scale, zero = _hqq_like(64, 128, 64, torch.float16, seed=1)
    b = pack_2xint4(W_q.T.contiguous()).to(dev)
    s, z = scale.T.contiguous().to(dev), zero.T.contiguous().to(dev)
    with pytest.raises(RuntimeError, match="1 to 64 rows"):
        ops.hqq_mixed_mm_mfma(torch.randn(65, 128, dtype=torch.float16, device=dev), b, s, z, 64, False)
    with pytest.raises(RuntimeError, match="incompatible dimensions"):
        ops.hqq_mixed_mm_mfma(torch.randn(4, 64, dtype=torch.float16, device=dev), b, s, z, 64, False)
    with pytest.raises(RuntimeError, match="transpose requires"):
        ops.hqq_mixed_mm_mfma(torch.randn(4, 128, dtype=torch.float16, device=dev), b, s, z, 64, True)
    # N = 40: fine forward (multiple of 4), refused transposed (needs a multiple of 16)
    W_q, scale, zero = _hqq_like(40, 128, 64, torch.float16, seed=2)
    b = pack_2xint4(W_q.T.contiguous()).to(dev)
    s, z = scale.T.contiguous().to(dev), zero.T.contiguous().to(dev)
    assert ops.hqq_mixed_mm_mfma(torch.randn(4, 128, dtype=torch.float16, device=dev), b, s, z, 64, False).shape == (4, 40)
    with pytest.raises(RuntimeError, match="multiple of 16"):
        ops.hqq_mixed_mm_mfma(torch.randn(4, 40, dtype=torch.float16, device=dev), b, s, z, 64, True)
