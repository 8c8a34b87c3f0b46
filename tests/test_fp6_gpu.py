"""GPU parity tests of the FP6-LLM path through the C ABI / ops: quantize+pack bit-exact against the oracle
(which is pinned to the reference's packer and cast tables), dequantize bit-exact, linear within the reference
test's tolerance (mean relative error < 1e-3, test/test_ops.py:47-62) and the north star's 1e-3 relative L2."""
import numpy as np
import pytest
import torch

from _util import bits16, rel_l2

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(64, 64), (256, 128), (512, 1024)])
def test_quantize_pack_bit_exact(oracle, shape, dtype):
    from ao_amd import ops

    N, K = shape
    print(f"case fp6 quantize_pack N={N} K={K} {dtype}", flush=True)
    g = torch.Generator().manual_seed(N + K)
    w = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    w[1, :] = 0          # all-zero row: scale clamps at 1e-12 / 28
    w[2, 5] = 3.0        # outlier
    data, scale = ops.fp6_quantize_pack(w.to(_dev()), 3, 2)
    code = {torch.float32: oracle.F32, torch.bfloat16: oracle.BF16, torch.float16: oracle.F16}[dtype]
    wn = w.numpy() if dtype is torch.float32 else bits16(w)
    codes_ref, scale_ref = oracle.fpx_quantize(wn, code, 3, 2)
    packed_ref = oracle.pack_tc_fp6(codes_ref)
    assert np.array_equal(bits16(scale), scale_ref)
    assert np.array_equal(data.cpu().numpy(), packed_ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("fmt", [(3, 2), (2, 3)])
@pytest.mark.parametrize("shape", [(64, 64), (128, 4096), (64, 8192), (128, 14336), (64, 16384), (64, 16448)])
def test_quantize_pack_16_bit_rows_bit_exact_on_edge_cases(oracle, shape, fmt, dtype):
    """The one-pass kernel for 16-bit weights (rows of up to 16384 values; the last shape is past it and takes the
    three-launch path): the division by the row scale is a reciprocal with two corrections and the cast is the hardware's
    8-bit float conversion, so the cases are the ones where either could differ from the reference's division and
    bitwise cast: ties of the FP6 grid (scale a power of two), values a hair off the ties, signed zeros, a row that is
    all zero, rows so small or large that the scale leaves the range the shortcut is used in, NaN and inf."""
    from ao_amd import ops

    N, K = shape
    ebits, mbits = fmt
    print(f"case fp6 quantize_pack edge rows N={N} K={K} e{ebits}m{mbits} {dtype}", flush=True)
    g = torch.Generator().manual_seed(N * 7 + K + ebits)
    w = (torch.randn(N, K, generator=g) * torch.logspace(-3, 1, N).unsqueeze(1)).float()
    max_normal = {(3, 2): 28.0, (2, 3): 7.5}[fmt]
    # row 0: amax = max_normal * 2^-6, so the scale is 2^-6 and every multiple of the half step is a tie
    steps = torch.arange(K) % 449
    w[0] = (steps.float() - 224.0) * (max_normal / 224.0) * 2.0 ** -6 * (0.25 if fmt == (3, 2) else 1.0)
    w[0, 0] = max_normal * 2.0 ** -6
    # row 1: the same grid, nudged by the input dtype's own rounding
    w[1] = w[0] * (1.0 + 2.0 ** -9)
    w[2] = 0.0
    w[2, 1::2] = -0.0
    w[3] = w[3] * 0.0 + 1e-30 if dtype is torch.bfloat16 else w[3] * 1e-7     # far below the 1e-12 clamp / fp16 subnormals
    w[4, ::3] = -0.0
    w[5] = w[5].abs() * -1.0
    if dtype is torch.bfloat16:
        w[6] = w[6] * 1e30          # scale beyond the shortcut's range
        w[7] = w[7] * 1e-25
    w[8, 3] = float("inf")
    w[9, 5] = float("nan")
    w[10, 7] = float("-inf")
    w[11] = 65504.0 if dtype is torch.float16 else 3.0e38
    w[11, ::2] = -w[11, ::2] * 0.5
    wd = w.to(dtype)
    data, scale = ops.fp6_quantize_pack(wd.to(_dev()), ebits, mbits)
    code = {torch.bfloat16: oracle.BF16, torch.float16: oracle.F16}[dtype]
    codes_ref, scale_ref = oracle.fpx_quantize(bits16(wd), code, ebits, mbits)
    packed_ref = oracle.pack_tc_fp6(codes_ref)
    bad_scales = np.nonzero(bits16(scale) != scale_ref)[0].tolist()
    got = oracle.unpack_tc_fp6(data.cpu().numpy(), N, K)
    bad_rows = np.nonzero((got != codes_ref).any(axis=1))[0].tolist()
    assert bad_scales == [] and bad_rows == []
    assert np.array_equal(data.cpu().numpy(), packed_ref)


def test_dequantize_and_repack_round_trip(oracle):
    from ao_amd import ops

    dev = _dev()
    rng = np.random.default_rng(3)
    N, K = 128, 192
    codes = rng.integers(0, 64, (N, K), dtype=np.uint8)
    scale = (rng.random(N) * 0.01 + 1e-3).astype(np.float16)
    packed = oracle.pack_tc_fp6(codes)
    pd = torch.from_numpy(packed).to(dev)
    sd = torch.from_numpy(scale).to(dev)
    out = ops.fp6_dequantize(pd, sd, 3, 2).cpu().numpy()
    ref = oracle.fpx_to_f32(codes, 3, 2) * scale.astype(np.float32)[:, None]
    assert np.array_equal(out, ref)
    out_noscale = ops.fp6_dequantize(pd, None, 3, 2).cpu().numpy()
    assert np.array_equal(out_noscale, oracle.fpx_to_f32(codes, 3, 2))
    # native order: value i of lane (row%16, k%128/32) at bit 6*i, K padded to 256 with zero codes
    native = ops.fp6_repack(pd).cpu().numpy().view(np.uint32).reshape(N // 16, 2, 384)
    for (row, k) in [(0, 0), (5, 7), (17, 33), (127, 191), (64, 100), (31, 127), (40, 128)]:
        tile = native[row // 16, k // 128]
        lane = (row % 16) + 16 * ((k % 128) // 32)
        words = np.concatenate([tile[lane * 4: lane * 4 + 4], tile[256 + lane * 2: 256 + lane * 2 + 2]])
        big = sum(int(wd) << (32 * j) for j, wd in enumerate(words))
        assert (big >> (6 * (k % 32))) & 63 == codes[row, k]
    assert np.all(native[:, 1, :].reshape(-1, 384)[:, :0] == 0)


@pytest.mark.parametrize("M", [1, 2, 16, 40, 130, 257])
@pytest.mark.parametrize("shape", [(256, 1024), (2048, 4096), (512, 192), (320, 256)])
def test_linear_matches_oracle(oracle, shape, M):
    """Shapes include the reference op test's (BS, OC, IC) = (1, 2048, 4096) (test/test_ops.py:49-51); inputs as there:
    activations rand + 0.5, random bytes as weights, scales rand + 0.5."""
    from ao_amd import ops

    N, K = shape
    print(f"case fp6 linear N={N} K={K} M={M}", flush=True)
    dev = _dev()
    g = torch.Generator().manual_seed(N * 3 + K + M)
    x = (torch.rand(M, K, generator=g) + 0.5).half()
    packed = torch.randint(0, 256, (N, K // 8 * 6), dtype=torch.uint8, generator=g)
    scale = (torch.rand(N, generator=g) + 0.5).half()
    y = ops.quant_llm_linear(3, 2, x.to(dev), packed.to(dev), scale.to(dev), 1).float().cpu().numpy()
    codes = oracle.unpack_tc_fp6(packed.numpy(), N, K)
    y_ref = oracle.fpx_linear(bits16(x), codes, bits16(scale), 3, 2)
    y_ref16 = y_ref.astype(np.float16).astype(np.float32)
    assert rel_l2(y, y_ref16) <= 1e-3
    rel = np.abs(y - y_ref16) / np.maximum(np.abs(y_ref16), 1e-6)
    assert rel.mean() < 1e-3


@pytest.mark.parametrize("N,K,M", [(14336, 1024, 16), (14336, 512, 8), (6144, 576, 5), (3072, 320, 40), (2048, 192, 100), (4096, 4096, 16),
                                   (14336, 1024, 17), (12288, 512, 32), (14336, 4096, 29)])
def test_linear_with_shared_activation_tiles_matches_oracle(oracle, N, K, M):
    """Sizes at which a wave of the few-row kernel multiplies one activation tile against 4 or 2 row blocks (4 or more
    activation rows, 192 or more workgroups left), with whole and half last K tiles and more than one 16-row chunk;
    and 17 to 32 rows on weights with 768 or more row blocks, where two activation blocks share each weight fragment."""
    from ao_amd import ops

    print(f"case fp6 linear shared activation tiles N={N} K={K} M={M}", flush=True)
    dev = _dev()
    g = torch.Generator().manual_seed(N + K + M)
    x = (torch.rand(M, K, generator=g) + 0.5).half()
    packed = torch.randint(0, 256, (N, K // 8 * 6), dtype=torch.uint8, generator=g)
    scale = (torch.rand(N, generator=g) + 0.5).half()
    y = ops.quant_llm_linear(3, 2, x.to(dev), packed.to(dev), scale.to(dev), 1).float().cpu().numpy()
    codes = oracle.unpack_tc_fp6(packed.numpy(), N, K)
    y_ref16 = oracle.fpx_linear(bits16(x), codes, bits16(scale), 3, 2).astype(np.float16).astype(np.float32)
    assert rel_l2(y, y_ref16) <= 1e-3
    rel = np.abs(y - y_ref16) / np.maximum(np.abs(y_ref16), 1e-6)
    assert rel.mean() < 1e-3


def test_e2m3_format(oracle):
    from ao_amd import ops

    dev = _dev()
    g = torch.Generator().manual_seed(11)
    N, K = 256, 256
    w = (torch.randn(N, K, generator=g) * 0.05)
    data, scale = ops.fp6_quantize_pack(w.to(dev), 2, 3)
    codes_ref, scale_ref = oracle.fpx_quantize(w.numpy(), oracle.F32, 2, 3)
    assert np.array_equal(data.cpu().numpy(), oracle.pack_tc_fp6(codes_ref))
    assert np.array_equal(bits16(scale), scale_ref)
    x = torch.randn(3, K, generator=g).half()
    y = ops.quant_llm_linear(2, 3, x.to(dev), data, scale, 1).float().cpu().numpy()
    y_ref = oracle.fpx_linear(bits16(x), codes_ref, scale_ref, 2, 3).astype(np.float16).astype(np.float32)
    assert rel_l2(y, y_ref) <= 1e-3


@pytest.mark.parametrize("fmt", [(2, 2), (3, 1)])
@pytest.mark.parametrize("shape", [(64, 64), (256, 384), (512, 1024)])
def test_fp5_formats(oracle, fmt, shape):
    """e2m2 / e3m1 (torchao/csrc/cuda/fp6_llm/fp6_linear.cu:176-183): quantize + pack bit-exact against the oracle's
    cast and the generic 1 + 4 bit packer, dequantize exact, linear within the reference test's tolerance
    (test/test_ops.py:47-62 runs e2m2 alongside e3m2)."""
    from ao_amd import ops
    from ao_amd.prototype.quant_llm import QuantLlmLinearWeight

    ebits, mbits = fmt
    N, K = shape
    print(f"case fp5 e{ebits}m{mbits} N={N} K={K}", flush=True)
    dev = _dev()
    g = torch.Generator().manual_seed(N + K + ebits)
    w = (torch.randn(N, K, generator=g) * 0.05).half()
    data, scale = ops.fp6_quantize_pack(w.to(dev), ebits, mbits)
    codes_ref, scale_ref = oracle.fpx_quantize(bits16(w), oracle.F16, ebits, mbits)
    assert data.shape == (N, K * 5 // 8)
    assert np.array_equal(data.cpu().numpy(), oracle.pack_tc_fpx_generic(codes_ref, 5))
    assert np.array_equal(bits16(scale), scale_ref)
    dq = ops.fp6_dequantize(data, scale, ebits, mbits).cpu().numpy()
    assert np.array_equal(dq, oracle.fpx_to_f32(codes_ref, ebits, mbits) * scale_ref.view(np.float16).astype(np.float32)[:, None])
    for M in (1, 5, 40, 300):
        x = (torch.rand(M, K, generator=g) + 0.5).half()
        y = ops.quant_llm_linear(ebits, mbits, x.to(dev), data, scale, 1).float().cpu().numpy()
        y_ref = oracle.fpx_linear(bits16(x), codes_ref, scale_ref, ebits, mbits).astype(np.float16).astype(np.float32)
        assert rel_l2(y, y_ref) <= 1e-3, M
    if N % 256 == 0:
        qw = QuantLlmLinearWeight.from_float(w.to(dev), ebits, mbits)
        assert qw.shape == (N, K)
        y2 = torch.nn.functional.linear(x.to(dev), qw).float().cpu().numpy()
        assert rel_l2(y2, y_ref) <= 1e-3


def test_weight_subclass_and_api(oracle):
    """quantize(model, fp6_llm_weight_only()): shapes the kernel cannot take stay float; forward matches the oracle;
    leading dims and bias work (test/prototype/test_quant_llm.py:68-99)."""
    import ao_amd
    from ao_amd.prototype.quant_llm import QuantLlmLinearWeight

    dev = _dev()
    torch.manual_seed(0)
    m = torch.nn.Sequential(torch.nn.Linear(256, 512, bias=True), torch.nn.Linear(512, 100, bias=False)).half().to(dev)
    w0 = m[0].weight.detach().clone()
    ao_amd.quantize(m, ao_amd.fp6_llm_weight_only())
    assert isinstance(m[0].weight, QuantLlmLinearWeight) and m[0].weight.shape == (512, 256)
    assert not isinstance(m[1].weight, QuantLlmLinearWeight)  # 100 outputs: not a multiple of 256
    x = torch.randn(2, 3, 256, device=dev).half()
    with torch.no_grad():
        y = m[0](x)
    assert y.shape == (2, 3, 512) and y.dtype is torch.float16
    codes, scale = oracle.fpx_quantize(bits16(w0), oracle.F16, 3, 2)
    y_ref = oracle.fpx_linear(bits16(x.reshape(-1, 256)), codes, scale, 3, 2).astype(np.float16).astype(np.float32)
    y_ref = (torch.from_numpy(y_ref).half() + m[0].bias.detach().cpu()).float().numpy()
    assert rel_l2(y.float().cpu().numpy().reshape(-1, 512), y_ref) <= 2e-3
    dq = m[0].weight.dequantize(torch.float32).cpu().numpy()
    ref = oracle.fpx_to_f32(codes, 3, 2) * scale.view(np.float16).astype(np.float32)[:, None]
    assert np.array_equal(dq, ref)


@pytest.mark.parametrize("fmt,shape", [((3, 2), (256, 1024)), ((3, 2), (512, 192)), ((2, 3), (320, 256)), ((2, 2), (128, 320)),
                                       ((3, 1), (64, 128))])
def test_native_to_fp16_is_the_scaled_weight_and_feeds_the_two_pass_linear(oracle, fmt, shape, monkeypatch):
    """Prefill path: the native tiles converted to an fp16 matrix are bit for bit fp16(fpx value * scale) (oracle codes
    and scales, one fp16 multiply each, zero rows / ragged last K tile included), and the op's result from 1024 rows on
    (library GEMM on that matrix) stays within the op's tolerance of the oracle."""
    from ao_amd import _lib, ops

    e, m = fmt
    N, K = shape
    print(f"case fp6 two-pass fmt={fmt} N={N} K={K}", flush=True)
    dev = _dev()
    g = torch.Generator().manual_seed(N + K + e)
    w = (torch.randn(N, K, generator=g) * 0.05).half()
    w[3] = 0
    data, scale = ops.fp6_quantize_pack(w.to(dev), e, m)
    native = ops.fp6_repack(data, 1 + e + m)
    w16 = torch.empty((N, K), dtype=torch.float16, device=dev)
    _lib.check(_lib.lib().ao_amd_fp6_native_to_f16(native.data_ptr(), scale.data_ptr(), N, K, e, m, w16.data_ptr(),
                                                   _lib.current_stream(dev)))
    values = ops.fp6_dequantize(data, None, e, m)              # exact fpx values (fp32), unscaled
    want = (values.half() * scale.view(-1, 1))                  # one fp16 multiply, as the kernels do
    assert np.array_equal(bits16(w16), bits16(want))
    M = ops.FP6_TWO_PASS_MIN_M
    assert ops.fp6_two_pass(M, 14336, 4096) and not ops.fp6_two_pass(M, 1024, 4096) and ops.fp6_two_pass(3 * M, 1024, 4096)
    x = (torch.rand(M, K, generator=g) + 0.5).half().to(dev)
    monkeypatch.setattr(ops, "fp6_two_pass", lambda M, N, K: True)   # these small weights would stay on the fused kernel
    y = ops.fp6_linear_native(e, m, x, native, scale).float().cpu().numpy()
    ref = (x.double() @ want.double().t()).cpu().numpy()
    ref16 = ref.astype(np.float16).astype(np.float32)
    assert rel_l2(y, ref16) <= 1e-3
    monkeypatch.setattr(ops, "fp6_two_pass", lambda M, N, K: False)
    y_small = ops.fp6_linear_native(e, m, x[:64], native, scale).float().cpu().numpy()   # fused kernel, same rows
    assert rel_l2(y[:64], y_small) <= 1e-3
