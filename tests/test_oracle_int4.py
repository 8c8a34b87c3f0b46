"""Pins the CPU oracle of the affine primitives (CPU only, no GPU).

The checks are independent of the oracle's C code: the legacy tinygemm closed forms that the
reference's own tests hold (test/quantization/test_quant_primitives.py:50-127) are evaluated by
torch's CPU kernels -- for bf16 tensors those kernels round after every op by themselves -- and
torch.ops.quantized_decomposed.* covers the integer zero-point domain.  A dropped rounding, a wrong
sign or mid-point, or eps applied in the wrong place fails at least one of them.
"""
import numpy as np
import pytest
import torch

from _util import bits16, from_bits16, make_weight

_SEED = 1234  # seed of the reference's test module


def _legacy_qparams(w, n_bit=4, groupsize=128, dtype=torch.bfloat16):
    """test_quant_primitives.py:50-67 (ops run in w's dtype)."""
    to_quant = w.reshape(-1, groupsize)
    max_val = to_quant.amax(dim=1, keepdim=True)
    min_val = to_quant.amin(dim=1, keepdim=True)
    max_int = 2**n_bit - 1
    scales = (max_val - min_val).clamp(min=1e-6) / max_int
    zeros = min_val + scales * (2 ** (n_bit - 1))
    return scales.to(dtype).reshape(w.shape[0], -1), zeros.to(dtype).reshape(w.shape[0], -1)


def _legacy_quantize(w, scales, zeros, n_bit=4, groupsize=128):
    """test_quant_primitives.py:69-101."""
    to_quant = w.reshape(-1, groupsize)
    scales = scales.reshape(-1, 1)
    zeros = zeros.reshape(-1, 1)
    min_val = zeros - scales * (2 ** (n_bit - 1))
    return to_quant.sub(min_val).div(scales).round().clamp_(0, 2**n_bit - 1).to(torch.int32).reshape_as(w)


def _legacy_dequantize(q, scales, zeros, n_bit=4, groupsize=128):
    """test_quant_primitives.py:103-127."""
    qg = q.reshape(-1, groupsize)
    return qg.sub(2 ** (n_bit - 1)).mul(scales.reshape(-1, 1)).add(zeros.reshape(-1, 1)).reshape_as(q)


def _np(t):
    return t.detach().contiguous().numpy()


def test_choose_qparams_fp32_matches_legacy_form(oracle):
    """test_get_groupwise_affine_qparams (:451-480): fp32 input, bf16 qparams."""
    torch.manual_seed(_SEED)
    x = torch.randn(10, 256)
    s_ref, z_ref = _legacy_qparams(x, 4, 128, torch.bfloat16)
    s, z = oracle.choose_qparams_affine(_np(x), oracle.F32, (1, 128), 1, 0, 15, eps=1e-6, preserve_zero=False,
                                        zp_domain=1, scale_dtype=oracle.BF16, zp_dtype=oracle.BF16)
    assert np.array_equal(s, bits16(s_ref))
    assert np.array_equal(z, bits16(z_ref))


@pytest.mark.parametrize("g", [32, 64, 128, 256])
def test_choose_qparams_bf16_stepwise(oracle, g):
    """bf16 weights: every torch op rounds to bf16, so the closed form evaluated on bf16 tensors is the
    op-by-op chain of quant_primitives.py:355-365 (clamp applied to the scale after the division)."""
    w = make_weight(64, 1024, seed=g)
    w[3, :g] = 0.0123  # a whole constant group
    wg = w.view(64, 1024 // g, g)
    mn, mx = wg.amin(-1), wg.amax(-1)
    s0 = (mx - mn) / 15.0
    zp = mn + s0 * 8.0
    s = torch.clamp(s0, min=1e-6)
    so, zo = oracle.choose_qparams_affine(bits16(w), oracle.BF16, (1, g), 1, 0, 15, eps=1e-6, preserve_zero=False,
                                          zp_domain=1)
    assert np.array_equal(so, bits16(s)) and np.array_equal(zo, bits16(zp))
    # the planted constant group clamps to bf16(1e-6) = 0x3586 while its zero point used the raw scale
    assert so[3, 0] == 0x3586
    assert zo[3, 0] == bits16(torch.tensor([0.0123]).bfloat16())[0]


def test_quantize_fp32_matches_legacy_form(oracle):
    """test_groupwise_affine_quantize_tensor_from_qparams (:482-492)."""
    torch.manual_seed(_SEED)
    x = torch.randn(10, 256)
    scales = torch.randn(10, 2)
    zeros = torch.randn(10, 2)
    ref = _legacy_quantize(x, scales, zeros)
    q = oracle.quantize_affine(_np(x), oracle.F32, (1, 128), _np(scales), oracle.F32, _np(zeros), oracle.F32, 0, 15,
                               zp_domain=1)
    assert np.array_equal(q, ref.numpy())


def test_dequantize_bf16_matches_legacy_form(oracle):
    """test_groupwise_affine_dequantize_tensor_from_qparams (:494-504)."""
    torch.manual_seed(_SEED)
    q = torch.randint(0, 15, (10, 256), dtype=torch.int32)
    scales = torch.randn(10, 2).bfloat16()
    zeros = torch.randn(10, 2).bfloat16()
    # the reference subtracts the python float 8.0 from the int tensor (fp32), casts to bf16, then
    # multiplies and adds in place in bf16
    dq = (q.reshape(-1, 128) - 8.0).to(torch.bfloat16)
    dq *= scales.reshape(-1, 1)
    dq += zeros.reshape(-1, 1)
    out = oracle.dequantize_affine(q.numpy(), oracle.I32, (1, 128), bits16(scales), oracle.BF16, bits16(zeros),
                                   oracle.BF16, 0, 15, zp_domain=1, out_dtype=oracle.BF16)
    assert np.array_equal(out, bits16(dq.reshape(10, 256)))


@pytest.mark.parametrize("g", [32, 64, 128])
def test_int4wo_chain_bf16(oracle, g):
    """Whole int4 weight-only chain on bf16 weights against torch's bf16 kernels, incl. invariants."""
    w = make_weight(48, 512, seed=7 * g)
    wg = w.view(48, 512 // g, g)
    mn, mx = wg.amin(-1, keepdim=True), wg.amax(-1, keepdim=True)
    s0 = (mx - mn) / 15.0
    zp = mn + s0 * 8.0
    s = torch.clamp(s0, min=1e-6)
    mv = zp - s * 8.0
    q_ref = torch.clamp(torch.round((wg - mv) / s), 0, 15).to(torch.int32).view(48, 512)
    dq_ref = (q_ref.view(48, 512 // g, g) - 8.0).to(torch.bfloat16)
    dq_ref *= s
    dq_ref += zp
    codes, scale, zero = oracle.int4wo_quantize(bits16(w), oracle.BF16, g, 48, 512)
    assert np.array_equal(codes, q_ref.numpy())
    assert codes.min() >= 0 and codes.max() <= 15
    dq = oracle.dequantize_affine(codes, oracle.I32, (1, g), scale, oracle.BF16, zero, oracle.BF16, 0, 15, 1, oracle.BF16)
    assert np.array_equal(dq, bits16(dq_ref.view(48, 512)))
    # reconstruction error bound: half a step, plus the bf16 roundings of scale (x up to 15 steps), zero
    # point and result.  A wrong mid-point, sign or group index gives errors of several steps.
    wf = w.float().numpy()
    sf = np.repeat(oracle.bf16_bits_to_f32(scale), g, axis=1)
    err = np.abs(oracle.bf16_bits_to_f32(dq) - wf)
    assert np.all(err <= 0.75 * sf + np.abs(wf) * 2.0**-6 + 1e-6)
    # every non-constant group uses both ends of the code range
    cg = codes.reshape(48, 512 // g, g)
    nonconst = (mx - mn).squeeze(-1).float().numpy() > 1e-4
    assert np.all(cg.min(-1)[nonconst] == 0) and np.all(cg.max(-1)[nonconst] == 15)
    # quantizing the dequantized weight with the same qparams gives the codes back
    again = oracle.quantize_affine(dq, oracle.BF16, (1, g), scale, oracle.BF16, zero, oracle.BF16, 0, 15, zp_domain=1)
    assert np.array_equal(again, codes)


def test_zero_padding_semantics(oracle):
    """from_float zero-extends the weight before quantizing (affine_quantized_tensor.py:203-210): padded
    groups get scale bf16(1e-6), zero 0, code 8, and a group straddling the edge sees the zeros."""
    w = make_weight(20, 96, seed=3, special=False)
    codes, scale, zero = oracle.int4wo_quantize(bits16(w), oracle.BF16, 64, 32, 128)
    assert np.all(codes[20:, :] == 8) and np.all(scale[20:, :] == 0x3586) and np.all(zero[20:, :] == 0)
    wp = torch.zeros(32, 128, dtype=torch.bfloat16)
    wp[:20, :96] = w
    c2, s2, z2 = oracle.int4wo_quantize(bits16(wp), oracle.BF16, 64, 32, 128)
    assert np.array_equal(codes, c2) and np.array_equal(scale, s2) and np.array_equal(zero, z2)


def test_eps_default_is_dtype_eps(oracle):
    """test_choose_qparams_tensor_asym_eps (:385-392): all-zero input, per-tensor block -> scale = finfo.eps."""
    x = np.zeros((10, 10), np.float32)
    s, _ = oracle.choose_qparams_affine(x, oracle.F32, (10, 10), 1, -128, 127)
    assert s.shape == (1, 1) and s[0, 0] == np.float32(torch.finfo(torch.float32).eps)


def test_int_domain_matches_quantized_decomposed(oracle):
    """INT zero-point domain against torch's quantized_decomposed ops (what the reference's tests
    compare with at :184-371): per-tensor asymmetric uint8 and per-channel symmetric int8."""
    import torch.ao.quantization.fx._decomposed  # noqa: F401  (registers the ops)

    torch.manual_seed(_SEED)
    x = torch.randn(10, 10)
    # per tensor, asymmetric, preserve_zero
    scale_ref, zp_ref = torch.ops.quantized_decomposed.choose_qparams(x, 0, 255, torch.finfo(torch.float32).eps, torch.uint8)
    s, z = oracle.choose_qparams_affine(_np(x), oracle.F32, (10, 10), 1, 0, 255, scale_dtype=oracle.F32,
                                        zp_dtype=oracle.I64)
    np.testing.assert_allclose(s[0, 0], scale_ref.item(), rtol=1e-6)
    assert int(z[0, 0]) == int(zp_ref.item())
    q_ref = torch.ops.quantized_decomposed.quantize_per_tensor(x, float(s[0, 0]), int(z[0, 0]), 0, 255, torch.uint8)
    q = oracle.quantize_affine(_np(x), oracle.F32, (10, 10), s, oracle.F32, z, oracle.I64, 0, 255, zp_domain=0,
                               out_dtype=oracle.U8)
    assert np.array_equal(q, q_ref.numpy())
    dq_ref = torch.ops.quantized_decomposed.dequantize_per_tensor(q_ref, float(s[0, 0]), int(z[0, 0]), 0, 255, torch.uint8)
    dq = oracle.dequantize_affine(q, oracle.U8, (10, 10), s, oracle.F32, z, oracle.I64, 0, 255, zp_domain=0)
    assert np.array_equal(dq, dq_ref.numpy())
    # per channel (axis 0), symmetric int8
    s, z = oracle.choose_qparams_affine(_np(x), oracle.F32, (1, 10), 0, -128, 127, zp_dtype=oracle.I64)
    amax = x.abs().amax(dim=1)
    np.testing.assert_allclose(s[:, 0], (amax / 127.5).numpy(), rtol=1e-6)
    assert np.all(z == 0)
    q_ref = torch.ops.quantized_decomposed.quantize_per_channel(x, torch.from_numpy(s[:, 0].copy()),
                                                                torch.from_numpy(z[:, 0].copy()), 0, -128, 127, torch.int8)
    q = oracle.quantize_affine(_np(x), oracle.F32, (1, 10), s, oracle.F32, z, oracle.I64, -128, 127, zp_domain=0,
                               out_dtype=oracle.I8)
    assert np.array_equal(q, q_ref.numpy())


def test_error_paths(oracle):
    x = np.zeros((10, 256), np.float32)
    with pytest.raises(ValueError):  # symmetric + preserve_zero False (:350-351)
        oracle.choose_qparams_affine(x, oracle.F32, (1, 128), 0, 0, 15, preserve_zero=False)
    with pytest.raises(ValueError):  # block does not divide the shape
        oracle.choose_qparams_affine(x, oracle.F32, (1, 100), 1, 0, 15)


@pytest.mark.parametrize("g", [32, 64, 128, 256])
def test_pack_layout_brute_force(oracle, g):
    """The packed layout against its definition, element by element (brute force on a small weight)."""
    rng = np.random.default_rng(g)
    Np, Kp = 32, 512
    codes = rng.integers(0, 16, (Np, Kp), dtype=np.int32)
    scale = rng.integers(0, 65536, (Np, Kp // g)).astype(np.uint16)
    zero = rng.integers(0, 65536, (Np, Kp // g)).astype(np.uint16)
    packed, qparams = oracle.int4wo_pack(codes, scale, zero, g)
    assert packed.shape == (Np // 16, Kp // 128, 64, 4) and qparams.shape == (Np // 16, Kp // g, 16)
    for row in range(Np):
        for k in range(Kp):
            lane = (row % 16) + 16 * ((k % 128) // 32)
            dword = (k % 32) // 8
            e = k % 8
            shift = 4 * ((e >> 1) + 4 * (e & 1))
            assert (int(packed[row // 16, k // 128, lane, dword]) >> shift) & 15 == codes[row, k]
    for row in range(Np):
        for gi in range(Kp // g):
            v = int(qparams[row // 16, gi, row % 16])
            assert v & 0xFFFF == scale[row, gi] and v >> 16 == zero[row, gi]
    c2, s2, z2 = oracle.int4wo_unpack(packed, qparams, Np, Kp, g)
    assert np.array_equal(c2, codes) and np.array_equal(s2, scale) and np.array_equal(z2, zero)


def test_linear_against_float64(oracle):
    torch.manual_seed(0)
    w = make_weight(64, 512, seed=11)
    x = torch.randn(3, 512).bfloat16()
    bias = torch.randn(64).bfloat16()
    y = oracle.linear(bits16(x), oracle.BF16, bits16(w), oracle.BF16, bits16(bias), oracle.BF16)
    ref = x.double().numpy() @ w.double().numpy().T + bias.double().numpy()
    assert np.max(np.abs(y - ref)) <= 1e-5 * np.max(np.abs(ref))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_int8_symmetric_per_channel_stepwise(oracle, dtype):
    """The int8 weight-only recipe (symmetric, block (1, K), eps = finfo(float32).eps, zero point int64;
    torchao/quantization/quant_api.py:390-405) against torch's own CPU kernels run op by op in the weight's dtype:
    quant_primitives.py:335-367 for the parameters, :191-194 for the codes.  For bf16 tensors torch rounds after
    every op by itself, which is the behaviour the oracle has to restate."""
    w = make_weight(48, 256, seed=77, dtype=dtype)
    eps = torch.finfo(torch.float32).eps
    mn, mx = w.amin(dim=1), w.amax(dim=1)
    mn_neg, mx_pos = torch.min(mn, torch.zeros_like(mn)), torch.max(mx, torch.zeros_like(mx))
    scale_ref = torch.clamp(torch.max(-mn_neg, mx_pos) / (float(127 - (-128)) / 2), min=eps)
    q_ref = torch.clamp(torch.round(w * (1.0 / scale_ref.reshape(-1, 1))) + torch.zeros(48, 1, dtype=torch.int64),
                        -128, 127).to(torch.int8)
    code = oracle.BF16 if dtype is torch.bfloat16 else oracle.F32
    wn = bits16(w) if dtype is torch.bfloat16 else _np(w)
    s, z = oracle.choose_qparams_affine(wn, code, (1, 256), 0, -128, 127, eps=eps, zp_dtype=oracle.I64)
    if dtype is torch.bfloat16:
        assert np.array_equal(s[:, 0], bits16(scale_ref))
    else:
        assert np.array_equal(s[:, 0], _np(scale_ref))
    assert np.all(z == 0)
    q = oracle.quantize_affine(wn, code, (1, 256), s, code, z, oracle.I64, -128, 127, zp_domain=0, out_dtype=oracle.I8)
    assert np.array_equal(q, q_ref.numpy())
    assert q.min() >= -128 and q.max() <= 127 and np.abs(q).max() >= 127   # the row maximum maps to +-127 or -128
