"""CPU pins of the oracle's HQQ mixed-matmul dequantization (reference torchao/prototype/hqq/kernels.py:318-358,
mixed_mm.py:13-35).  The reference's own test (test/hqq/test_triton_mm.py) needs the `hqq` package and a GPU, neither of
which exists here; its oracle is `x @ W_dq` with W_dq = (W_q - zero) * scale computed by torch in the compute dtype,
which is what these tests restate with engines independent of the C code: numpy's float16 arithmetic and torch's CPU
bfloat16 arithmetic (both round after every operation)."""
import numpy as np
import pytest
import torch

from _util import bits16


def _pack_ref(codes_kn):
    """Element-by-element restatement of pack_2xint4's documented example (mixed_mm.py:14-31): consecutive rows
    2i, 2i+1 share byte row i, the even row in the low nibble."""
    K, N = codes_kn.shape
    out = np.zeros((K // 2, N), np.uint8)
    for k in range(K):
        for n in range(N):
            out[k // 2, n] |= (int(codes_kn[k, n]) & 15) << (4 * (k & 1))
    return out


def test_pack_2xint4_matches_the_documented_example_and_a_brute_force_packer():
    from ao_amd.prototype.hqq import pack_2xint4

    t = torch.arange(16, dtype=torch.uint8).reshape(4, 4)
    assert pack_2xint4(t).tolist() == [[0 | 4 << 4, 1 | 5 << 4, 2 | 6 << 4, 3 | 7 << 4],
                                       [8 | 12 << 4, 9 | 13 << 4, 10 | 14 << 4, 11 | 15 << 4]]
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 16, (12, 7), dtype=np.uint8)
    assert np.array_equal(pack_2xint4(torch.from_numpy(codes)).numpy(), _pack_ref(codes))
    signed = rng.integers(-8, 8, (6, 5)).astype(np.int8)
    assert np.array_equal(pack_2xint4(torch.from_numpy(signed)).numpy().view(np.uint8), _pack_ref(signed))


@pytest.mark.parametrize("signed", [False, True])
def test_unit_scale_returns_the_codes(oracle, signed):
    """zero = 0, scale = 1: the dequantized matrix is the code matrix itself, which pins the nibble order, the
    row interleaving and the sign handling."""
    rng = np.random.default_rng(1)
    K, N, g = 8, 16, 4
    codes = rng.integers(-8, 8, (K, N)).astype(np.int8) if signed else rng.integers(0, 16, (K, N)).astype(np.uint8)
    packed = _pack_ref(codes).view(np.int8 if signed else np.uint8)
    one = np.full((K // g, N), 0x3C00, np.uint16)   # fp16 1.0
    zero = np.zeros((K // g, N), np.uint16)
    out = oracle.hqq_dequantize(packed, one, zero, g, oracle.F16)
    assert np.array_equal(out.view(np.float16).astype(np.int32), codes.astype(np.int32))
    one_bf = np.full((K // g, N), 0x3F80, np.uint16)  # bf16 1.0
    out = oracle.hqq_dequantize(packed, one_bf, zero, g, oracle.BF16)
    assert np.array_equal(oracle.bf16_bits_to_f32(out).astype(np.int32), codes.astype(np.int32))


@pytest.mark.parametrize("g", [2, 8, 32])
def test_fp16_against_numpy_half_arithmetic(oracle, g):
    rng = np.random.default_rng(g)
    K, N = 64, 48
    codes = rng.integers(0, 16, (K, N), dtype=np.uint8)
    s = (rng.random((K // g, N)) * 0.02 + 1e-3).astype(np.float16)
    z = (rng.random((K // g, N)) * 6 + 5).astype(np.float16)
    out = oracle.hqq_dequantize(_pack_ref(codes), s.view(np.uint16), z.view(np.uint16), g, oracle.F16)
    expect = (codes.astype(np.float16) - np.repeat(z, g, axis=0)) * np.repeat(s, g, axis=0)  # float16 op by op
    assert expect.dtype == np.float16
    assert np.array_equal(out, expect.view(np.uint16))


@pytest.mark.parametrize("g", [2, 16, 64])
def test_bf16_against_torch_cpu_arithmetic(oracle, g):
    gen = torch.Generator().manual_seed(g)
    K, N = 128, 32
    codes = torch.randint(0, 16, (K, N), generator=gen, dtype=torch.uint8)
    s = (torch.rand(K // g, N, generator=gen) * 0.02 + 1e-3).bfloat16()
    z = (torch.rand(K // g, N, generator=gen) * 6 + 5).bfloat16()
    out = oracle.hqq_dequantize(_pack_ref(codes.numpy()), bits16(s), bits16(z), g, oracle.BF16)
    expect = (codes.to(torch.bfloat16) - z.repeat_interleave(g, 0)) * s.repeat_interleave(g, 0)  # bf16 op by op
    assert expect.dtype is torch.bfloat16
    assert np.array_equal(out, bits16(expect))


def test_conversion_to_the_affine_form_keeps_codes_and_reconstruction():
    """HQQ (W_q - zero) * scale against the affine (q - 8) * scale + zero' produced by the converter: the codes come
    back unchanged and zero' = 8 * scale - zero * scale (closed form of the reference's derivation, :189-193), so
    both forms reconstruct the same weight up to the bf16 rounding of zero'.  Runs on the CPU (plain torch ops)."""
    from ao_amd.prototype.hqq.hqq_tinygemm_linear import hqq_to_affine_int4

    gen = torch.Generator().manual_seed(5)
    N, K, g = 24, 256, 64
    W_q = torch.randint(0, 16, (N * K // g, g), generator=gen).float()
    scale = (torch.rand(N * K // g, 1, generator=gen) * 0.02 + 1e-3).bfloat16()
    zero = (torch.rand(N * K // g, 1, generator=gen) * 6 + 5).bfloat16()
    codes, s, z_aff = hqq_to_affine_int4(W_q, scale, zero, (N, K), 4, torch.bfloat16, "cpu")
    assert codes.dtype is torch.int32 and codes.shape == (N, K) and s.shape == z_aff.shape == (N, K // g)
    assert torch.equal(codes, W_q.reshape(N, K).to(torch.int32))
    assert torch.equal(s, scale.reshape(N, K // g))
    exact = 8 * scale.double() - zero.double() * scale.double()
    # 8 * scale is exact in bf16; zero * scale (zero <= 11) rounds once, the difference once more
    bound = 2.0 ** -8 * 11 * scale.double()
    assert bool(((z_aff.double().reshape(-1, 1) - exact).abs() <= bound).all())
    hqq_w = ((W_q.double() - zero.double()) * scale.double()).reshape(N, K)
    aff_w = (codes.double() - 8) * s.double().repeat_interleave(g, 1) + z_aff.double().repeat_interleave(g, 1)
    assert bool(((hqq_w - aff_w).abs() <= bound.reshape(N, K // g).repeat_interleave(g, 1)).all())
