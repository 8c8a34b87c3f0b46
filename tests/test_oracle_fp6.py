"""Pins the CPU oracle of the FP6-LLM path (CPU only).

Known answers come from the reference's own tests and tables: all 64 codes of e3m2 in both directions
(test/prototype/mx_formats/test_custom_cast.py:346-388), the RNE / underflow cases (:391-413) and the
interesting-value table (torchao/prototype/mx_formats/fp_format_spec.py:299-312).  The packer is pinned
by three independent formulations that must agree: explicit byte indices (C), the generic three-pass
view/permute packer (numpy), and an emulation of the order in which the reference CUDA kernel reads the
bytes back into mma fragments.
"""
import numpy as np
import pytest


def _e3m2_value(code):
    """Textbook e3m2: sign, 3 exponent bits (bias 3), 2 mantissa bits, subnormals, no inf/nan."""
    s = -1.0 if code & 0x20 else 1.0
    e = (code >> 2) & 7
    m = code & 3
    return s * (2.0 ** -2 * (m / 4.0) if e == 0 else 2.0 ** (e - 3) * (1 + m / 4.0))


def test_all_64_codes_both_directions(oracle):
    codes = np.arange(64, dtype=np.uint8)
    vals = oracle.fpx_to_f32(codes, 3, 2)
    assert np.array_equal(vals, np.array([_e3m2_value(c) for c in range(64)], np.float32))
    back = oracle.f32_to_fpx(vals, 3, 2)
    # -0.0 keeps its sign bit: code 32
    assert np.array_equal(back, codes)


def test_interesting_values_table(oracle):
    table = [(0.0, 0b000000), (0.0625, 0b000001), (0.1875, 0b000011), (0.25, 0b000100), (28.0, 0b011111)]
    for v, enc in table:
        assert oracle.f32_to_fpx(np.array([v], np.float32), 3, 2)[0] == enc
        assert oracle.fpx_to_f32(np.array([enc], np.uint8), 3, 2)[0] == np.float32(v)
        assert oracle.f32_to_fpx(np.array([-v], np.float32), 3, 2)[0] == enc | 0b100000
        assert oracle.fpx_to_f32(np.array([enc | 0b100000], np.uint8), 3, 2)[0] == np.float32(-v)


@pytest.mark.parametrize("val,enc", [(29.0, 0b011111), (26.0, 0b011110), (0.1251, 0b000010), (0.0314, 0b000001),
                                     (0.03, 0b000000)])
def test_rounding_known_answers(oracle, val, enc):
    assert oracle.f32_to_fpx(np.array([val], np.float32), 3, 2)[0] == enc
    assert oracle.f32_to_fpx(np.array([-val], np.float32), 3, 2)[0] == enc | 0b100000


def test_round_to_nearest_even_exhaustive(oracle):
    """Every fp32 midpoint between two neighbouring e3m2 values goes to the even code; values just
    beside the midpoint go to the nearer one; anything beyond 28 saturates."""
    grid = np.array([_e3m2_value(c) for c in range(32)], np.float64)
    for c in range(31):
        lo, hi = grid[c], grid[c + 1]
        mid = np.float32((lo + hi) / 2)
        even = c if c % 2 == 0 else c + 1
        assert oracle.f32_to_fpx(np.array([mid], np.float32), 3, 2)[0] == even
        below = np.nextafter(mid, np.float32(0), dtype=np.float32)
        above = np.nextafter(mid, np.float32(100), dtype=np.float32)
        assert oracle.f32_to_fpx(np.array([below], np.float32), 3, 2)[0] == c
        assert oracle.f32_to_fpx(np.array([above], np.float32), 3, 2)[0] == c + 1
    assert np.all(oracle.f32_to_fpx(np.array([28.0, 30.0, 1e9, np.inf], np.float32), 3, 2) == 31)
    assert np.all(oracle.f32_to_fpx(np.array([-28.5, -1e30], np.float32), 3, 2) == 63)


def test_other_formats_round_trip(oracle):
    """e2m2 (fp5) and e2m3: every code survives decode -> encode."""
    for ebits, mbits in ((2, 2), (2, 3), (3, 1)):
        n = 1 << (1 + ebits + mbits)
        codes = np.arange(n, dtype=np.uint8)
        assert np.array_equal(oracle.f32_to_fpx(oracle.fpx_to_f32(codes, ebits, mbits), ebits, mbits), codes)


@pytest.mark.parametrize("shape", [(64, 64), (256, 64), (128, 192), (256, 512)])
def test_pack_three_formulations_agree(oracle, shape):
    """test/prototype/test_quant_llm.py:27-33 compares the fast fp6 packer with the generic one; here the
    explicit-index C packer, the generic three-pass packer and the CUDA read order must all agree."""
    rng = np.random.default_rng(shape[0] * 7 + shape[1])
    codes = rng.integers(0, 64, shape, dtype=np.uint8)
    a = oracle.pack_tc_fp6(codes)
    b = oracle.pack_tc_fpx_generic(codes, 6)
    assert a.shape == (shape[0], shape[1] * 3 // 4)
    assert np.array_equal(a, b)
    assert np.array_equal(oracle.unpack_tc_fp6(a, *shape), codes)
    assert np.array_equal(oracle.fp6_cuda_read_order(a, *shape), codes)


def _fpx_value(code, ebits, mbits):
    """Textbook small float: sign, ebits exponent bits (bias 2^(ebits-1) - 1), mbits mantissa bits, subnormals,
    no inf / nan."""
    bias = (1 << (ebits - 1)) - 1
    s = -1.0 if (code >> (ebits + mbits)) & 1 else 1.0
    e = (code >> mbits) & ((1 << ebits) - 1)
    m = code & ((1 << mbits) - 1)
    frac = m / float(1 << mbits)
    return s * (2.0 ** (1 - bias) * frac if e == 0 else 2.0 ** (e - bias) * (1 + frac))


@pytest.mark.parametrize("fmt", [(2, 2), (3, 1), (2, 3)])
def test_five_bit_formats_all_codes_and_rounding(oracle, fmt):
    """e2m2 and e3m1 (the 5-bit formats the reference kernel dispatches, fp6_linear.cu:176-183) and e2m3: every
    code against the textbook value, every midpoint to the even neighbour, saturation at the largest normal
    (7.0 for e2m2, 24.0 for e3m1, 7.5 for e2m3)."""
    ebits, mbits = fmt
    n = 1 << (ebits + mbits)
    vals = oracle.fpx_to_f32(np.arange(2 * n, dtype=np.uint8), ebits, mbits)
    assert np.array_equal(vals, np.array([_fpx_value(c, ebits, mbits) for c in range(2 * n)], np.float32))
    assert np.array_equal(oracle.f32_to_fpx(vals, ebits, mbits), np.arange(2 * n, dtype=np.uint8))
    grid = np.array([_fpx_value(c, ebits, mbits) for c in range(n)], np.float64)
    assert grid[-1] == {(2, 2): 7.0, (3, 1): 24.0, (2, 3): 7.5}[fmt]
    for c in range(n - 1):
        mid = np.float32((grid[c] + grid[c + 1]) / 2)
        even = c if c % 2 == 0 else c + 1
        assert oracle.f32_to_fpx(np.array([mid], np.float32), ebits, mbits)[0] == even
        assert oracle.f32_to_fpx(np.array([np.nextafter(mid, np.float32(0), dtype=np.float32)], np.float32), ebits, mbits)[0] == c
        assert oracle.f32_to_fpx(np.array([np.nextafter(mid, np.float32(100), dtype=np.float32)], np.float32), ebits, mbits)[0] == c + 1
    assert np.all(oracle.f32_to_fpx(np.array([grid[-1], grid[-1] * 1.2, 1e9, np.inf], np.float32), ebits, mbits) == n - 1)
    # a 5-bit code and the 6-bit code with one more (zero) mantissa bit are the same number
    if 1 + ebits + mbits == 5:
        wide = oracle.fpx_to_f32((np.arange(2 * n, dtype=np.uint8) << 1).astype(np.uint8), ebits, mbits + 1)
        assert np.array_equal(wide, vals)


@pytest.mark.parametrize("shape", [(64, 64), (256, 64), (128, 192)])
def test_pack_fp5_two_formulations_agree(oracle, shape):
    """5-bit codes: the generic three-pass packer (1-bit plane, then 4-bit plane) against the order in which the
    reference CUDA kernel reads those planes back (utils_parallel_dequant.cuh:85-113)."""
    rng = np.random.default_rng(shape[0] + shape[1])
    codes = rng.integers(0, 32, shape, dtype=np.uint8)
    packed = oracle.pack_tc_fpx_generic(codes, 5)
    assert packed.shape == (shape[0], shape[1] * 5 // 8)
    assert np.array_equal(oracle.fpx_cuda_read_order(packed, shape[0], shape[1], 5), codes)
    # the 4-bit plane is the same whatever the high plane is
    p6 = oracle.pack_tc_fpx_generic(codes, 6).reshape(-1)
    assert np.array_equal(packed.reshape(-1)[codes.size // 8:], p6[codes.size // 4:])


def test_pack_single_element_positions(oracle):
    """One non-zero code at a time: its 2 high bits and 4 low bits land in exactly one byte each, in the
    right plane (first R*C/4 bytes = 2-bit plane)."""
    R, C = 64, 64
    for (r, c) in [(0, 0), (1, 0), (0, 1), (8, 3), (17, 9), (40, 31), (63, 63), (33, 48)]:
        codes = np.zeros((R, C), np.uint8)
        codes[r, c] = 0b111111
        p = oracle.pack_tc_fp6(codes).reshape(-1)
        plane2, plane4 = p[: R * C // 4], p[R * C // 4:]
        assert np.count_nonzero(plane2) == 1 and np.count_nonzero(plane4) == 1
        assert bin(int(plane2[np.nonzero(plane2)[0][0]])).count("1") == 2
        assert bin(int(plane4[np.nonzero(plane4)[0][0]])).count("1") == 4


def test_quantize_scale_closed_form(oracle):
    """to_scaled_tc_fpx (quant_llm.py:116-130): scale = amax|row| / 28 in fp32, returned as fp16; the
    largest element of each row therefore encodes as +-28; round trip is exact on representable values."""
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((64, 128)) * 0.02).astype(np.float32)
    codes, scale = oracle.fpx_quantize(w, oracle.F32, 3, 2)
    amax = np.abs(w).max(axis=1)
    expect = (amax / np.float32(28.0)).astype(np.float16).view(np.uint16)
    assert np.array_equal(scale, expect)
    idx = np.abs(w).argmax(axis=1)
    assert np.all((codes[np.arange(64), idx] & 31) == 31)
    # exactly representable weights quantize without error (test_quant_llm.py:44-54)
    grid = oracle.fpx_to_f32(np.arange(64, dtype=np.uint8), 3, 2)
    wexact = grid[rng.integers(0, 64, (64, 64))]
    wexact[:, 0] = 28.0  # pins the row scale to 1
    c2, s2 = oracle.fpx_quantize(wexact, oracle.F32, 3, 2)
    assert np.all(s2 == np.float16(1.0).view(np.uint16))
    assert np.array_equal(oracle.fpx_to_f32(c2, 3, 2), wexact)


def test_fpx_linear_against_float64(oracle):
    rng = np.random.default_rng(9)
    codes = rng.integers(0, 64, (64, 128), dtype=np.uint8)
    scale = (rng.random(64) * 0.01 + 0.001).astype(np.float16)
    x = (rng.standard_normal((2, 128))).astype(np.float16)
    y = oracle.fpx_linear(x.view(np.uint16), codes, scale.view(np.uint16), 3, 2)
    w = (oracle.fpx_to_f32(codes, 3, 2) * scale.astype(np.float32)[:, None]).astype(np.float16)
    ref = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.max(np.abs(y - ref)) <= 1e-5 * max(1.0, np.max(np.abs(ref)))
