"""Regression against the vectors under tests/golden/ (written by tests/golden/make_fixtures.py from the pinned
oracle): the oracle must still give them (CPU), and the HIP kernels must give them bit for bit (GPU; linear outputs
within the path's 1e-3 relative L2)."""
import glob
import os

import numpy as np
import pytest
import torch

from _util import from_bits16, rel_l2

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
INT4 = sorted(glob.glob(os.path.join(GOLDEN, "int4wo_*.npz")))
FPX = sorted(glob.glob(os.path.join(GOLDEN, "fp[56]_*.npz")))
HQQ = sorted(glob.glob(os.path.join(GOLDEN, "hqq_*.npz")))


def _load(path):
    return np.load(path, allow_pickle=False)


def test_fixture_set_is_complete():
    assert len(INT4) == 4 and len(FPX) == 4 and len(HQQ) == 1


@pytest.mark.parametrize("path", INT4, ids=os.path.basename)
def test_oracle_reproduces_int4(oracle, path):
    f = _load(path)
    g = int(f["group"])
    N, K = f["w_bits"].shape
    Np, Kp = oracle.int4wo_padded_shape(N, K, g)
    codes, scale, zero = oracle.int4wo_quantize(f["w_bits"], oracle.BF16, g, Np, Kp)
    assert np.array_equal(codes, f["codes"]) and np.array_equal(scale, f["scale_bits"]) and np.array_equal(zero, f["zero_bits"])
    packed, qparams = oracle.int4wo_pack(codes, scale, zero, g)
    assert np.array_equal(packed, f["packed"]) and np.array_equal(qparams, f["qparams"])
    dq = oracle.dequantize_affine(codes, oracle.I32, (1, g), scale, oracle.BF16, zero, oracle.BF16, 0, 15, 1, oracle.BF16)
    assert np.array_equal(dq[:N, :K], f["dequant_bits"])
    # invariants the reference's tests state (test_quant_primitives.py:42-47, 121-126): codes in range, and the
    # dequantized value within half a step (+ one bf16 rounding) of the weight wherever it was not clipped
    assert codes.min() >= 0 and codes.max() <= 15
    w = oracle.bf16_bits_to_f32(f["w_bits"]).astype(np.float64)
    d = oracle.bf16_bits_to_f32(f["dequant_bits"]).astype(np.float64)
    s = np.repeat(oracle.bf16_bits_to_f32(f["scale_bits"])[:N, : K // g].astype(np.float64), g, axis=1)
    inner = (f["codes"][:N, :K] > 0) & (f["codes"][:N, :K] < 15)
    assert np.all(np.abs(w - d)[inner] <= 0.5 * s[inner] + 2.0 ** -7 * np.abs(w)[inner] + 2.0 ** -7 * 8 * s[inner])


@pytest.mark.parametrize("path", FPX, ids=os.path.basename)
def test_oracle_reproduces_fpx(oracle, path):
    f = _load(path)
    e, m = int(f["ebits"]), int(f["mbits"])
    codes, scale = oracle.fpx_quantize(f["w_bits"], oracle.F16, e, m)
    assert np.array_equal(codes, f["codes"]) and np.array_equal(scale, f["scale_bits"])
    packed = oracle.pack_tc_fp6(codes) if e + m == 5 else oracle.pack_tc_fpx_generic(codes, 1 + e + m)
    assert np.array_equal(packed, f["packed"])
    assert np.array_equal(oracle.fpx_linear(f["x_bits"], codes, scale, e, m), f["y_f32"])


@pytest.mark.parametrize("path", HQQ, ids=os.path.basename)
def test_oracle_reproduces_hqq(oracle, path):
    f = _load(path)
    for tag, code in (("bf16", oracle.BF16), ("f16", oracle.F16)):
        out = oracle.hqq_dequantize(f["packed"], f[f"scale_{tag}"], f[f"zero_{tag}"], int(f["group"]), code)
        assert np.array_equal(out, f[f"dequant_{tag}"])


# ------------------------------------------------------------------------------------------------ GPU

def _dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


@pytest.mark.gpu
@pytest.mark.parametrize("path", INT4, ids=os.path.basename)
def test_hip_reproduces_int4(path):
    from ao_amd import ops

    f = _load(path)
    g = int(f["group"])
    N, K = f["w_bits"].shape
    dev = _dev()
    w = from_bits16(f["w_bits"]).to(dev)
    packed, qp = ops.int4wo_quantize_pack(w, g)
    assert np.array_equal(packed.cpu().numpy().view(np.uint32), f["packed"])
    assert np.array_equal(qp.cpu().numpy().view(np.uint32), f["qparams"])
    if K % g == 0:
        codes, scale, zero = ops.int4wo_unpack(packed, qp, N, K, g)
        assert np.array_equal(codes.cpu().numpy(), f["codes"][:N, :K].astype(np.int32))
    dq = ops.int4wo_dequantize(packed, qp, N, K, g)
    assert np.array_equal(dq.cpu().view(torch.int16).numpy().view(np.uint16), f["dequant_bits"])
    x = from_bits16(f["x_bits"]).to(dev)
    y = ops.int4wo_linear(x, packed, qp, g, N, None, True).cpu().numpy()
    assert rel_l2(y, f["y_f32"]) <= 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("path", FPX, ids=os.path.basename)
def test_hip_reproduces_fpx(path):
    from ao_amd import ops

    f = _load(path)
    e, m = int(f["ebits"]), int(f["mbits"])
    dev = _dev()
    w = from_bits16(f["w_bits"], torch.float16).to(dev)
    data, scale = ops.fp6_quantize_pack(w, e, m)
    assert np.array_equal(data.cpu().numpy(), f["packed"])
    assert np.array_equal(scale.cpu().view(torch.int16).numpy().view(np.uint16), f["scale_bits"])
    x = from_bits16(f["x_bits"], torch.float16).to(dev)
    y = ops.quant_llm_linear(e, m, x, data, scale, 1).float().cpu().numpy()
    ref = f["y_f32"].astype(np.float16).astype(np.float32)
    assert rel_l2(y, ref) <= 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("path", HQQ, ids=os.path.basename)
def test_hip_reproduces_hqq(path):
    from ao_amd import ops

    f = _load(path)
    dev = _dev()
    packed = torch.from_numpy(f["packed"]).to(dev)
    for tag, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        s = from_bits16(f[f"scale_{tag}"], dt).to(dev)
        z = from_bits16(f[f"zero_{tag}"], dt).to(dev)
        out = ops.hqq_dequantize(packed, s, z, int(f["group"]))
        assert np.array_equal(out.cpu().view(torch.int16).numpy().view(np.uint16), f[f"dequant_{tag}"])
