"""GPU parity tests of the int4 weight-only path: HIP kernels (through the C ABI) vs the CPU oracle.

Quantize / pack / unpack / dequantize: bit-exact.  Linear: relative L2 <= 1e-3 against the
fp32-accumulated dequantize-then-linear oracle (tolerance stated by the task's north star).
"""
import ctypes

import numpy as np
import pytest
import torch

from _util import bits16, from_bits16, make_act, make_weight, rel_l2

pytestmark = pytest.mark.gpu

REL_L2_TOL = 1e-3

SHAPES = [  # (N, K)
    (64, 256),
    (48, 192),    # K padded to the next multiple of max(128, g)
    (17, 64),     # ragged rows, K smaller than one super-slice
    (256, 1024),
    (8, 512),
]
GROUPS = [32, 64, 128, 256]


def _dev():
    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch.device("cuda:0")


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _quantize_pack(cabi, w_dev, g):
    N, K = w_dev.shape
    Np, Kp, pbytes, qbytes = cabi.packed_shape(N, K, g)
    packed = torch.empty(pbytes // 4, dtype=torch.int32, device=w_dev.device)
    qparams = torch.empty(qbytes // 4, dtype=torch.int32, device=w_dev.device)
    cabi.check(cabi.lib().ao_amd_int4wo_quantize_pack(w_dev.data_ptr(), N, K, w_dev.stride(0), g, packed.data_ptr(),
                                                      qparams.data_ptr(), _stream()))
    torch.cuda.synchronize()
    return packed, qparams, Np, Kp


def _oracle_packed(oracle, w, g):
    N, K = w.shape
    Np, Kp = oracle.int4wo_padded_shape(N, K, g)
    codes, scale, zero = oracle.int4wo_quantize(bits16(w), oracle.BF16, g, Np, Kp)
    packed, qparams = oracle.int4wo_pack(codes, scale, zero, g)
    return codes, scale, zero, packed, qparams, Np, Kp


@pytest.mark.parametrize("g", GROUPS)
@pytest.mark.parametrize("shape", SHAPES)
def test_quantize_pack_bit_exact(cabi, oracle, shape, g):
    N, K = shape
    print(f"case quantize_pack N={N} K={K} g={g}", flush=True)
    w = make_weight(N, K, seed=1234 + N + K + g)
    packed, qparams, Np, Kp = _quantize_pack(cabi, w.to(_dev()), g)
    _, _, _, p_ref, q_ref, Np_o, Kp_o = _oracle_packed(oracle, w, g)
    assert (Np, Kp) == (Np_o, Kp_o)
    assert np.array_equal(qparams.cpu().numpy().view(np.uint32).reshape(q_ref.shape), q_ref)
    assert np.array_equal(packed.cpu().numpy().view(np.uint32).reshape(p_ref.shape), p_ref)


def test_quantize_pack_strided_and_config1(cabi, oracle):
    """Config 1 of the baseline: 4096x4096 bf16 ~N(0,0.02), group 128 (bit-exact codes/scales/zeros), plus a
    row-strided view of a larger buffer."""
    print("case quantize_pack config1 4096x4096 g=128", flush=True)
    w = make_weight(4096, 4096, seed=1234, special=False)
    packed, qparams, Np, Kp = _quantize_pack(cabi, w.to(_dev()), 128)
    _, _, _, p_ref, q_ref, _, _ = _oracle_packed(oracle, w, 128)
    assert np.array_equal(qparams.cpu().numpy().view(np.uint32).reshape(q_ref.shape), q_ref)
    assert np.array_equal(packed.cpu().numpy().view(np.uint32).reshape(p_ref.shape), p_ref)

    big = make_weight(64, 640, seed=7)
    view = big[:, 128:384]  # row stride 640, offset keeps 16-byte alignment
    wd = big.to(_dev())[:, 128:384]
    packed, qparams, _, _ = _quantize_pack(cabi, wd, 64)
    _, _, _, p_ref, q_ref, _, _ = _oracle_packed(oracle, view.contiguous(), 64)
    assert np.array_equal(packed.cpu().numpy().view(np.uint32).reshape(p_ref.shape), p_ref)
    assert np.array_equal(qparams.cpu().numpy().view(np.uint32).reshape(q_ref.shape), q_ref)


@pytest.mark.parametrize("g", [32, 128])
@pytest.mark.parametrize("shape", [(48, 256), (17, 128), (64, 1024)])
def test_pack_unpack_dequantize(cabi, oracle, shape, g):
    N, K = shape
    print(f"case pack/unpack N={N} K={K} g={g}", flush=True)
    dev = _dev()
    rng = np.random.default_rng(N * 131 + K + g)
    codes = rng.integers(0, 16, size=(N, K), dtype=np.int32)
    scale = bits16((torch.rand(N, K // g) * 0.01 + 1e-4).bfloat16())
    zero = bits16((torch.randn(N, K // g) * 0.01).bfloat16())
    Np, Kp, pbytes, qbytes = cabi.packed_shape(N, K, g)
    cd = torch.from_numpy(codes).to(dev)
    sd = from_bits16(scale).to(dev)
    zd = from_bits16(zero).to(dev)
    packed = torch.empty(pbytes // 4, dtype=torch.int32, device=dev)
    qparams = torch.empty(qbytes // 4, dtype=torch.int32, device=dev)
    L = cabi.lib()
    cabi.check(L.ao_amd_int4wo_pack(cd.data_ptr(), sd.data_ptr(), zd.data_ptr(), N, K, g, packed.data_ptr(),
                                    qparams.data_ptr(), _stream()))
    # oracle: pad with what quantizing zero padding gives (code 8, scale bf16(1e-6), zero 0)
    cpad = np.full((Np, Kp), 8, np.int32)
    cpad[:N, :K] = codes
    spad = np.full((Np, Kp // g), 0x3586, np.uint16)
    spad[:N, : K // g] = scale
    zpad = np.zeros((Np, Kp // g), np.uint16)
    zpad[:N, : K // g] = zero
    p_ref, q_ref = oracle.int4wo_pack(cpad, spad, zpad, g)
    assert np.array_equal(packed.cpu().numpy().view(np.uint32).reshape(p_ref.shape), p_ref)
    assert np.array_equal(qparams.cpu().numpy().view(np.uint32).reshape(q_ref.shape), q_ref)

    c2 = torch.empty((N, K), dtype=torch.int32, device=dev)
    s2 = torch.empty((N, K // g), dtype=torch.bfloat16, device=dev)
    z2 = torch.empty_like(s2)
    cabi.check(L.ao_amd_int4wo_unpack(packed.data_ptr(), qparams.data_ptr(), N, K, g, c2.data_ptr(), s2.data_ptr(),
                                      z2.data_ptr(), _stream()))
    assert np.array_equal(c2.cpu().numpy(), codes)
    assert np.array_equal(bits16(s2), scale) and np.array_equal(bits16(z2), zero)

    out = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
    cabi.check(L.ao_amd_int4wo_dequantize(packed.data_ptr(), qparams.data_ptr(), N, K, g, out.data_ptr(), _stream()))
    dq_ref = oracle.dequantize_affine(codes, oracle.I32, (1, g), scale, oracle.BF16, zero, oracle.BF16, 0, 15, 1,
                                      oracle.BF16)
    assert np.array_equal(bits16(out), dq_ref)


def _linear(cabi, x_dev, packed, qparams, N, g, bias=None, fp32=True):
    M, K = x_dev.shape
    y = torch.empty((M, N), dtype=torch.float32 if fp32 else torch.bfloat16, device=x_dev.device)
    cabi.check(cabi.lib().ao_amd_int4wo_linear(x_dev.data_ptr(), M, K, x_dev.stride(0), packed.data_ptr(),
                                               qparams.data_ptr(), N, g, None if bias is None else bias.data_ptr(),
                                               y.data_ptr(), cabi.F32 if fp32 else cabi.BF16, N, _stream()))
    torch.cuda.synchronize()
    return y


def _oracle_linear(oracle, w, x, g, bias=None):
    """dequantize-then-linear with fp32 accumulation.  The weight is zero-extended to the packed
    shape before quantization (as from_float pads it), then the logical [N,K] part is used."""
    N, K = w.shape
    Np, Kp = oracle.int4wo_padded_shape(N, K, g)
    codes, scale, zero = oracle.int4wo_quantize(bits16(w), oracle.BF16, g, Np, Kp)
    dq = oracle.dequantize_affine(codes, oracle.I32, (1, g), scale, oracle.BF16, zero, oracle.BF16, 0, 15, 1, oracle.BF16)
    dq = np.ascontiguousarray(dq[:N, :K])
    return dq, oracle.linear(bits16(x), oracle.BF16, dq, oracle.BF16, None if bias is None else bits16(bias),
                             None if bias is None else oracle.BF16)


@pytest.mark.parametrize("g", GROUPS)
def test_linear_one_hot_is_exact_dequant(cabi, oracle, g):
    """With one-hot activation rows the linear returns single dequantized weights, so its in-register
    dequantization can be compared bit for bit with dequantize_affine."""
    N, K = 64, 512
    print(f"case linear one-hot g={g}", flush=True)
    w = make_weight(N, K, seed=99 + g)
    packed, qparams, _, _ = _quantize_pack(cabi, w.to(_dev()), g)
    ks = [0, 1, 7, 8, 31, 32, 33, 63, 64, 127, 128, 255, 256, 300, 510, 511, 200, 77]
    ks += [(37 * i + 5) % K for i in range(70 - len(ks))]
    x = torch.zeros(len(ks), K, dtype=torch.bfloat16)
    for m, k in enumerate(ks):
        x[m, k] = 1.0
    dq, _ = _oracle_linear(oracle, w, x, g)
    dqf = oracle.bf16_bits_to_f32(dq)
    # 70 rows run on the tiled GEMM kernel, 18 on the streaming kernel in two chunks, 16 and 1 on the decode kernel:
    # each has its own dequantization code
    for rows in (len(ks), 18, 16, 1):
        y = _linear(cabi, x[:rows].contiguous().to(_dev()), packed, qparams, N, g, fp32=True).cpu().numpy()
        for m, k in enumerate(ks[:rows]):
            assert np.array_equal(y[m], dqf[:, k]), (rows, m, k)


@pytest.mark.parametrize("M", [1, 4, 16, 33])
@pytest.mark.parametrize("g", [64, 128])
@pytest.mark.parametrize("shape", [(256, 1024), (48, 192), (1024, 4096)])
def test_linear_matches_oracle(cabi, oracle, shape, g, M):
    N, K = shape
    print(f"case linear N={N} K={K} g={g} M={M}", flush=True)
    w = make_weight(N, K, seed=5 + N + g)
    x = make_act(M, K, seed=M + K)
    bias = (torch.randn(N) * 0.1).bfloat16() if M == 4 else None
    dev = _dev()
    packed, qparams, _, _ = _quantize_pack(cabi, w.to(dev), g)
    _, y_ref = _oracle_linear(oracle, w, x, g, bias)
    bd = None if bias is None else bias.to(dev)
    y32 = _linear(cabi, x.to(dev), packed, qparams, N, g, bias=bd, fp32=True).cpu().numpy()
    err = rel_l2(y32, y_ref)
    print(f"  rel_l2 fp32-out = {err:.3e}", flush=True)
    assert err <= REL_L2_TOL
    # bf16 output (what F.linear returns): compare with the oracle rounded to bf16 the same way
    y16 = _linear(cabi, x.to(dev), packed, qparams, N, g, bias=bd, fp32=False)
    y_ref16 = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(y_ref))
    err16 = rel_l2(y16.float().cpu().numpy(), y_ref16)
    print(f"  rel_l2 bf16-out vs bf16(oracle) = {err16:.3e}", flush=True)
    assert err16 <= REL_L2_TOL


@pytest.mark.parametrize("g", [32, 64, 128, 256])
@pytest.mark.parametrize("case", [(272, 1024, 200), (128, 512, 128), (1040, 2048, 333), (100, 256, 17)])
def test_linear_gemm_path(cabi, oracle, case, g):
    """M > 16 goes through the LDS-tiled GEMM kernel: ragged N (not a multiple of 128 or 16), ragged M, bias."""
    N, K, M = case
    print(f"case gemm N={N} K={K} M={M} g={g}", flush=True)
    w = make_weight(N, K, seed=77 + N + g)
    x = make_act(M, K, seed=M + K + 1)
    bias = (torch.randn(N) * 0.1).bfloat16()
    dev = _dev()
    packed, qparams, _, _ = _quantize_pack(cabi, w.to(dev), g)
    _, y_ref = _oracle_linear(oracle, w, x, g, bias)
    y32 = _linear(cabi, x.to(dev), packed, qparams, N, g, bias=bias.to(dev), fp32=True).cpu().numpy()
    err = rel_l2(y32, y_ref)
    print(f"  rel_l2 fp32-out = {err:.3e}", flush=True)
    assert err <= REL_L2_TOL
    y16 = _linear(cabi, x.to(dev), packed, qparams, N, g, bias=bias.to(dev), fp32=False)
    y_ref16 = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(y_ref))
    assert rel_l2(y16.float().cpu().numpy(), y_ref16) <= REL_L2_TOL


@pytest.mark.parametrize("case", [(272, 1024, 512, 64, True), (1040, 2048, 700, 128, False), (48, 192, 600, 32, True)])
def test_linear_op_prefill_two_pass(oracle, case, monkeypatch):
    """From 4096 activation rows on the op dequantizes the weight once (tiled HIP kernel, bit-exact
    against the oracle's dequantize_affine) and calls the library bf16 GEMM: same tolerance against the oracle as
    the fused kernel, and close to the fused kernel's own result."""
    from ao_amd import ops

    N, K, M, g, with_bias = case
    print(f"case two-pass N={N} K={K} M={M} g={g}", flush=True)
    dev = _dev()
    w = make_weight(N, K, seed=88 + N + g)
    x = make_act(M, K, seed=M + K + 2)
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(3)) * 0.1).bfloat16() if with_bias else None
    bias_d = None if bias is None else bias.to(dev)
    packed, qp = ops.int4wo_quantize_pack(w.to(dev), g)
    dq = ops.int4wo_dequantize(packed, qp, N, K, g)
    Np, Kp = oracle.int4wo_padded_shape(N, K, g)
    codes, scale, zero = oracle.int4wo_quantize(bits16(w), oracle.BF16, g, Np, Kp)
    dq_ref = oracle.dequantize_affine(codes, oracle.I32, (1, g), scale, oracle.BF16, zero, oracle.BF16, 0, 15, 1, oracle.BF16)
    assert np.array_equal(bits16(dq), dq_ref[:N, :K])
    monkeypatch.setattr(ops, "TWO_PASS_MIN_M", 1)  # these small weights would otherwise stay on the fused kernel
    assert ops.int4wo_two_pass(M, N, K)
    y = ops.int4wo_linear(x.to(dev), packed, qp, g, N, bias_d)
    monkeypatch.setattr(ops, "TWO_PASS_MIN_M", 1 << 30)
    assert not ops.int4wo_two_pass(M, N, K)
    y_fused = ops.int4wo_linear(x.to(dev), packed, qp, g, N, bias_d)
    assert y.dtype is torch.bfloat16 and y.shape == (M, N)
    _, y_ref = _oracle_linear(oracle, w, x, g, bias)
    y_ref16 = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(y_ref))
    assert rel_l2(y.float().cpu().numpy(), y_ref16) <= REL_L2_TOL
    assert rel_l2(y.float().cpu().numpy(), y_fused.float().cpu().numpy()) <= REL_L2_TOL


def test_two_pass_rule():
    from ao_amd import ops

    assert ops.int4wo_two_pass(4096, 14336, 4096) and ops.int4wo_two_pass(4096, 4096, 14336)
    assert not ops.int4wo_two_pass(2048, 14336, 4096) and not ops.int4wo_two_pass(2048, 128256, 4096)
    assert not ops.int4wo_two_pass(4096, 1024, 4096) and ops.int4wo_two_pass(8192, 1024, 4096)


def test_linear_rejects_bad_arguments(cabi):
    dev = _dev()
    x = torch.zeros(1, 128, dtype=torch.bfloat16, device=dev)
    buf = torch.zeros(4096, dtype=torch.int32, device=dev)
    y = torch.zeros(1, 16, dtype=torch.bfloat16, device=dev)
    L = cabi.lib()
    rc = L.ao_amd_int4wo_linear(x.data_ptr(), 1, 128, 128, buf.data_ptr(), buf.data_ptr(), 16, 48, None, y.data_ptr(),
                                cabi.BF16, 16, _stream())
    assert rc != 0 and b"group_size" in L.ao_amd_last_error()
    rc = L.ao_amd_int4wo_linear(x.data_ptr(), 1, 128, 64, buf.data_ptr(), buf.data_ptr(), 16, 64, None, y.data_ptr(),
                                cabi.BF16, 16, _stream())
    assert rc != 0 and b"stride" in L.ao_amd_last_error()
    rc = L.ao_amd_int4wo_linear(None, 1, 128, 128, buf.data_ptr(), buf.data_ptr(), 16, 64, None, y.data_ptr(),
                                cabi.BF16, 16, _stream())
    assert rc != 0 and b"null" in L.ao_amd_last_error()
