"""GPU parity tests of the int8 weight-only path (symmetric per-channel, plain layout): quantization through the
generic primitives bit-exact against the CPU oracle; the linear against the oracle's fp32-accumulated product with
the reference's rounding chain bf16(bf16(x @ q^T) * scale) (+ bias) applied on top
(torchao/dtypes/affine_quantized_tensor.py:641-665)."""
import numpy as np
import pytest
import torch

from _util import bits16, make_act, make_weight, rel_l2

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def _rb(oracle, a):
    return oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(np.asarray(a, np.float32)))


def _oracle_quant(oracle, w):
    eps = float(torch.finfo(torch.float32).eps)
    N, K = w.shape
    s, z = oracle.choose_qparams_affine(bits16(w), oracle.BF16, (1, K), 0, -128, 127, eps=eps, zp_dtype=oracle.I64)
    q = oracle.quantize_affine(bits16(w), oracle.BF16, (1, K), s, oracle.BF16, z, oracle.I64, -128, 127, zp_domain=0,
                               out_dtype=oracle.I8)
    return q, s, z


@pytest.mark.parametrize("shape", [(64, 256), (48, 192), (17, 64), (256, 1024)])
def test_quantize_bit_exact(oracle, shape):
    from ao_amd.dtypes import AffineQuantizedTensor
    from ao_amd.quantization import int8_weight_only

    N, K = shape
    print(f"case int8 quantize N={N} K={K}", flush=True)
    w = make_weight(N, K, seed=3 * N + K)
    qw = int8_weight_only()(w.to(_dev()))
    assert isinstance(qw, AffineQuantizedTensor) and qw.shape == (N, K) and qw.dtype is torch.bfloat16
    int_data, scale, zero = qw.layout_tensor.get_plain()
    q, s, z = _oracle_quant(oracle, w)
    assert int_data.dtype is torch.int8 and scale.dtype is torch.bfloat16 and zero.dtype is torch.int64
    assert np.array_equal(int_data.cpu().numpy(), q)
    assert np.array_equal(bits16(scale).reshape(-1), s.reshape(-1))
    assert np.array_equal(zero.cpu().numpy().reshape(-1), z.reshape(-1))


@pytest.mark.parametrize("M", [1, 4, 16, 33, 130, 300])  # from 128 rows on the two-pass path is checked as well
@pytest.mark.parametrize("shape", [(256, 1024), (48, 256), (1000, 4096)])
def test_linear_matches_oracle(oracle, shape, M, monkeypatch):
    from ao_amd import ops

    N, K = shape
    print(f"case int8 linear N={N} K={K} M={M}", flush=True)
    dev = _dev()
    w = make_weight(N, K, seed=5 + N)
    x = make_act(M, K, seed=M + K)
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(9)) * 0.1).bfloat16() if M in (4, 130) else None
    q, s, _ = _oracle_quant(oracle, w)
    acc = oracle.linear(bits16(x), oracle.BF16, q, oracle.I8)            # fp32-accumulated x @ q^T
    sf = oracle.bf16_bits_to_f32(s.reshape(1, -1))
    pre = _rb(oracle, acc) * sf                                          # value before the last rounding
    if bias is not None:
        pre = _rb(oracle, pre) + bias.float().numpy().reshape(1, -1)
    expect = _rb(oracle, pre)
    qd = torch.from_numpy(q).to(dev)
    sd = torch.from_numpy(s.reshape(-1).view(np.int16)).view(torch.bfloat16).to(dev)
    bd = None if bias is None else bias.to(dev)
    y32 = ops.int8wo_linear(x.to(dev), qd, sd, bd, True).cpu().numpy()
    y16 = ops.int8wo_linear(x.to(dev), qd, sd, bd, False).float().cpu().numpy()
    # the accumulation order differs from the oracle's: an element whose sum sits on a bf16 rounding boundary may
    # move by one bf16 ulp, everything else is identical
    assert rel_l2(y32, pre) <= 1e-3
    assert rel_l2(y16, expect) <= 1e-3
    assert np.count_nonzero(y16 != expect) <= 0.02 * y16.size + 1
    if M >= ops.INT8_TWO_PASS_MIN_M:
        # large weights take the bf16 copy of the codes + the library GEMM from here on (ops.int8wo_two_pass): same bar
        monkeypatch.setattr(ops, "int8wo_two_pass", lambda M, N, K: True)
        y2p = ops.int8wo_linear(x.to(dev), qd, sd, bd, False).float().cpu().numpy()
        assert rel_l2(y2p, expect) <= 1e-3
        assert np.count_nonzero(y2p != expect) <= 0.02 * y2p.size + 1


def test_one_hot_rows_return_scaled_codes(oracle):
    """x = e_k: the product is the code itself, so the output must be exactly bf16(q[n,k] * scale[n])."""
    from ao_amd import ops

    dev = _dev()
    N, K = 80, 512
    w = make_weight(N, K, seed=123)
    q, s, _ = _oracle_quant(oracle, w)
    ks = [0, 1, 3, 4, 7, 8, 31, 32, 33, 127, 128, 255, 256, 300, 510, 511]
    x = torch.zeros(len(ks), K, dtype=torch.bfloat16)
    for m, k in enumerate(ks):
        x[m, k] = 1.0
    sd = torch.from_numpy(s.reshape(-1).view(np.int16)).view(torch.bfloat16)
    y = ops.int8wo_linear(x.to(dev), torch.from_numpy(q).to(dev), sd.to(dev), None, False).float().cpu().numpy()
    sf = oracle.bf16_bits_to_f32(s.reshape(-1))
    for m, k in enumerate(ks):
        assert np.array_equal(y[m], _rb(oracle, q[:, k].astype(np.float32) * sf)), (m, k)


def test_module_api_and_fallback():
    """quantize_(model, int8_weight_only()) swaps nn.Linear weights; F.linear runs the HIP kernel for bf16
    activations when in_features is a multiple of 128, and the reference's own op sequence (:655-665: the product
    formed in the activation's dtype, times scale, plus bias, cast back) for other activation dtypes and ragged
    in_features."""
    from ao_amd import int8_weight_only, quantize_
    from ao_amd.dtypes import AffineQuantizedTensor

    dev = _dev()
    torch.manual_seed(0)
    for K in (256, 192):
        lin = torch.nn.Linear(K, 96, bias=True).to(dev).bfloat16()
        ref_w = lin.weight.detach().clone()
        x = torch.randn(5, K, device=dev).bfloat16()
        quantize_(lin, int8_weight_only())
        assert isinstance(lin.weight, AffineQuantizedTensor)
        with torch.no_grad():
            y = lin(x)
            y_ref = torch.nn.functional.linear(x, lin.weight.dequantize(), lin.bias)
            y_fp = torch.nn.functional.linear(x, ref_w, lin.bias)
        assert y.shape == (5, 96) and y.dtype is torch.bfloat16
        assert rel_l2(y.float().cpu().numpy(), y_ref.float().cpu().numpy()) <= 1e-2   # two bf16 rounding chains
        assert rel_l2(y.float().cpu().numpy(), y_fp.float().cpu().numpy()) <= 3e-2    # 8-bit quantization error
        # fp16 / fp32 activations on the bf16 module (the reference multiplies in the activation's dtype and returns it)
        for dt in (torch.float16, torch.float32):
            xd = torch.randn(2, 3, K, device=dev, dtype=dt)
            with torch.no_grad():
                yd = lin(xd)
                w_t = lin.weight.layout_tensor.int_data.t().to(dt)
                want = (torch.mm(xd.reshape(-1, K), w_t) * lin.weight.layout_tensor.scale).reshape(2, 3, 96)
                want += lin.bias
            assert yd.shape == (2, 3, 96) and yd.dtype is dt
            assert torch.equal(yd, want.to(dt))


def test_rejects_bad_arguments(cabi):
    dev = _dev()
    x = torch.zeros(1, 192, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(16, 192, dtype=torch.int8, device=dev)
    s = torch.ones(16, dtype=torch.bfloat16, device=dev)
    y = torch.zeros(1, 16, dtype=torch.bfloat16, device=dev)
    rc = cabi.lib().ao_amd_int8wo_linear(x.data_ptr(), 1, 192, 192, w.data_ptr(), 192, s.data_ptr(), 16, None, y.data_ptr(),
                                         cabi.BF16, 16, None)
    assert rc != 0 and b"multiple of 128" in cabi.lib().ao_amd_last_error()


@pytest.mark.parametrize("M", [1, 3, 16])
def test_fused_epilogues_match_the_module_chain(M):
    """residual add and SiLU(gate) * up fused into the linear: identical to the separate bf16 ops but for rare
    elements where the device's expf differs from torch's by an ulp."""
    from ao_amd import ops

    dev = _dev()
    N, K = 512, 1024
    gen = torch.Generator().manual_seed(77)
    q = torch.randint(-127, 128, (N, K), generator=gen, dtype=torch.int8).to(dev)
    s = (torch.rand(N, generator=gen) * 1e-3 + 1e-4).bfloat16().to(dev)
    x = make_act(M, K, seed=78).to(dev)
    other = make_act(M, N, seed=79).to(dev)
    y = ops.int8wo_linear(x, q, s)
    assert torch.equal(ops.int8wo_linear_residual(x, q, s, other), other + y)
    got = ops.int8wo_linear_gated(x, q, s, other).float().cpu().numpy()
    want = (torch.nn.functional.silu(other) * y).float().cpu().numpy()
    assert np.count_nonzero(got != want) <= 0.002 * got.size + 1 and rel_l2(got, want) <= 1e-3


@pytest.mark.parametrize("M,N,K", [(1, 512, 1024), (3, 512, 1024), (16, 256, 2048), (1, 6144, 4096), (1, 4096, 14336),
                                   (1, 1000, 4096), (2, 8208, 4096)])
def test_fused_rmsnorm_matches_the_separate_kernels(M, N, K):
    """RMSNorm applied while the activation rows are staged in LDS: the normalized rows are those of the stand-alone
    RMSNorm kernel unless the two sums of squares (different summation orders) round apart, so the linear is compared
    with a tolerance of a few bf16 steps on few elements; with and without the SiLU(gate) epilogue."""
    from ao_amd import ops

    print(f"case int8 fused norm M={M} N={N} K={K}", flush=True)
    dev = _dev()
    gen = torch.Generator().manual_seed(M * 7 + N)
    q = torch.randint(-127, 128, (N, K), generator=gen, dtype=torch.int8).to(dev)
    s = (torch.rand(N, generator=gen) * 1e-3 + 1e-4).bfloat16().to(dev)
    x = (make_act(M, K, seed=80 + M) * 3).to(dev)
    nw = (1 + 0.1 * torch.randn(K, generator=gen)).bfloat16().to(dev)
    gate = make_act(M, N, seed=81).to(dev)
    xn = ops.rmsnorm(x, nw, 1e-5)
    want = ops.int8wo_linear(xn, q, s).float().cpu().numpy()
    got = ops.int8wo_rmsnorm_linear(x, nw, 1e-5, q, s).float().cpu().numpy()
    assert rel_l2(got, want) <= 2e-3 and np.count_nonzero(got != want) <= 0.02 * got.size + 1
    want_g = ops.int8wo_linear_gated(xn, q, s, gate).float().cpu().numpy()
    got_g = ops.int8wo_rmsnorm_linear(x, nw, 1e-5, q, s, gate).float().cpu().numpy()
    assert rel_l2(got_g, want_g) <= 2e-3 and np.count_nonzero(got_g != want_g) <= 0.02 * got_g.size + 1


def test_fused_rmsnorm_rejects_rows_that_do_not_fit_lds():
    from ao_amd import ops
    from ao_amd._lib import AoAmdError

    dev = _dev()
    q = torch.zeros(256, 4096, dtype=torch.int8, device=dev)
    s = torch.ones(256, dtype=torch.bfloat16, device=dev)
    nw = torch.ones(4096, dtype=torch.bfloat16, device=dev)
    with pytest.raises(AoAmdError, match="fit in LDS"):
        ops.int8wo_rmsnorm_linear(torch.zeros(16, 4096, dtype=torch.bfloat16, device=dev), nw, 1e-5, q, s)


@pytest.mark.parametrize("M,N,K", [(1, 512, 1024), (4, 1000, 2048), (1, 14336, 4096), (16, 256, 1024)])
@pytest.mark.parametrize("with_norm", [False, True])
def test_two_weight_swiglu_matches_the_gated_chain(M, N, K, with_norm):
    """One launch over w1 and w3 against linear -> gated linear: every rounding is the same, so equality but for
    elements where the accumulation order of a sum sitting on a bf16 boundary differs (none expected: same order)."""
    from ao_amd import ops

    print(f"case int8 swiglu M={M} N={N} K={K} norm={with_norm}", flush=True)
    dev = _dev()
    gen = torch.Generator().manual_seed(M + N + K)
    qg = torch.randint(-127, 128, (N, K), generator=gen, dtype=torch.int8).to(dev)
    qu = torch.randint(-127, 128, (N, K), generator=gen, dtype=torch.int8).to(dev)
    sg = (torch.rand(N, generator=gen) * 1e-3 + 1e-4).bfloat16().to(dev)
    su = (torch.rand(N, generator=gen) * 1e-3 + 1e-4).bfloat16().to(dev)
    x = (make_act(M, K, seed=90 + M) * 2).to(dev)
    nw = (1 + 0.1 * torch.randn(K, generator=gen)).bfloat16().to(dev) if with_norm else None
    if with_norm:
        gate = ops.int8wo_rmsnorm_linear(x, nw, 1e-5, qg, sg)
        want = ops.int8wo_rmsnorm_linear(x, nw, 1e-5, qu, su, gate)
    else:
        want = ops.int8wo_linear_gated(x, qu, su, ops.int8wo_linear(x, qg, sg))
    got = ops.int8wo_swiglu(x, qg, sg, qu, su, nw, 1e-5)
    assert got.shape == (M, N) and got.dtype is torch.bfloat16
    g, w = got.float().cpu().numpy(), want.float().cpu().numpy()
    assert rel_l2(g, w) <= 1e-3 and np.count_nonzero(g != w) <= 0.01 * g.size + 1


def test_legacy_entry_points_map_to_quantize():
    """change_linear_weights_to_int{4,8}_woqtensors (reference quant_api.py:103-141) compute what quantize_ with the
    matching constructor computes; the int4 one installs the legacy subclass (reference subclass.py:394), the int8 one
    the same tensor class as quantize_."""
    import copy

    from ao_amd import int4_weight_only, int8_weight_only, quantize_
    from ao_amd.quantization import (Int4WeightOnlyQuantizedLinearWeight, change_linear_weights_to_int4_woqtensors,
                                     change_linear_weights_to_int8_woqtensors)

    dev = _dev()
    torch.manual_seed(1)
    base = torch.nn.Sequential(torch.nn.Linear(256, 128, bias=False)).to(dev).bfloat16()
    x = torch.randn(3, 256, device=dev).bfloat16()
    for legacy, modern, cls in ((lambda m: change_linear_weights_to_int4_woqtensors(m, groupsize=64),
                                 lambda m: quantize_(m, int4_weight_only(group_size=64)), Int4WeightOnlyQuantizedLinearWeight),
                                (change_linear_weights_to_int8_woqtensors, lambda m: quantize_(m, int8_weight_only()), None)):
        a, b = copy.deepcopy(base), copy.deepcopy(base)
        legacy(a)
        modern(b)
        same_class = type(a[0].weight) is (type(b[0].weight) if cls is None else cls)
        with torch.no_grad():
            same_output = torch.equal(a(x), b(x))
        assert same_class and same_output


@pytest.mark.parametrize("M,N,K,bias", [(16, 14336, 4096, False), (13, 12352, 1024, True), (40, 16384, 2048, True),
                                        (29, 14336, 1024, False)])
def test_four_row_blocks_per_workgroup_kernel(M, N, K, bias):
    """int8wo_linear_rb4_kernel (activation rows that do not fit the LDS staging, weights with 768 or more 16-row
    blocks: four row blocks per workgroup share the activation loads, two activation blocks from 17 rows on): the linear against an fp32 matmul on the int8
    codes with the module's roundings, one-hot rows bit for bit, and the fused residual / gate epilogues against the
    separate bf16 ops."""
    from ao_amd import ops

    print(f"case int8 rb4 M={M} N={N} K={K} bias={bias}", flush=True)
    dev = _dev()
    gen = torch.Generator().manual_seed(M + N + K)
    q = torch.randint(-127, 128, (N, K), generator=gen, dtype=torch.int8).to(dev)
    s = (torch.rand(N, generator=gen) * 1e-3 + 1e-4).bfloat16().to(dev)
    b = (torch.randn(N, generator=gen) * 0.1).bfloat16().to(dev) if bias else None
    x = make_act(M, K, seed=M + 1).to(dev)
    acc = x.float() @ q.float().t()
    pre = acc.bfloat16().float() * s.float()
    if bias:
        pre = pre.bfloat16().float() + b.float()
    y32 = ops.int8wo_linear(x, q, s, b, True)
    y16 = ops.int8wo_linear(x, q, s, b, False)
    err32 = float((y32 - pre).norm() / pre.norm())
    err16 = float((y16.float() - pre.bfloat16().float()).norm() / pre.norm())
    assert err32 <= 1e-3 and err16 <= 1.5e-3
    # one-hot rows: the codes times the scale, exactly
    ks = torch.randint(0, K, (M,), generator=gen).to(dev)
    xh = torch.zeros(M, K, dtype=torch.bfloat16, device=dev)
    xh[torch.arange(M, device=dev), ks] = 1.0
    yh = ops.int8wo_linear(xh, q, s, None, True)
    exact = bool(torch.equal(yh, q.float().t()[ks] * s.float()))
    assert exact
    other = make_act(M, N, seed=M + 2).to(dev)
    y = ops.int8wo_linear(x, q, s)
    same_residual = bool(torch.equal(ops.int8wo_linear_residual(x, q, s, other), other + y))
    got = ops.int8wo_linear_gated(x, q, s, other).float().cpu().numpy()
    want = (torch.nn.functional.silu(other) * y).float().cpu().numpy()
    assert same_residual and np.count_nonzero(got != want) <= 0.002 * got.size + 1 and rel_l2(got, want) <= 1e-3
