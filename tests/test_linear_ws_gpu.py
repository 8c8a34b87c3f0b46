"""ao_amd_int4wo_linear_ws: the int4 linear with a caller-owned workspace, which splits K over workgroups where the tiles
of 17-256 rows leave most CUs idle (same product as ao_amd_int4wo_linear, `aten::_weight_int4pack_mm` as called from
torchao/dtypes/affine_quantized_tensor.py:600-640, summed in another order).  Checked through the C ABI: against the
fp32-accumulated product with the dequantized weight (<= 1e-3 relative L2 after the bf16 rounding, 2e-5 for fp32 output),
one-hot rows bit for bit against ao_amd_int4wo_dequantize, and against the plain entry point."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _setup(N, K, g, seed):
    from ao_amd import ops
    dev = torch.device("cuda:0")
    w = (torch.randn(N, K, generator=torch.Generator().manual_seed(seed)) * 0.02).bfloat16().to(dev)
    packed, qp = ops.int4wo_quantize_pack(w, g)
    dq = ops.int4wo_dequantize(packed, qp, N, K, g)
    return packed, qp, dq


def _ws_call(x, packed, qp, N, g, bias, fp32, ws_bytes_override=None):
    from ao_amd import _lib
    L = _lib.lib()
    M, K = x.shape
    need = ctypes.c_int64(-1)
    _lib.check(L.ao_amd_int4wo_linear_ws_bytes(M, K, N, g, ctypes.byref(need)))
    nbytes = need.value if ws_bytes_override is None else ws_bytes_override
    ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=x.device)
    y = torch.empty(M, N, dtype=torch.float32 if fp32 else torch.bfloat16, device=x.device)
    rc = L.ao_amd_int4wo_linear_ws(x.data_ptr(), M, K, x.stride(0), packed.data_ptr(), qp.data_ptr(), N, g,
                                   None if bias is None else bias.data_ptr(), y.data_ptr(), _lib.F32 if fp32 else _lib.BF16, N,
                                   ws.data_ptr() if nbytes else None, nbytes, torch.cuda.current_stream().cuda_stream)
    return rc, y, need.value


# (N, K, g, M, parts the rule gives)
CASES = [
    (4096, 14336, 64, 16, 4), (4096, 14336, 64, 24, 4), (4096, 14336, 64, 32, 4), (4096, 14336, 64, 64, 4),
    (4096, 14336, 64, 100, 2), (4096, 14336, 64, 128, 2), (4096, 14336, 64, 8, 1), (4096, 14336, 64, 256, 1),
    (4096, 4096, 128, 32, 4), (4096, 4096, 128, 64, 4), (4096, 4096, 128, 128, 1), (4096, 4096, 128, 16, 1),
    (6144, 4096, 32, 32, 2), (6144, 4096, 32, 16, 1), (6144, 4096, 32, 64, 1),
    (1024, 4096, 256, 128, 4), (1024, 4096, 256, 256, 4), (1024, 4096, 256, 64, 1),
    (14336, 4096, 64, 32, 1), (4100, 8192, 64, 40, 2), (4099, 8192, 64, 40, 2),
]


@pytest.mark.parametrize("N,K,g,M,parts", CASES)
def test_workspace_linear_matches_the_plain_one_and_the_fp32_product(N, K, g, M, parts):
    from ao_amd import _lib
    print(f"case int4wo_linear_ws N={N} K={K} g={g} M={M} parts={parts}", flush=True)
    L = _lib.lib()
    dev = torch.device("cuda:0")
    assert L.ao_amd_int4wo_linear_ws_parts(M, K, N, g) == parts
    packed, qp, dq = _setup(N, K, g, seed=N + K + g)
    gen = torch.Generator().manual_seed(M)
    x = torch.randn(M, K, generator=gen).bfloat16().to(dev)
    bias = torch.randn(N, generator=gen).bfloat16().to(dev)
    for b in (None, bias):
        for fp32 in (False, True):
            rc, y, need = _ws_call(x, packed, qp, N, g, b, fp32)
            assert rc == 0, L.ao_amd_last_error()
            assert need == (parts * M * N * 4 if parts > 1 else 0)
            ref = x.float() @ dq.float().t() + (0 if b is None else b.float())
            if not fp32:
                ref = ref.bfloat16().float()
            err = float((y.float() - ref).norm() / ref.norm())
            assert err <= (2e-5 if fp32 else 1e-3), (err, fp32)
            y0 = torch.empty_like(y)
            _lib.check(L.ao_amd_int4wo_linear(x.data_ptr(), M, K, K, packed.data_ptr(), qp.data_ptr(), N, g,
                                              None if b is None else b.data_ptr(), y0.data_ptr(),
                                              _lib.F32 if fp32 else _lib.BF16, N, torch.cuda.current_stream().cuda_stream))
            if parts == 1 or N % 4:
                same = bool(torch.equal(y, y0))   # no split (N = 4099: partial rows need a multiple of 4): the same launch
                assert same
            else:
                d = float((y.float() - y0.float()).norm() / y0.float().norm())
                assert d <= (2e-5 if fp32 else 1e-3), d
    # one-hot rows read single columns of the dequantized weight back, bit for bit (the other parts add exact zeros)
    ks = torch.randint(0, K, (M,), generator=gen)
    ks[0], ks[-1] = 0, K - 1
    xh = torch.zeros(M, K, dtype=torch.bfloat16)
    xh[torch.arange(M), ks] = 1.0
    rc, yh, _ = _ws_call(xh.to(dev), packed, qp, N, g, None, False)
    assert rc == 0
    exact = bool(torch.equal(yh, dq[:, ks.to(dev)].t().contiguous()))
    assert exact


def test_workspace_linear_refusals_and_fallbacks():
    from ao_amd import _lib, ops
    L = _lib.lib()
    dev = torch.device("cuda:0")
    N, K, g, M = 4096, 8192, 64, 32
    packed, qp, dq = _setup(N, K, g, seed=5)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(6)).bfloat16().to(dev)
    rc, _, need = _ws_call(x, packed, qp, N, g, None, False, ws_bytes_override=1024)
    assert rc != 0 and need == 4 * M * N * 4 and b"workspace" in L.ao_amd_last_error()
    # rows that are not 16-byte aligned: the plain kernels take the call, the workspace is left alone
    xp = torch.zeros(M, K + 3, dtype=torch.bfloat16, device=dev)
    xp[:, :K] = x
    rc, y, _ = _ws_call(xp[:, :K], packed, qp, N, g, None, False)
    assert rc == 0
    ref = (x.float() @ dq.float().t()).bfloat16().float()
    assert float((y.float() - ref).norm() / ref.norm()) <= 1e-3
    # the operator takes the same route: same bits as the C call with a workspace
    rc, y_ws, _ = _ws_call(x, packed, qp, N, g, None, False)
    assert rc == 0 and bool(torch.equal(ops.int4wo_linear(x, packed, qp, g, N), y_ws))


# (N, K, M, parts the rule gives) for ao_amd_fp6_linear_ws
FP6_CASES = [
    (4096, 14336, 16, 4), (4096, 14336, 32, 4), (4096, 14336, 64, 4), (4096, 14336, 100, 2), (4096, 14336, 256, 1),
    (4096, 4096, 32, 4), (4096, 4096, 64, 4), (4096, 4096, 128, 1), (4096, 4096, 16, 1),
    (6144, 4096, 32, 2), (6144, 4096, 64, 1), (1024, 4096, 40, 4), (1024, 4096, 256, 4), (14336, 4096, 32, 1),
    (4096, 8192 + 64, 32, 1),
]


@pytest.mark.parametrize("ebits,mbits", [(3, 2), (2, 3)])
@pytest.mark.parametrize("N,K,M,parts", FP6_CASES)
def test_fp6_workspace_linear(N, K, M, parts, ebits, mbits):
    """ao_amd_fp6_linear_ws (where torchao::quant_llm_linear takes splitK and a [splitK, M, N] workspace,
    torchao/csrc/cuda/fp6_llm/fp6_linear.cu:104-111, 167-168): <= 1e-3 relative L2 of the fp32 product with the dequantized
    weight rounded to fp16, one-hot rows bit for bit, and against the plain entry point.  K = 8256 is not a multiple of
    128: no split."""
    from ao_amd import _lib, ops
    print(f"case fp6_linear_ws N={N} K={K} M={M} parts={parts} e{ebits}m{mbits}", flush=True)
    L = _lib.lib()
    dev = torch.device("cuda:0")
    assert L.ao_amd_fp6_linear_ws_parts(M, K, N) == parts
    gen = torch.Generator().manual_seed(N + K + M)
    w = (torch.randn(N, K, generator=gen) * 0.05).half().to(dev)
    tc, scale = ops.fp6_quantize_pack(w, ebits, mbits)
    native = ops.fp6_repack(tc, 1 + ebits + mbits)
    wd = ops.fp6_dequantize(tc, scale, ebits, mbits).half()      # the kernels multiply fp16(value * scale)
    x = torch.randn(M, K, generator=gen).half().to(dev)
    st = torch.cuda.current_stream().cuda_stream

    def run(xin):
        need = ctypes.c_int64(-1)
        _lib.check(L.ao_amd_fp6_linear_ws_bytes(M, K, N, ctypes.byref(need)))
        assert need.value == (parts * M * N * 4 if parts > 1 else 0)
        ws = torch.empty(max(need.value // 4, 1), dtype=torch.float32, device=dev)
        y = torch.empty(M, N, dtype=torch.float16, device=dev)
        _lib.check(L.ao_amd_fp6_linear_ws(xin.data_ptr(), M, K, native.data_ptr(), scale.data_ptr(), N, ebits, mbits, y.data_ptr(),
                                          ws.data_ptr() if need.value else None, need.value, st))
        return y

    y = run(x)
    ref = (x.float() @ wd.float().t()).half().float()
    err = float((y.float() - ref).norm() / ref.norm())
    assert err <= 1e-3, err
    y0 = torch.empty_like(y)
    _lib.check(L.ao_amd_fp6_linear(x.data_ptr(), M, K, native.data_ptr(), scale.data_ptr(), N, ebits, mbits, y0.data_ptr(), st))
    if parts == 1:
        same = bool(torch.equal(y, y0))
        assert same
    else:
        d = float((y.float() - y0.float()).norm() / y0.float().norm())
        assert d <= 1e-3, d
        # the operator takes the same route
        same = bool(torch.equal(ops.fp6_linear_native(ebits, mbits, x, native, scale), y))
        assert same
    ks = torch.randint(0, K, (M,), generator=gen)
    ks[0], ks[-1] = 0, K - 1
    xh = torch.zeros(M, K, dtype=torch.float16)
    xh[torch.arange(M), ks] = 1.0
    yh = run(xh.to(dev))
    exact = bool(torch.equal(yh, wd[:, ks.to(dev)].t().contiguous()))
    assert exact
