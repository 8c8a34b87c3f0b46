"""choose_qparams_affine / quantize_affine / dequantize_affine on the GPU against the CPU oracle, bit for bit, over the
dtype, zero-point-domain and block-shape combinations the reference's callers use (quant_api.py:376-405,
test_quant_primitives.py:184-371).  Each kernel has a path that takes eight elements per thread (row blocks whose
length is a multiple of 8) and a generic path (any block): the shapes below reach both."""
import numpy as np
import pytest
import torch

from _util import bits16

pytestmark = pytest.mark.gpu

_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2, torch.int32: 3, torch.int64: 4, torch.int8: 5,
         torch.uint8: 6}


def _to_np(t):
    return bits16(t) if t.dtype in (torch.bfloat16, torch.float16) else t.detach().cpu().contiguous().numpy()


def _weight(N, K, dtype, seed, zero_row=True):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(N, K, generator=g) * 0.05).to(dtype)
    w[0, : min(K, 16)] = 0.0123  # a constant run: the scale falls onto eps
    if N > 2 and zero_row:
        w[2, :] = 0
    w[N - 1, K - 1] = 1.75
    return w


# (N, K, block): 8-per-thread paths for both kernels, groups of 8..512, rows of any length, 2-D and per-tensor blocks,
# long row blocks (one wave per block: whole and partial rounds of 64 and 256 chunks, several blocks per row)
_SHAPES = [
    (64, 256, (1, 64)), (16, 4096, (1, 128)), (33, 512, (1, 512)), (8, 64, (1, 8)), (40, 200, (1, 8)),
    (24, 192, (1, 192)), (17, 64, (1, 64)), (32, 96, (1, 4)), (32, 128, (32, 128)), (16, 64, (4, 16)), (7, 9, (1, 9)),
    (12, 1024, (1, 1024)), (5, 136, (1, 8)), (3, 1032, (1, 24)),
    (6, 4096, (1, 4096)), (5, 2560, (1, 2560)), (4, 1544, (1, 1544)), (2, 12288, (1, 3072)), (9, 14336, (1, 14336)),
]


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("N,K,block", _SHAPES)
def test_tinygemm_flavour_float_zero_point(oracle, N, K, block, in_dtype):
    """The int4 weight-only call: asymmetric, codes 0..15 as int32, zero point in the float domain."""
    from ao_amd.quantization.quant_primitives import (MappingType, ZeroPointDomain, choose_qparams_affine,
                                                      dequantize_affine, quantize_affine)

    print(f"case float-zp N={N} K={K} block={block} {in_dtype}", flush=True)
    w = _weight(N, K, in_dtype, seed=N * 131 + K)
    dc = _CODE[in_dtype]
    s, z = choose_qparams_affine(w.cuda(), MappingType.ASYMMETRIC, block, torch.int32, 0, 15, 1e-6, in_dtype, in_dtype,
                                 preserve_zero=False, zero_point_domain=ZeroPointDomain.FLOAT)
    so, zo = oracle.choose_qparams_affine(_to_np(w), dc, block, 1, 0, 15, eps=1e-6, preserve_zero=False, zp_domain=1)
    assert np.array_equal(_to_np(s).reshape(so.shape), so) and np.array_equal(_to_np(z).reshape(zo.shape), zo)
    q = quantize_affine(w.cuda(), block, s, z, torch.int32, 0, 15, ZeroPointDomain.FLOAT)
    qo = oracle.quantize_affine(_to_np(w), dc, block, so, dc, zo, dc, 0, 15, zp_domain=1, out_dtype=oracle.I32)
    assert q.dtype is torch.int32 and np.array_equal(q.cpu().numpy(), qo)
    dq = dequantize_affine(q, block, s, z, torch.int32, 0, 15, ZeroPointDomain.FLOAT, output_dtype=in_dtype)
    dqo = oracle.dequantize_affine(qo, oracle.I32, block, so, dc, zo, dc, 0, 15, zp_domain=1, out_dtype=dc)
    assert dq.dtype is in_dtype and np.array_equal(_to_np(dq), dqo)


@pytest.mark.parametrize("code_dtype,qmin,qmax", [(torch.int8, -128, 127), (torch.uint8, 0, 255), (torch.int32, -8, 7)])
@pytest.mark.parametrize("mapping", [0, 1])
@pytest.mark.parametrize("N,K,block", _SHAPES)
def test_integer_zero_point(oracle, N, K, block, mapping, code_dtype, qmin, qmax):
    """The int8 weight-only call and its relatives: integer zero point, symmetric or asymmetric."""
    from ao_amd.quantization.quant_primitives import (MappingType, ZeroPointDomain, choose_qparams_affine,
                                                      dequantize_affine, quantize_affine)

    print(f"case int-zp N={N} K={K} block={block} mapping={mapping} {code_dtype}", flush=True)
    in_dtype = torch.bfloat16 if (N + K) % 2 == 0 else torch.float32
    # no all-zero block here: its integer zero point is the cast of 0 / 0 to int64, which the reference leaves to the
    # hardware (INT64_MIN on x86, 0 on GPUs)
    w = _weight(N, K, in_dtype, seed=N * 17 + K + mapping, zero_row=False)
    dc, cc = _CODE[in_dtype], _CODE[code_dtype]
    eps = float(torch.finfo(torch.float32).eps)
    s, z = choose_qparams_affine(w.cuda(), MappingType(mapping), block, code_dtype, qmin, qmax, eps, None, torch.int64)
    so, zo = oracle.choose_qparams_affine(_to_np(w), dc, block, mapping, qmin, qmax, eps=eps, zp_dtype=oracle.I64)
    assert np.array_equal(_to_np(s).reshape(so.shape), so) and np.array_equal(_to_np(z).reshape(zo.shape), zo)
    q = quantize_affine(w.cuda(), block, s, z, code_dtype, qmin, qmax, ZeroPointDomain.INT)
    qo = oracle.quantize_affine(_to_np(w), dc, block, so, dc, zo, oracle.I64, qmin, qmax, zp_domain=0, out_dtype=cc)
    assert q.dtype is code_dtype and np.array_equal(q.cpu().numpy(), qo)
    for out_dtype in (torch.float32, torch.bfloat16):
        dq = dequantize_affine(q, block, s, z, code_dtype, qmin, qmax, ZeroPointDomain.INT, output_dtype=out_dtype)
        dqo = oracle.dequantize_affine(qo, cc, block, so, dc, zo, oracle.I64, qmin, qmax, zp_domain=0,
                                       out_dtype=_CODE[out_dtype])
        assert np.array_equal(_to_np(dq), dqo)


def test_nan_and_offset_views(oracle):
    """A NaN poisons its own block only; an input that starts 2 bytes into an allocation (not 16-byte aligned) and a
    quantize without a zero point give the same bits as the oracle."""
    from ao_amd.quantization.quant_primitives import (MappingType, ZeroPointDomain, choose_qparams_affine,
                                                      dequantize_affine, quantize_affine)

    print("case nan / unaligned", flush=True)
    N, K, block = 8, 256, (1, 64)
    w = _weight(N, K, torch.bfloat16, seed=5)
    w[4, 70] = float("nan")
    s, z = choose_qparams_affine(w.cuda(), MappingType.ASYMMETRIC, block, torch.int32, 0, 15, 1e-6, None, None,
                                 preserve_zero=False, zero_point_domain=ZeroPointDomain.FLOAT)
    so, zo = oracle.choose_qparams_affine(_to_np(w), 1, block, 1, 0, 15, eps=1e-6, preserve_zero=False, zp_domain=1)
    sf = s.float().cpu().reshape(so.shape)
    assert torch.isnan(sf[4, 1]) and int(torch.isnan(sf).sum()) == 1
    ok = ~np.isnan(oracle.bf16_bits_to_f32(so))
    assert np.array_equal(_to_np(s).reshape(so.shape)[ok], so[ok]) and np.array_equal(_to_np(z).reshape(zo.shape)[ok], zo[ok])

    flat = torch.zeros(N * K + 8, dtype=torch.bfloat16, device="cuda")
    view = flat[1:1 + N * K].view(N, K)
    w2 = _weight(N, K, torch.bfloat16, seed=6)
    view.copy_(w2)
    assert view.data_ptr() % 16 != 0 and view.is_contiguous()
    s2, z2 = choose_qparams_affine(view, MappingType.SYMMETRIC, block, torch.int8, -128, 127, 1e-5, None, torch.int64)
    s2o, z2o = oracle.choose_qparams_affine(_to_np(w2), 1, block, 0, -128, 127, eps=1e-5, zp_dtype=oracle.I64)
    assert np.array_equal(_to_np(s2).reshape(s2o.shape), s2o) and np.array_equal(_to_np(z2).reshape(z2o.shape), z2o)
    q2 = quantize_affine(view, block, s2, None, torch.int8, -128, 127, ZeroPointDomain.INT)
    q2o = oracle.quantize_affine(_to_np(w2), 1, block, s2o, 1, None, 0, -128, 127, zp_domain=0, out_dtype=oracle.I8)
    assert np.array_equal(q2.cpu().numpy(), q2o)
    dq2 = dequantize_affine(q2, block, s2, None, torch.int8, -128, 127, ZeroPointDomain.INT, output_dtype=torch.bfloat16)
    dq2o = oracle.dequantize_affine(q2o, oracle.I8, block, s2o, 1, None, 0, -128, 127, zp_domain=0, out_dtype=1)
    assert np.array_equal(_to_np(dq2), dq2o)


@pytest.mark.parametrize("N,K,bK", [(24, 256, 64), (7, 4096, 4096), (5, 2560, 2560), (9, 1024, 128), (6, 200, 8)])
def test_row_stride_larger_than_k_through_the_c_abi(N, K, bK):
    """ao_amd_choose_qparams_affine / ao_amd_quantize_affine on rows that lie `ld` > K elements apart (the columns of a
    wider matrix) give the bits they give on a contiguous copy, for the int4 and the int8 weight-only argument sets."""
    from ao_amd import _lib

    print(f"case row stride N={N} K={K} bK={bK}", flush=True)
    L = _lib.lib()
    st = torch.cuda.current_stream().cuda_stream
    dev = torch.device("cuda:0")
    BF16, I32, I64, I8 = 1, 3, 4, 5
    ld = K + 24
    wide = (torch.randn(N, ld, device=dev) * 0.05).bfloat16()
    view = wide[:, 16:16 + K]
    dense = view.contiguous()
    assert view.data_ptr() % 16 == 0 and view.stride(0) == ld
    eps32 = float(torch.finfo(torch.float32).eps)
    for name, args in (("int4", (1, 0, 15, 1e-6, 0, 1, BF16, BF16)), ("int8", (0, -128, 127, eps32, 1, 0, BF16, I64))):
        mapping, qmin, qmax, eps, preserve_zero, domain, sdt, zdt = args
        zt = torch.bfloat16 if zdt == BF16 else torch.int64
        ct, cdt = (torch.int32, I32) if name == "int4" else (torch.int8, I8)
        got = []
        for src, stride in ((view, ld), (dense, K)):
            s = torch.empty(N, K // bK, dtype=torch.bfloat16, device=dev)
            z = torch.empty(N, K // bK, dtype=zt, device=dev)
            q = torch.empty(N, K, dtype=ct, device=dev)
            _lib.check(L.ao_amd_choose_qparams_affine(src.data_ptr(), BF16, N, K, stride, 1, bK, mapping, qmin, qmax, eps,
                                                      preserve_zero, domain, sdt, zdt, s.data_ptr(), z.data_ptr(), st))
            _lib.check(L.ao_amd_quantize_affine(src.data_ptr(), BF16, N, K, stride, 1, bK, s.data_ptr(), sdt, z.data_ptr(),
                                                zdt, qmin, qmax, domain, q.data_ptr(), cdt, st))
            torch.cuda.synchronize()
            got.append((s.view(torch.int16), z.view(torch.int16) if zdt == BF16 else z, q))
        for a, b in zip(*got):
            assert torch.equal(a, b), (name, N, K, bK)
