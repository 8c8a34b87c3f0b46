"""torch.library.opcheck of the registered operators, as the reference runs it on its own operator
(test/test_ops.py:35-45: test_schema, test_autograd_registration, test_faketensor, test_aot_dispatch_dynamic): the schema
matches what the implementation does to its arguments, the fake (meta) implementation returns the shapes, dtypes and
strides of the real one, and the operator traces under AOT dispatch with dynamic shapes."""
import pytest
import torch

_UTILS = ["test_schema", "test_autograd_registration", "test_faketensor", "test_aot_dispatch_dynamic"]


@pytest.mark.gpu
@pytest.mark.parametrize("ebits,mbits", [(3, 2), (2, 2)])
def test_opcheck_quant_llm_linear(ebits, mbits):
    from ao_amd import ops

    print(f"case opcheck quant_llm_linear e{ebits}m{mbits}", flush=True)
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    BS, OC, IC = 2, 256, 256   # the reference's case
    w = (torch.randn(OC, IC, device=dev) * 0.05).half()
    fpx, scale = ops.fp6_quantize_pack(w, ebits, mbits)
    act = (torch.rand(BS, IC, device=dev) + 0.5).half()
    torch.ops.torchao.quant_llm_linear(ebits, mbits, act, fpx, scale, 1)
    torch.library.opcheck(torch.ops.torchao.quant_llm_linear.default, (ebits, mbits, act, fpx, scale, 1), test_utils=_UTILS)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,g", [(1, 512, 1024, 64), (3, 300, 512, 128), (40, 1024, 2048, 32)])
def test_opcheck_int4_operators(M, N, K, g):
    from ao_amd import ops  # noqa: F401  (registers the operators)

    print(f"case opcheck int4 M={M} N={N} K={K} g={g}", flush=True)
    dev = torch.device("cuda:0")
    torch.manual_seed(1)
    w = (torch.randn(N, K, device=dev) * 0.02).bfloat16()
    x = torch.randn(M, K, device=dev).bfloat16()
    b = torch.randn(N, device=dev).bfloat16()
    torch.library.opcheck(torch.ops.torchao.int4wo_quantize_pack.default, (w, g), test_utils=_UTILS)
    packed, qp = torch.ops.torchao.int4wo_quantize_pack(w, g)
    torch.library.opcheck(torch.ops.torchao.int4wo_linear.default, (x, packed, qp, g, N, b, False), test_utils=_UTILS)
    torch.library.opcheck(torch.ops.torchao.int4wo_linear.default, (x, packed, qp, g, N, None, True), test_utils=_UTILS)
    torch.library.opcheck(torch.ops.torchao.int4wo_dequantize.default, (packed, qp, N, K, g), test_utils=_UTILS)
    codes, scale, zero = torch.ops.torchao.int4wo_unpack(packed, qp, N, K, g)
    torch.library.opcheck(torch.ops.torchao.int4wo_pack.default, (codes, scale, zero, g), test_utils=_UTILS)
    r = torch.randn(M, N, device=dev).bfloat16()
    torch.library.opcheck(torch.ops.torchao.int4wo_linear_residual.default, (x, packed, qp, g, N, None, r), test_utils=_UTILS)


@pytest.mark.gpu
def test_opcheck_fp6_pack_operators():
    from ao_amd import ops  # noqa: F401

    print("case opcheck fp6 pack / dequantize / repack", flush=True)
    dev = torch.device("cuda:0")
    torch.manual_seed(2)
    w = (torch.randn(256, 512, device=dev) * 0.05).half()
    torch.library.opcheck(torch.ops.torchao.fp6_quantize_pack.default, (w, 3, 2), test_utils=_UTILS)
    fpx, scale = torch.ops.torchao.fp6_quantize_pack(w, 3, 2)
    torch.library.opcheck(torch.ops.torchao.fp6_dequantize.default, (fpx, scale, 3, 2), test_utils=_UTILS)
    torch.library.opcheck(torch.ops.torchao.fp6_repack.default, (fpx, 6), test_utils=_UTILS)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_opcheck_hqq_operators(dtype):
    from ao_amd import ops  # noqa: F401
    from ao_amd.prototype.hqq import pack_2xint4

    print(f"case opcheck hqq {dtype}", flush=True)
    dev = torch.device("cuda:0")
    torch.manual_seed(3)
    N, K, g = 256, 512, 64
    packed = pack_2xint4(torch.randint(0, 16, (K, N), dtype=torch.uint8)).to(dev)
    s = (torch.rand(K // g, N, device=dev) * 0.02 + 1e-3).to(dtype)
    z = (torch.rand(K // g, N, device=dev) * 6 + 5).to(dtype)
    torch.library.opcheck(torch.ops.torchao.hqq_dequantize.default, (packed, s, z, g), test_utils=_UTILS)
    x = torch.randn(5, K, device=dev).to(dtype)
    torch.library.opcheck(torch.ops.torchao.hqq_mixed_mm_small.default, (x, packed, s, z, g), test_utils=_UTILS)
    torch.library.opcheck(torch.ops.torchao.hqq_mixed_mm_mfma.default, (x, packed, s, z, g, False), test_utils=_UTILS)
    xt = torch.randn(33, N, device=dev).to(dtype)
    torch.library.opcheck(torch.ops.torchao.hqq_mixed_mm_mfma.default, (xt, packed, s, z, g, True), test_utils=_UTILS)
