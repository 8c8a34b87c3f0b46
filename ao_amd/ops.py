"""Operator layer: torch.library ops in the `torchao` namespace backed by the gfx950 HIP kernels.

Mirrors torchao/ops.py (python wrapper + fake impl per op, reference lines 15-55) and the schema
registration of torchao/csrc/fp6_llm.cpp:5-8.  The device implementations call the C ABI of
include/ao_amd.h with raw pointers on torch's current stream; there is no CPU implementation:
a CPU tensor raises.
"""
import torch
from torch import Tensor

from . import _lib
from ._lib import BF16, DTYPE_CODE, F32, check, current_stream, lib, require_cuda

__all__ = [
    "int4wo_quantize_pack",
    "int4wo_pack",
    "int4wo_unpack",
    "int4wo_dequantize",
    "int4wo_linear",
    "int4wo_packed_shapes",
]

_LIB = torch.library.Library("torchao", "FRAGMENT")
_LIB.define("int4wo_quantize_pack(Tensor w, int group_size) -> (Tensor, Tensor)")
_LIB.define("int4wo_pack(Tensor codes, Tensor scale, Tensor zero_point, int group_size) -> (Tensor, Tensor)")
_LIB.define("int4wo_unpack(Tensor packed, Tensor qparams, int N, int K, int group_size) -> (Tensor, Tensor, Tensor)")
_LIB.define("int4wo_dequantize(Tensor packed, Tensor qparams, int N, int K, int group_size) -> Tensor")
_LIB.define("int4wo_linear(Tensor x, Tensor packed, Tensor qparams, int group_size, int N, Tensor? bias, bool fp32_out) -> Tensor")


def int4wo_packed_shapes(N: int, K: int, group_size: int):
    """Tensor shapes (int32) of the packed codes and of the interleaved (scale, zero) words."""
    if group_size not in (32, 64, 128, 256):
        raise ValueError(f"group_size must be one of 32, 64, 128, 256, got {group_size}")
    Np = (N + 15) // 16 * 16
    kq = max(128, group_size)
    Kp = (K + kq - 1) // kq * kq
    return (Np // 16, Kp // 128, 64, 4), (Np // 16, Kp // group_size, 16)


# ------------------------------------------------------------------------------------ device impls

def _quantize_pack_cuda(w: Tensor, group_size: int):
    require_cuda(w)
    torch._check(w.dim() == 2, lambda: f"weight should be a 2d tensor, got {w.dim()}D")
    torch._check(w.dtype is torch.bfloat16, lambda: f"int4 weight-only quantization needs a bfloat16 weight, got {w.dtype}")
    if w.stride(1) != 1:
        w = w.contiguous()
    N, K = w.shape
    pshape, qshape = int4wo_packed_shapes(N, K, group_size)
    packed = torch.empty(pshape, dtype=torch.int32, device=w.device)
    qparams = torch.empty(qshape, dtype=torch.int32, device=w.device)
    check(lib().ao_amd_int4wo_quantize_pack(w.data_ptr(), N, K, w.stride(0), group_size, packed.data_ptr(),
                                            qparams.data_ptr(), current_stream(w.device)))
    return packed, qparams


def _pack_cuda(codes: Tensor, scale: Tensor, zero_point: Tensor, group_size: int):
    require_cuda(codes, scale, zero_point)
    torch._check(codes.dim() == 2, lambda: f"codes should be a 2d tensor, got {codes.dim()}D")
    N, K = codes.shape
    torch._check(K % group_size == 0, lambda: f"in_features {K} not divisible by group_size {group_size}")
    torch._check(scale.dtype is torch.bfloat16 and zero_point.dtype is torch.bfloat16,
                 lambda: f"scales and zeros must be bfloat16, got {scale.dtype} and {zero_point.dtype}")
    torch._check(scale.numel() == N * (K // group_size) and zero_point.numel() == scale.numel(),
                 lambda: "scale / zero_point size does not match codes and group_size")
    codes = codes.to(torch.int32).contiguous()
    scale = scale.contiguous()
    zero_point = zero_point.contiguous()
    pshape, qshape = int4wo_packed_shapes(N, K, group_size)
    packed = torch.empty(pshape, dtype=torch.int32, device=codes.device)
    qparams = torch.empty(qshape, dtype=torch.int32, device=codes.device)
    check(lib().ao_amd_int4wo_pack(codes.data_ptr(), scale.data_ptr(), zero_point.data_ptr(), N, K, group_size,
                                   packed.data_ptr(), qparams.data_ptr(), current_stream(codes.device)))
    return packed, qparams


def _check_packed(packed: Tensor, qparams: Tensor, N: int, K: int, group_size: int):
    pshape, qshape = int4wo_packed_shapes(N, K, group_size)
    torch._check(tuple(packed.shape) == pshape and packed.dtype is torch.int32 and packed.is_contiguous(),
                 lambda: f"packed weight must be a contiguous int32 tensor of shape {pshape}, got {packed.dtype} {tuple(packed.shape)}")
    torch._check(tuple(qparams.shape) == qshape and qparams.dtype is torch.int32 and qparams.is_contiguous(),
                 lambda: f"qparams must be a contiguous int32 tensor of shape {qshape}, got {qparams.dtype} {tuple(qparams.shape)}")


def _unpack_cuda(packed: Tensor, qparams: Tensor, N: int, K: int, group_size: int):
    require_cuda(packed, qparams)
    _check_packed(packed, qparams, N, K, group_size)
    torch._check(K % group_size == 0, lambda: f"in_features {K} not divisible by group_size {group_size}")
    codes = torch.empty((N, K), dtype=torch.int32, device=packed.device)
    scale = torch.empty((N, K // group_size), dtype=torch.bfloat16, device=packed.device)
    zero = torch.empty_like(scale)
    check(lib().ao_amd_int4wo_unpack(packed.data_ptr(), qparams.data_ptr(), N, K, group_size, codes.data_ptr(),
                                     scale.data_ptr(), zero.data_ptr(), current_stream(packed.device)))
    return codes, scale, zero


def _dequantize_cuda(packed: Tensor, qparams: Tensor, N: int, K: int, group_size: int):
    require_cuda(packed, qparams)
    _check_packed(packed, qparams, N, K, group_size)
    out = torch.empty((N, K), dtype=torch.bfloat16, device=packed.device)
    check(lib().ao_amd_int4wo_dequantize(packed.data_ptr(), qparams.data_ptr(), N, K, group_size, out.data_ptr(),
                                         current_stream(packed.device)))
    return out


def _linear_cuda(x: Tensor, packed: Tensor, qparams: Tensor, group_size: int, N: int, bias, fp32_out: bool):
    require_cuda(x, packed, qparams, bias)
    torch._check(x.dim() == 2, lambda: f"input should be a 2d tensor, got {x.dim()}D")
    torch._check(x.dtype is torch.bfloat16, lambda: f"input must be bfloat16, got {x.dtype}")
    M, K = x.shape
    _check_packed(packed, qparams, N, K, group_size)
    if x.stride(1) != 1:
        x = x.contiguous()
    if bias is not None:
        torch._check(bias.dtype is torch.bfloat16 and bias.numel() == N, lambda: "bias must be bfloat16 of size N")
        bias = bias.contiguous()
    y = torch.empty((M, N), dtype=torch.float32 if fp32_out else torch.bfloat16, device=x.device)
    check(lib().ao_amd_int4wo_linear(x.data_ptr(), M, K, x.stride(0) if M > 0 else K, packed.data_ptr(),
                                     qparams.data_ptr(), N, group_size, None if bias is None else bias.data_ptr(),
                                     y.data_ptr(), F32 if fp32_out else BF16, N, current_stream(x.device)))
    return y


_LIB.impl("int4wo_quantize_pack", _quantize_pack_cuda, "CUDA")
_LIB.impl("int4wo_pack", _pack_cuda, "CUDA")
_LIB.impl("int4wo_unpack", _unpack_cuda, "CUDA")
_LIB.impl("int4wo_dequantize", _dequantize_cuda, "CUDA")
_LIB.impl("int4wo_linear", _linear_cuda, "CUDA")


def _no_cpu(name):
    def impl(*args, **kwargs):
        raise _lib.AoAmdError(f"torchao::{name} has no CPU implementation: ao_amd runs on the GPU only")
    return impl


for _name in ("int4wo_quantize_pack", "int4wo_pack", "int4wo_unpack", "int4wo_dequantize", "int4wo_linear"):
    _LIB.impl(_name, _no_cpu(_name), "CPU")


# ------------------------------------------------------------------------------------ fake (meta) impls
# The quantize API is also run on meta-device weights when a checkpoint is loaded into a model skeleton
# (reference test/integration/test_integration.py:987-997), so every op propagates shapes without data.

@torch.library.register_fake("torchao::int4wo_quantize_pack")
def _(w, group_size):
    torch._check(w.dim() == 2, lambda: f"weight should be a 2d tensor, got {w.dim()}D")
    pshape, qshape = int4wo_packed_shapes(w.shape[0], w.shape[1], group_size)
    return w.new_empty(pshape, dtype=torch.int32), w.new_empty(qshape, dtype=torch.int32)


@torch.library.register_fake("torchao::int4wo_pack")
def _(codes, scale, zero_point, group_size):
    pshape, qshape = int4wo_packed_shapes(codes.shape[0], codes.shape[1], group_size)
    return codes.new_empty(pshape, dtype=torch.int32), codes.new_empty(qshape, dtype=torch.int32)


@torch.library.register_fake("torchao::int4wo_unpack")
def _(packed, qparams, N, K, group_size):
    return (packed.new_empty((N, K), dtype=torch.int32),
            packed.new_empty((N, K // group_size), dtype=torch.bfloat16),
            packed.new_empty((N, K // group_size), dtype=torch.bfloat16))


@torch.library.register_fake("torchao::int4wo_dequantize")
def _(packed, qparams, N, K, group_size):
    return packed.new_empty((N, K), dtype=torch.bfloat16)


@torch.library.register_fake("torchao::int4wo_linear")
def _(x, packed, qparams, group_size, N, bias, fp32_out):
    torch._check(x.dim() == 2, lambda: f"input should be a 2d tensor, got {x.dim()}D")
    torch._check(x.dtype is torch.bfloat16, lambda: f"input must be bfloat16, got {x.dtype}")
    return x.new_empty((x.shape[0], N), dtype=torch.float32 if fp32_out else torch.bfloat16)


# ------------------------------------------------------------------------------------ python wrappers

def int4wo_quantize_pack(w: Tensor, group_size: int):
    """Fused choose_qparams + quantize + pack of a bf16 weight [N,K] -> (packed int32, qparams int32)."""
    return torch.ops.torchao.int4wo_quantize_pack.default(w, group_size)


def int4wo_pack(codes: Tensor, scale: Tensor, zero_point: Tensor, group_size: int):
    """Plain (codes int32 [N,K], scale / zero bf16 [N,K/g]) -> packed layout."""
    return torch.ops.torchao.int4wo_pack.default(codes, scale, zero_point, group_size)


def int4wo_unpack(packed: Tensor, qparams: Tensor, N: int, K: int, group_size: int):
    """Inverse of int4wo_pack."""
    return torch.ops.torchao.int4wo_unpack.default(packed, qparams, N, K, group_size)


def int4wo_dequantize(packed: Tensor, qparams: Tensor, N: int, K: int, group_size: int) -> Tensor:
    """bf16 [N,K] = dequantize_affine of the packed weight."""
    return torch.ops.torchao.int4wo_dequantize.default(packed, qparams, N, K, group_size)


def int4wo_linear(x: Tensor, packed: Tensor, qparams: Tensor, group_size: int, N: int, bias=None,
                  fp32_out: bool = False) -> Tensor:
    """x [M,K] bf16 @ dequant(W)[N,K]^T (+bias) -> [M,N] bf16 (fp32 when fp32_out)."""
    return torch.ops.torchao.int4wo_linear.default(x, packed, qparams, group_size, N, bias, fp32_out)
