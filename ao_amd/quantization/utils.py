"""tinygemm-flavoured helpers over the affine primitives (torchao/quantization/utils.py:274-392)."""
import torch

from .quant_primitives import (
    MappingType,
    ZeroPointDomain,
    choose_qparams_affine,
    dequantize_affine,
    quantize_affine,
)

__all__ = [
    "compute_error",
    "get_groupwise_affine_qparams",
    "pack_tinygemm_scales_and_zeros",
    "unpack_tinygemm_scales_and_zeros",
    "groupwise_affine_quantize_tensor_from_qparams",
    "groupwise_affine_dequantize_tensor_from_qparams",
    "groupwise_affine_quantize_tensor",
    "groupwise_affine_dequantize_tensor",
    "recommended_inductor_config_setter",
]


def compute_error(x, y):
    """Signal to quantization noise ratio in dB (reference :50-53)."""
    Ps = torch.linalg.norm(x)
    Pn = torch.linalg.norm(x - y)
    return 20 * torch.log10(Ps / Pn)


def guard_dtype_size(tensor_arg, arg_name, dtype=None, size=None):
    if dtype is not None and tensor_arg.dtype != dtype:
        raise ValueError(f"Expected Tensor argument {arg_name} to have dtype {dtype}, but got {tensor_arg.dtype} instead.")
    if size is not None and tensor_arg.size() != size:
        raise ValueError(f"Expected Tensor argument {arg_name} to have size {size}, but got {tensor_arg.size()} instead.")


def get_groupwise_affine_qparams(w, n_bit=4, groupsize=128, dtype=torch.bfloat16):
    """Per-group (scale, zero) of an asymmetric uint`n_bit` quantization, float zero point (reference :274-308)."""
    if groupsize > w.shape[-1]:
        groupsize = w.shape[-1]
    assert groupsize > 1
    assert w.shape[-1] % groupsize == 0
    assert w.dim() == 2
    assert n_bit <= 8, f"only n_bit smaller than 8 is supported, got: {n_bit}"
    scale, zero_point = choose_qparams_affine(
        w, MappingType.ASYMMETRIC, (1, groupsize), torch.int32, 0, 2**n_bit - 1, 1e-6, scale_dtype=dtype,
        zero_point_dtype=dtype, preserve_zero=False, zero_point_domain=ZeroPointDomain.FLOAT)
    return scale.to(dtype=dtype).reshape(w.shape[0], -1), zero_point.to(dtype=dtype).reshape(w.shape[0], -1)


def pack_tinygemm_scales_and_zeros(scales, zeros):
    """[N, K/g] x 2 -> [K/g, N, 2] bf16, the tinygemm interchange form of the qparams (reference :310-322)."""
    guard_dtype_size(scales, "scales", dtype=torch.bfloat16, size=zeros.size())
    guard_dtype_size(zeros, "zeros", dtype=torch.bfloat16)
    return torch.stack([scales, zeros], dim=2).transpose(0, 1).contiguous()


def unpack_tinygemm_scales_and_zeros(scales_and_zeros):
    assert len(scales_and_zeros.shape) == 3 and scales_and_zeros.shape[2] == 2
    return torch.split(scales_and_zeros.transpose(0, 1), 1, 2)


def groupwise_affine_quantize_tensor_from_qparams(w, scales, zeros, n_bit=4, groupsize=128):
    assert groupsize > 1
    if groupsize > w.shape[-1] and scales.shape[-1] == 1:  # GPTQ single-column case
        groupsize = w.shape[-1]
    assert w.shape[-1] % groupsize == 0
    assert w.dim() == 2
    return quantize_affine(w, (1, groupsize), scales, zeros, torch.int32, 0, 2**n_bit - 1,
                           zero_point_domain=ZeroPointDomain.FLOAT)


def groupwise_affine_dequantize_tensor_from_qparams(w_int4x8, scales, zeros, n_bit=4, groupsize=128):
    assert groupsize > 1
    if groupsize > w_int4x8.shape[-1] and scales.shape[-1] == 1:
        groupsize = w_int4x8.shape[-1]
    assert w_int4x8.shape[-1] % groupsize == 0
    assert w_int4x8.dim() == 2
    return dequantize_affine(w_int4x8, (1, groupsize), scales, zeros, torch.int32, 0, 2**n_bit - 1,
                             zero_point_domain=ZeroPointDomain.FLOAT, output_dtype=scales.dtype)


def groupwise_affine_quantize_tensor(w, n_bit=4, groupsize=128, dtype=torch.bfloat16):
    scales, zeros = get_groupwise_affine_qparams(w, n_bit, groupsize, dtype)
    w_int4x8 = groupwise_affine_quantize_tensor_from_qparams(w, scales, zeros, n_bit, groupsize)
    return w_int4x8, pack_tinygemm_scales_and_zeros(scales, zeros)


def groupwise_affine_dequantize_tensor(w_int4x8, scales_and_zeros, n_bit=4, groupsize=128):
    scales, zeros = unpack_tinygemm_scales_and_zeros(scales_and_zeros)
    return groupwise_affine_dequantize_tensor_from_qparams(w_int4x8, scales, zeros, n_bit, groupsize)


def recommended_inductor_config_setter():
    """The reference tunes torch.compile here (:461-476).  This library does not go through inductor:
    kernels are launched directly and decode loops are captured in HIP graphs, so there is nothing to set."""
    return None
