"""Affine quantization primitives on the GPU.

Same names, argument meaning and error behaviour as torchao/quantization/quant_primitives.py
(choose_qparams_affine :278-367, quantize_affine :134-206, dequantize_affine :208-276); the
arithmetic runs in hand-written HIP kernels that reproduce the reference's eager op-by-op rounding
bit for bit.  Tensors must live on the GPU (meta tensors propagate shapes only).
"""
from enum import Enum
from typing import Dict, Optional, Tuple

import torch

from .._lib import DTYPE_CODE, check, current_stream, lib, require_cuda

__all__ = [
    "MappingType",
    "ZeroPointDomain",
    "choose_qparams_affine",
    "quantize_affine",
    "dequantize_affine",
]


class MappingType(Enum):
    """SYMMETRIC maps (-max|x|, max|x|) onto the integer range; ASYMMETRIC maps (min, max)."""
    SYMMETRIC = 0
    ASYMMETRIC = 1


class ZeroPointDomain(Enum):
    """INT: q = round(x / scale) + zp.  FLOAT: q = round((x - (zp - scale * mid)) / scale)."""
    INT = 0
    FLOAT = 1


_DTYPE_TO_QVALUE_BOUNDS: Dict[torch.dtype, Tuple[int, int]] = {
    torch.uint8: (0, 255),
    torch.int8: (-128, 127),
    torch.int16: (-(2**15), 2**15 - 1),
    torch.int32: (-(2**31), 2**31 - 1),
}
for _bits in range(1, 8):
    _DTYPE_TO_QVALUE_BOUNDS[getattr(torch, f"uint{_bits}")] = (0, 2**_bits - 1)

_FLOAT_DTYPES = (torch.float32, torch.float16, torch.bfloat16)


def _get_and_check_qmin_qmax(dtype, quant_min, quant_max):
    """Default quant_min / quant_max from `dtype` and bounds check (reference :73-93)."""
    if dtype not in _DTYPE_TO_QVALUE_BOUNDS:
        raise ValueError(f"Unsupported dtype: {dtype}")
    lo, hi = _DTYPE_TO_QVALUE_BOUNDS[dtype]
    quant_min = lo if quant_min is None else quant_min
    quant_max = hi if quant_max is None else quant_max
    assert quant_min >= lo, f"quant_min out of bound for dtype, quant_min_lower_bound: {lo} quant_min: {quant_min}"
    assert quant_max <= hi, f"quant_max out of bound for dtype, quant_max_upper_bound: {hi} quant_max: {quant_max}"
    return quant_min, quant_max


def _get_reduction_params(block_size, input_size):
    """View shape + reduction dims for a block partition (reference :95-131); used for shape checks and
    to size the qparam tensors exactly as the reference does."""
    assert len(block_size) == len(input_size)
    shape_for_reduction, reduction_dims = [], []
    cur_dim = 0
    for i in range(len(block_size)):
        if block_size[i] != input_size[i] and block_size[i] > 1:
            assert input_size[i] % block_size[i] == 0, (
                f"Expecting input size at {i} dimension: {input_size[i]} to be divisible by block_size at {i} "
                f"dimension: {block_size[i]}")
            shape_for_reduction += [input_size[i] // block_size[i], block_size[i]]
            reduction_dims.append(cur_dim + 1)
            cur_dim += 2
        else:
            shape_for_reduction.append(input_size[i])
            if block_size[i] != 1:
                reduction_dims.append(cur_dim)
            cur_dim += 1
    return shape_for_reduction, reduction_dims


def _qparam_shape(block_size, input_size):
    shape, dims = _get_reduction_params(block_size, input_size)
    return [s for i, s in enumerate(shape) if i not in dims]


def _as_2d_blocks(block_size, shape):
    """Express an n-d block partition as a 2-d tensor [N, K] with block (bN, bK) for the kernels.

    Supported: 2-d inputs with any (bN, bK), and n-d inputs whose blocks are contiguous runs of memory
    (leading block dims 1, then one split dim, then full trailing dims): per tensor, per token / row,
    per channel on axis 0, per group on the last dim."""
    block_size, shape = list(block_size), list(shape)
    if len(shape) == 2:
        return shape[0], shape[1], block_size[0], block_size[1]
    i = 0
    while i < len(shape) and block_size[i] == 1:
        i += 1
    if i == len(shape):  # every element has its own qparams
        n = 1
        for s in shape:
            n *= s
        return n, 1, 1, 1
    if any(block_size[j] != shape[j] for j in range(i + 1, len(shape))):
        raise NotImplementedError(
            f"block_size {tuple(block_size)} on shape {tuple(shape)}: only blocks that are contiguous in memory are "
            "implemented by the HIP kernels")
    lead = 1
    for s in shape[:i]:
        lead *= s
    trail = 1
    for s in shape[i + 1:]:
        trail *= s
    return lead * (shape[i] // block_size[i]), block_size[i] * trail, 1, block_size[i] * trail


def _code(dtype, what):
    if dtype not in DTYPE_CODE:
        raise ValueError(f"Unsupported {what} dtype: {dtype}")
    return DTYPE_CODE[dtype]


def choose_qparams_affine(
    input: torch.Tensor,
    mapping_type: MappingType,
    block_size: Tuple[int, ...],
    target_dtype: torch.dtype,
    quant_min: Optional[int] = None,
    quant_max: Optional[int] = None,
    eps: Optional[float] = None,
    scale_dtype: Optional[torch.dtype] = None,
    zero_point_dtype: Optional[torch.dtype] = None,
    preserve_zero: bool = True,
    zero_point_domain=ZeroPointDomain.INT,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Scale and zero point per block of `block_size` elements (reference :278-367)."""
    quant_min, quant_max = _get_and_check_qmin_qmax(target_dtype, quant_min, quant_max)
    assert mapping_type in [MappingType.SYMMETRIC, MappingType.ASYMMETRIC], f"Unsupported mapping type: {mapping_type}"
    assert input.dtype in _FLOAT_DTYPES, f"Unsupported input dtype: {input.dtype}"
    scale_dtype = input.dtype if scale_dtype is None else scale_dtype
    zero_point_dtype = input.dtype if zero_point_dtype is None else zero_point_dtype
    assert len(block_size) == input.dim()
    out_shape = _qparam_shape(block_size, input.size())
    if mapping_type == MappingType.SYMMETRIC:
        if not preserve_zero:
            raise ValueError("preserve_zero == False is not supported for symmetric quantization")
        if zero_point_domain != ZeroPointDomain.INT:
            raise ValueError("zero_point_domain != ZeroPointDomain.INT is not supported for symmetric quantization")
    elif not preserve_zero:
        assert zero_point_domain == ZeroPointDomain.FLOAT, "if not preserve_zero, zero_point must be in FLOAT domain"
    scale = torch.empty(out_shape, dtype=scale_dtype, device=input.device)
    zero_point = torch.empty(out_shape, dtype=zero_point_dtype, device=input.device)
    if input.is_meta:
        return scale, zero_point
    require_cuda(input)
    x = input.contiguous()
    N, K, bN, bK = _as_2d_blocks(block_size, x.shape)
    check(lib().ao_amd_choose_qparams_affine(
        x.data_ptr(), _code(x.dtype, "input"), N, K, K, bN, bK, mapping_type.value, quant_min, quant_max,
        -1.0 if eps is None else float(eps), int(bool(preserve_zero)), zero_point_domain.value,
        _code(scale_dtype, "scale"), _code(zero_point_dtype, "zero_point"), scale.data_ptr(), zero_point.data_ptr(),
        current_stream(x.device)))
    return scale, zero_point


def _check_qparam(t, name, block_size, input_size):
    expect = 1
    for s in _qparam_shape(block_size, input_size):
        expect *= s
    if t.numel() != expect:
        # same failure class as the reference's scale.view(shape_after_reduction)
        raise RuntimeError(f"shape '{_qparam_shape(block_size, input_size)}' is invalid for input of size {t.numel()} ({name})")


def quantize_affine(
    input: torch.Tensor,
    block_size: Tuple[int, ...],
    scale: torch.Tensor,
    zero_point: Optional[torch.Tensor],
    output_dtype: torch.dtype,
    quant_min: Optional[int] = None,
    quant_max: Optional[int] = None,
    zero_point_domain: ZeroPointDomain = ZeroPointDomain.INT,
) -> torch.Tensor:
    """Float tensor -> integer codes of `output_dtype` (reference :134-206)."""
    assert input.dtype in _FLOAT_DTYPES, f"Unsupported input dtype: {input.dtype}"
    quant_min, quant_max = _get_and_check_qmin_qmax(output_dtype, quant_min, quant_max)
    _get_reduction_params(block_size, input.size())
    _check_qparam(scale, "scale", block_size, input.size())
    if zero_point is not None:
        _check_qparam(zero_point, "zero_point", block_size, input.size())
    assert zero_point_domain in (ZeroPointDomain.INT, ZeroPointDomain.FLOAT)
    out = torch.empty(input.shape, dtype=output_dtype, device=input.device)
    if input.is_meta:
        return out
    require_cuda(input, scale, zero_point)
    x = input.contiguous()
    N, K, bN, bK = _as_2d_blocks(block_size, x.shape)
    scale = scale.contiguous()
    zp = None if zero_point is None else zero_point.contiguous()
    check(lib().ao_amd_quantize_affine(
        x.data_ptr(), _code(x.dtype, "input"), N, K, K, bN, bK, scale.data_ptr(), _code(scale.dtype, "scale"),
        None if zp is None else zp.data_ptr(), 0 if zp is None else _code(zp.dtype, "zero_point"), quant_min, quant_max,
        zero_point_domain.value, out.data_ptr(), _code(output_dtype, "output"), current_stream(x.device)))
    return out


def dequantize_affine(
    input: torch.Tensor,
    block_size: Tuple[int, ...],
    scale: torch.Tensor,
    zero_point: Optional[torch.Tensor],
    input_dtype: torch.dtype,
    quant_min: Optional[int] = None,
    quant_max: Optional[int] = None,
    zero_point_domain: ZeroPointDomain = ZeroPointDomain.INT,
    *,
    output_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Integer codes -> float tensor of `output_dtype` (reference :208-276)."""
    assert input.dtype == input_dtype, f"Expected: {input_dtype}, got: {input.dtype}"
    assert output_dtype in _FLOAT_DTYPES, f"Unsupported output dtype: {output_dtype}"
    quant_min, quant_max = _get_and_check_qmin_qmax(input_dtype, quant_min, quant_max)
    _get_reduction_params(block_size, input.size())
    _check_qparam(scale, "scale", block_size, input.size())
    assert zero_point_domain in (ZeroPointDomain.INT, ZeroPointDomain.FLOAT), \
        f"Unexpected zero point domain: {zero_point_domain}"
    out = torch.empty(input.shape, dtype=output_dtype, device=input.device)
    if input.is_meta:
        return out
    require_cuda(input, scale, zero_point)
    q = input.contiguous()
    N, K, bN, bK = _as_2d_blocks(block_size, q.shape)
    scale = scale.contiguous()
    zp = None if zero_point is None else zero_point.contiguous()
    check(lib().ao_amd_dequantize_affine(
        q.data_ptr(), _code(q.dtype, "input"), N, K, bN, bK, scale.data_ptr(), _code(scale.dtype, "scale"),
        None if zp is None else zp.data_ptr(), 0 if zp is None else _code(zp.dtype, "zero_point"), quant_min, quant_max,
        zero_point_domain.value, out.data_ptr(), _code(output_dtype, "output"), current_stream(q.device)))
    return out
