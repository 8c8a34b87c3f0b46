"""AffineQuantizedTensor and its layouts.

Host-side mirror of torchao/dtypes/affine_quantized_tensor.py: the same tensor-subclass protocol
(`_make_wrapper_subclass`, `__tensor_flatten__`, `__torch_function__` for F.linear, `__torch_dispatch__`
for mm / addmm / detach / clone / _to_copy / t) and the same layout plugin seam.  The int4 layout is this
library's own wave64 tile order ("gfx950_wave_tiled", also reachable under the reference's name
"tensor_core_tiled"), produced and consumed by the HIP kernels behind `torch.ops.torchao.int4wo_*`.
"""
from typing import Optional, Tuple

import torch
from torch.utils._python_dispatch import return_and_correct_aliasing

from .. import ops
from ..quantization.quant_primitives import (
    MappingType,
    ZeroPointDomain,
    choose_qparams_affine,
    dequantize_affine,
    quantize_affine,
)
from .utils import (
    _ATEN_OP_OR_TORCH_FN_TABLE,
    _get_layout_tensor_constructor,
    _implements,
    _register_layout_cls,
)

aten = torch.ops.aten

__all__ = [
    "AQTLayout",
    "AffineQuantizedTensor",
    "PlainAQTLayout",
    "Gfx950WaveTiledAQTLayout",
    "TensorCoreTiledAQTLayout",
    "to_affine_quantized",
    "register_layout_cls",
    "get_layout_tensor_constructor",
    "implements",
]


def _to_kwargs(tensor, *args, **kwargs):
    device, dtype, _, memory_format = torch._C._nn._parse_to(*args, **kwargs)
    return {
        "device": tensor.device if device is None else device,
        "dtype": tensor.dtype if dtype is None else dtype,
        "memory_format": torch.preserve_format if memory_format is None else memory_format,
    }


class AQTLayout(torch.Tensor):
    """Base class of the storage ("layout") tensors held by an AffineQuantizedTensor
    (reference :51-84).  A layout knows how to be built from plain (int_data, scale, zero_point)
    and how to give them back."""

    extended_layout: Optional[str] = None

    def get_plain(self) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        raise NotImplementedError

    @classmethod
    def from_plain(cls, int_data, scale, zero_point):
        raise NotImplementedError

    __torch_function__ = torch._C._disabled_torch_function_impl


def _is_uint4(aqt) -> bool:
    return aqt.quant_min == 0 and aqt.quant_max == 15


class AffineQuantizedTensor(torch.Tensor):
    """quantized = float / scale + zero_point, stored by a layout tensor (reference :86-303).

    shape / dtype describe the tensor as the model sees it (the original float weight); `layout_tensor`
    holds the quantized data in whatever order the kernels want."""

    @staticmethod
    def __new__(cls, layout_tensor, block_size, shape, quant_min=None, quant_max=None,
                zero_point_domain=ZeroPointDomain.INT, dtype=None, strides=None):
        kwargs = {"device": layout_tensor.device, "layout": layout_tensor.layout, "dtype": dtype,
                  "requires_grad": False}
        if strides is not None:
            kwargs["strides"] = strides
        return torch.Tensor._make_wrapper_subclass(cls, shape, **kwargs)

    def __init__(self, layout_tensor, block_size, shape, quant_min=None, quant_max=None,
                 zero_point_domain=ZeroPointDomain.INT, dtype=None, strides=None):
        self.layout_tensor = layout_tensor
        self.block_size = tuple(block_size)
        self.quant_min = quant_min
        self.quant_max = quant_max
        self.zero_point_domain = zero_point_domain

    def __repr__(self):
        return (f"{self.__class__.__name__}(layout={self.extended_layout}, block_size={self.block_size}, "
                f"shape={tuple(self.shape)}, device={self.device}, dtype={self.dtype})")

    @property
    def extended_layout(self) -> str:
        return self.layout_tensor.extended_layout

    def dequantize(self, output_dtype=None):
        output_dtype = self.dtype if output_dtype is None else output_dtype
        layout = self.layout_tensor
        if isinstance(layout, Gfx950WaveTiledAQTLayout) and output_dtype is torch.bfloat16 \
                and self.zero_point_domain == ZeroPointDomain.FLOAT:
            out = layout.dequantize_bf16()
            return out.t() if layout.transposed else out
        int_data, scale, zero_point = layout.get_plain()
        block_size = self.block_size
        if getattr(layout, "transposed", False):
            block_size = block_size[::-1]
        out = dequantize_affine(int_data, block_size, scale, zero_point, int_data.dtype, self.quant_min,
                                self.quant_max, self.zero_point_domain, output_dtype=output_dtype)
        return out.t() if getattr(layout, "transposed", False) else out

    def __tensor_flatten__(self):
        return ["layout_tensor"], [self.block_size, self.shape, self.quant_min, self.quant_max,
                                   self.zero_point_domain, self.dtype]

    @classmethod
    def __tensor_unflatten__(cls, tensor_data_dict, tensor_attributes, outer_size, outer_stride):
        block_size, shape, quant_min, quant_max, zero_point_domain, dtype = tensor_attributes
        return cls(tensor_data_dict["layout_tensor"], block_size, shape if outer_size is None else outer_size,
                   quant_min, quant_max, zero_point_domain, dtype=dtype, strides=outer_stride)

    @classmethod
    def from_float(cls, input_float, mapping_type, block_size, target_dtype, quant_min=None, quant_max=None,
                   eps=None, scale_dtype=None, zero_point_dtype=None, preserve_zero=True,
                   zero_point_domain=ZeroPointDomain.INT, extended_layout="plain", inner_k_tiles=None):
        """Quantize a float tensor (reference :184-229).

        For the int4 weight-only recipe on a bf16 weight the whole chain (zero padding, choose_qparams,
        quantize, pack) is one fused kernel; any other combination runs the primitives one by one and
        hands plain tensors to the layout constructor."""
        original_shape = input_float.shape
        tiled = extended_layout in ("gfx950_wave_tiled", "tensor_core_tiled")
        int4_recipe = (
            tiled and input_float.dim() == 2 and input_float.dtype is torch.bfloat16
            and mapping_type == MappingType.ASYMMETRIC and len(block_size) == 2 and block_size[0] == 1
            and block_size[1] in (32, 64, 128, 256) and quant_min == 0 and quant_max == 15 and eps == 1e-6
            and scale_dtype in (None, torch.bfloat16) and zero_point_dtype is torch.bfloat16
            and not preserve_zero and zero_point_domain == ZeroPointDomain.FLOAT
        )
        if int4_recipe:
            packed, qparams = ops.int4wo_quantize_pack(input_float, block_size[1])
            layout_tensor = Gfx950WaveTiledAQTLayout(packed, qparams, original_shape[0], original_shape[1],
                                                     block_size[1], False)
        else:
            if tiled:
                # the reference zero-extends K (to 1024) and N (to 8) before quantizing; the groups that
                # matter here are those that overlap the real weight, which need K up to a group multiple
                g = block_size[-1]
                pad_k = (-input_float.shape[-1]) % g
                if pad_k:
                    input_float = torch.nn.functional.pad(input_float, (0, pad_k))
            scale, zero_point = choose_qparams_affine(input_float, mapping_type, block_size, target_dtype, quant_min,
                                                      quant_max, eps, scale_dtype, zero_point_dtype, preserve_zero,
                                                      zero_point_domain)
            int_data = quantize_affine(input_float, block_size, scale, zero_point, target_dtype, quant_min, quant_max,
                                       zero_point_domain)
            ctor = get_layout_tensor_constructor(extended_layout)
            if tiled:
                layout_tensor = ctor(int_data, scale, zero_point, inner_k_tiles)
                layout_tensor.K = original_shape[1]
            else:
                layout_tensor = ctor(int_data, scale, zero_point)
        return cls(layout_tensor, block_size, original_shape, quant_min, quant_max, zero_point_domain,
                   dtype=input_float.dtype)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = {} if kwargs is None else kwargs
        handler = _ATEN_OP_OR_TORCH_FN_TABLE[cls].get(func)
        if handler is not None:
            return handler(*args, **kwargs)
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **kwargs)

    def to(self, *args, **kwargs):
        kw = _to_kwargs(self, *args, **kwargs)
        return self.__class__(self.layout_tensor.to(kw["device"]), self.block_size, self.shape, self.quant_min,
                              self.quant_max, self.zero_point_domain, dtype=kw["dtype"])

    def _apply_fn_to_data(self, fn):
        return self.__class__(fn(self.layout_tensor), self.block_size, self.shape, self.quant_min, self.quant_max,
                              self.zero_point_domain, dtype=self.dtype, strides=self.stride())

    @classmethod
    def __torch_dispatch__(cls, func, types, args, kwargs):
        handler = _ATEN_OP_OR_TORCH_FN_TABLE[cls].get(func)
        if handler is not None:
            return handler(func, *args, **(kwargs or {}))
        raise NotImplementedError(f"AffineQuantizedTensor dispatch: attempting to run {func}, this is not supported")


def implements(aten_ops_or_torch_fn):
    return _implements(AffineQuantizedTensor, aten_ops_or_torch_fn)


def register_layout_cls(extended_layout: str, *aliases: str):
    return _register_layout_cls(AffineQuantizedTensor, extended_layout, *aliases)


def get_layout_tensor_constructor(extended_layout: str):
    return _get_layout_tensor_constructor(AffineQuantizedTensor, extended_layout)


@register_layout_cls("plain")
class PlainAQTLayout(AQTLayout):
    """int_data, scale and zero_point kept as plain tensors (reference :314-407)."""

    @staticmethod
    def __new__(cls, int_data, scale, zero_point):
        return torch.Tensor._make_wrapper_subclass(cls, int_data.shape, device=int_data.device, layout=int_data.layout,
                                                   dtype=int_data.dtype, requires_grad=False)

    def __init__(self, int_data, scale, zero_point):
        self.int_data = int_data
        self.scale = scale
        self.zero_point = zero_point

    def __tensor_flatten__(self):
        return ["int_data", "scale", "zero_point"], []

    @classmethod
    def __tensor_unflatten__(cls, tensor_data_dict, tensor_attributes, outer_size, outer_stride):
        return cls(tensor_data_dict["int_data"], tensor_data_dict["scale"], tensor_data_dict["zero_point"])

    def to(self, *args, **kwargs):
        device = _to_kwargs(self, *args, **kwargs)["device"]
        return self.__class__(self.int_data.to(device), self.scale.to(device), self.zero_point.to(device))

    def _apply_fn_to_data(self, fn):
        return self.__class__(fn(self.int_data), fn(self.scale), fn(self.zero_point))

    @classmethod
    def __torch_dispatch__(cls, func, types, args, kwargs):
        kwargs = {} if kwargs is None else kwargs
        if func is aten.detach.default:
            return return_and_correct_aliasing(func, args, kwargs, args[0]._apply_fn_to_data(torch.detach))
        if func is aten.clone.default:
            return return_and_correct_aliasing(func, args, kwargs, args[0]._apply_fn_to_data(torch.clone))
        if func is aten.t.default:
            t = args[0]
            new = t.__class__(t.int_data.view(t.shape[::-1]), t.scale, t.zero_point)
            return return_and_correct_aliasing(func, args, kwargs, new)
        raise NotImplementedError(f"PlainAQTLayout dispatch: attempting to run {func}, this is not supported")

    def get_plain(self):
        return self.int_data, self.scale, self.zero_point

    @classmethod
    def from_plain(cls, int_data, scale, zero_point):
        return cls(int_data, scale, zero_point)


@register_layout_cls("gfx950_wave_tiled", "tensor_core_tiled")
class Gfx950WaveTiledAQTLayout(AQTLayout):
    """uint4 codes in wave64 tile order plus interleaved (scale, zero) words.

    Takes the place of the reference's TensorCoreTiledAQTLayout (:409-537), whose packed tensor is the
    tensor-core tile order of aten::_convert_weight_to_int4pack.  Fields:
      packed_weight  int32 [Np/16, Kp/128, 64, 4]   (see include/ao_amd.h for the element order)
      scale_and_zero int32 [Np/16, Kp/g, 16]        scale_bf16 | zero_bf16 << 16
      N, K, group_size                              logical weight shape and group size
      transposed                                    flipped by .t(); the data is never repacked
    """

    @staticmethod
    def __new__(cls, packed_weight, scale_and_zero, N, K, group_size, transposed):
        return torch.Tensor._make_wrapper_subclass(cls, packed_weight.shape, device=packed_weight.device,
                                                   layout=packed_weight.layout, dtype=packed_weight.dtype,
                                                   requires_grad=False)

    def __init__(self, packed_weight, scale_and_zero, N, K, group_size, transposed):
        self.packed_weight = packed_weight
        self.scale_and_zero = scale_and_zero
        self.N = int(N)
        self.K = int(K)
        self.group_size = int(group_size)
        self.transposed = bool(transposed)

    def __tensor_flatten__(self):
        return ["packed_weight", "scale_and_zero"], [self.N, self.K, self.group_size, self.transposed]

    @classmethod
    def __tensor_unflatten__(cls, tensor_data_dict, tensor_attributes, outer_size, outer_stride):
        N, K, group_size, transposed = tensor_attributes
        return cls(tensor_data_dict["packed_weight"], tensor_data_dict["scale_and_zero"], N, K, group_size, transposed)

    @classmethod
    def from_plain(cls, int_data, scale, zero_point, inner_k_tiles=None):
        """int_data int32 [N,K] in 0..15, scale / zero_point bf16 [N, K/g].  `inner_k_tiles` is a tuning
        knob of the tensor-core layout; it is accepted and has no meaning here."""
        N, K = int_data.shape
        scale = scale.reshape(N, -1)
        zero_point = zero_point.reshape(N, -1)
        group_size = K // scale.shape[1]
        packed, qparams = ops.int4wo_pack(int_data, scale, zero_point, group_size)
        return cls(packed, qparams, N, K, group_size, False)

    def get_plain(self):
        """(int_data int32 [N,Kg], scale bf16 [N,Kg/g], zero_point bf16 [N,Kg/g]) where Kg is K rounded up
        to a whole group (the width the weight was quantized at; equal to K for every real model shape)."""
        Kg = (self.K + self.group_size - 1) // self.group_size * self.group_size
        return ops.int4wo_unpack(self.packed_weight, self.scale_and_zero, self.N, Kg, self.group_size)

    def dequantize_bf16(self):
        return ops.int4wo_dequantize(self.packed_weight, self.scale_and_zero, self.N, self.K, self.group_size)

    def to(self, *args, **kwargs):
        device = _to_kwargs(self, *args, **kwargs)["device"]
        if torch.device(device).type not in ("cuda", "meta"):
            raise ValueError(f"{self.__class__.__name__} is only available for cuda device, can't convert to {device}")
        return self.__class__(self.packed_weight.to(device), self.scale_and_zero.to(device), self.N, self.K,
                              self.group_size, self.transposed)

    def _apply_fn_to_data(self, fn):
        return self.__class__(fn(self.packed_weight), fn(self.scale_and_zero), self.N, self.K, self.group_size,
                              self.transposed)

    def __repr__(self):
        return (f"{self.__class__.__name__}(N={self.N}, K={self.K}, group_size={self.group_size}, "
                f"transposed={self.transposed}, device={self.device})")

    @classmethod
    def __torch_dispatch__(cls, func, types, args, kwargs):
        kwargs = {} if kwargs is None else kwargs
        if func is aten.detach.default:
            return return_and_correct_aliasing(func, args, kwargs, args[0]._apply_fn_to_data(torch.detach))
        if func is aten.clone.default:
            return return_and_correct_aliasing(func, args, kwargs, args[0]._apply_fn_to_data(torch.clone))
        if func is aten.t.default:
            t = args[0]
            new = cls(t.packed_weight, t.scale_and_zero, t.N, t.K, t.group_size, not t.transposed)
            return return_and_correct_aliasing(func, args, kwargs, new)
        raise NotImplementedError(f"{cls.__name__} dispatch: attempting to run {func}, this is not supported")


# the reference's class name, for code that imports it
TensorCoreTiledAQTLayout = Gfx950WaveTiledAQTLayout


def _quantized_linear_op(input_tensor, weight_qtensor, bias):
    """F.linear with a quantized weight (reference :539-670).  Raises NotImplementedError when no
    kernel matches so that the caller can dequantize instead."""
    if isinstance(input_tensor, AffineQuantizedTensor):
        input_tensor = input_tensor.dequantize()
    if not isinstance(weight_qtensor, AffineQuantizedTensor):
        raise NotImplementedError("weight is not an AffineQuantizedTensor")
    layout = weight_qtensor.layout_tensor
    if (
        isinstance(layout, Gfx950WaveTiledAQTLayout)
        and not layout.transposed
        and _is_uint4(weight_qtensor)
        and weight_qtensor.dtype is torch.bfloat16
        and weight_qtensor.dim() == 2
        and weight_qtensor.zero_point_domain == ZeroPointDomain.FLOAT
    ):
        assert weight_qtensor.block_size[0] == 1, \
            f"Requires groupwise quantization, got block_size: {weight_qtensor.block_size}"
        assert input_tensor.shape[-1] == weight_qtensor.shape[1], (
            f"need input_tensor shape: {input_tensor.shape} final dim to match weight_tensor shape: "
            f"{weight_qtensor.shape} second dim")
        orig_shape, orig_dtype = input_tensor.shape, input_tensor.dtype
        act = input_tensor.reshape(-1, orig_shape[-1]).to(torch.bfloat16)
        fused_bias = bias if (bias is not None and bias.dtype is torch.bfloat16) else None
        y = ops.int4wo_linear(act, layout.packed_weight, layout.scale_and_zero, layout.group_size, layout.N,
                              fused_bias)
        y = y.reshape(*orig_shape[:-1], layout.N)
        if bias is not None and fused_bias is None:
            y = y + bias
        return y.to(orig_dtype)
    if (
        isinstance(layout, PlainAQTLayout)
        and layout.int_data.dtype is torch.int8
        and weight_qtensor.dim() == 2
        and len(weight_qtensor.block_size) == 2
        and weight_qtensor.block_size[0] == 1
        and weight_qtensor.block_size[1] == weight_qtensor.shape[1]
        and weight_qtensor.zero_point_domain == ZeroPointDomain.INT
    ):
        # per-channel int8 weight-only (reference :641-665): mm(x, w_int8.t().to(x.dtype)) * scale, the symmetric
        # recipe's zero point is zero and, as in the reference, does not enter
        orig_shape, orig_dtype = input_tensor.shape, input_tensor.dtype
        if (
            orig_dtype is torch.bfloat16
            and weight_qtensor.dtype is torch.bfloat16
            and layout.int_data.is_cuda
            and weight_qtensor.shape[1] % 128 == 0
            and layout.int_data.stride(1) == 1 and layout.int_data.stride(0) % 16 == 0
        ):
            act = input_tensor.reshape(-1, orig_shape[-1])
            fused_bias = bias if (bias is not None and bias.dtype is torch.bfloat16) else None
            y = ops.int8wo_linear(act, layout.int_data, layout.scale.reshape(-1).to(torch.bfloat16), fused_bias)
            y = y.reshape(*orig_shape[:-1], weight_qtensor.shape[0])
            if bias is not None and fused_bias is None:
                y = y + bias
            return y.to(orig_dtype)
        # other activation dtypes (the product is formed in the activation's dtype there) and in_features that are
        # not a multiple of 128: the reference's own op sequence
        y = torch.mm(input_tensor.reshape(-1, orig_shape[-1]), layout.int_data.t().to(orig_dtype)) * layout.scale
        y = y.reshape(*orig_shape[:-1], y.shape[-1])
        if bias is not None:
            y += bias
        return y.to(orig_dtype)
    raise NotImplementedError("No specialized dispatch found for quantized linear op")


def _dequantize_args(*tensors):
    return [t.dequantize() if isinstance(t, AffineQuantizedTensor) else t for t in tensors]


@implements(torch.nn.functional.linear)
def _functional_linear(*args, **kwargs):
    input_tensor, weight_tensor = args[0], args[1]
    bias = args[2] if len(args) > 2 else kwargs.get("bias")
    try:
        return _quantized_linear_op(input_tensor, weight_tensor, bias)
    except NotImplementedError:
        input_tensor, weight_tensor = _dequantize_args(input_tensor, weight_tensor)
        return torch.nn.functional.linear(input_tensor, weight_tensor, bias)


@implements([aten.mm.default, aten.addmm.default])
def _aten_mm(func, *args, **kwargs):
    if func is aten.addmm.default:
        bias, input_tensor, weight_tensor = args[0], args[1], args[2]
    else:
        bias, input_tensor, weight_tensor = None, args[0], args[1]
    if not input_tensor.is_floating_point():
        raise NotImplementedError(f"{func} is not implemented for non floating point input")
    try:
        return _quantized_linear_op(input_tensor, weight_tensor.t(), bias)
    except NotImplementedError:
        input_tensor, weight_tensor = _dequantize_args(input_tensor, weight_tensor)
        return func(input_tensor, weight_tensor) if bias is None else func(bias, input_tensor, weight_tensor)


@implements([aten.detach.default])
def _detach(func, *args, **kwargs):
    return return_and_correct_aliasing(func, args, kwargs, args[0]._apply_fn_to_data(torch.detach))


@implements([aten.clone.default])
def _clone(func, *args, **kwargs):
    return return_and_correct_aliasing(func, args, kwargs, args[0]._apply_fn_to_data(torch.clone))


@implements([aten._to_copy.default])
def _to_copy(func, *args, **kwargs):
    return return_and_correct_aliasing(func, args, kwargs, args[0].to(*args[1:], **kwargs)._apply_fn_to_data(torch.clone))


@implements([aten.t.default])
def _t(func, *args, **kwargs):
    tensor = args[0]
    assert len(tensor.block_size) == 2
    new = tensor.__class__(tensor.layout_tensor.t(), tensor.block_size[::-1], tensor.shape[::-1], tensor.quant_min,
                           tensor.quant_max, tensor.zero_point_domain, dtype=tensor.dtype, strides=tensor.stride())
    return return_and_correct_aliasing(func, args, kwargs, new)


to_affine_quantized = AffineQuantizedTensor.from_float
