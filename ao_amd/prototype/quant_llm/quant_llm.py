"""FP6-LLM / Quant-LLM weight-only linear (FPx with 1 + ebits + mbits bits, per-row fp16 scale).

Host-side mirror of torchao/prototype/quant_llm/quant_llm.py: `to_scaled_tc_fpx` (:116-130),
`from_scaled_tc_fpx` (:203-208), `QuantLlmLinearWeight` (:348-417), its F.linear handler (:419-445) and
the `quant_llm_fpx_weight_only` / `fp6_llm_weight_only` constructors (:453-463).  The packed bytes are
the reference's TC-FPx interchange format bit for bit; the gfx950 kernel reads a one-time device repack
of them that the weight subclass carries along.
"""
from typing import Tuple

import torch
from torch import Tensor
from torch.utils._python_dispatch import return_and_correct_aliasing

from ... import ops
from ...dtypes.utils import _ATEN_OP_OR_TORCH_FN_TABLE, _implements

__all__ = ["to_scaled_tc_fpx", "from_scaled_tc_fpx", "QuantLlmLinearWeight", "quant_llm_fpx_weight_only",
           "fp6_llm_weight_only"]


def _check_fp6(ebits: int, mbits: int):
    # the formats the reference kernel dispatches (torchao/csrc/cuda/fp6_llm/fp6_linear.cu:173-184)
    if (ebits, mbits) not in ((3, 2), (2, 3), (2, 2), (3, 1)):
        raise NotImplementedError(f"FP{1 + ebits + mbits} E{ebits}M{mbits} is not supported "
                                  "(e3m2, e2m3, e2m2 and e3m1 only)")


def to_scaled_tc_fpx(tensor: Tensor, ebits: int, mbits: int) -> Tuple[Tensor, Tensor]:
    """float [N,K] -> (TC-FPx bytes uint8 [N, K*nbits/8], per-row scale fp16 [N])."""
    _check_fp6(ebits, mbits)
    return ops.fp6_quantize_pack(tensor, ebits, mbits)


def from_scaled_tc_fpx(tensor: Tensor, ebits: int, mbits: int, scale=None) -> Tensor:
    """TC-FPx bytes (+ scale) -> fp32 [N,K]."""
    _check_fp6(ebits, mbits)
    return ops.fp6_dequantize(tensor, scale, ebits, mbits)


class QuantLlmLinearWeight(Tensor):
    """Weight of a linear layer stored as packed FPx + fp16 row scales.

    `fpx_data` / `scale` are the serialised state (the reference's format); `_native` is the same
    bits rearranged for the wave64 kernel, rebuilt whenever the tensor is constructed."""

    implements = classmethod(_implements)

    @staticmethod
    def __new__(cls, fpx_data: Tensor, scale: Tensor, ebits: int, mbits: int):
        assert fpx_data.ndim == 2
        assert fpx_data.dtype == torch.uint8
        shape = (fpx_data.shape[0], fpx_data.shape[1] // (1 + ebits + mbits) * 8)
        return Tensor._make_wrapper_subclass(cls, shape, device=fpx_data.device, requires_grad=False)

    def __init__(self, fpx_data: Tensor, scale: Tensor, ebits: int, mbits: int):
        self.fpx_data = fpx_data
        self.scale = scale
        self.ebits = ebits
        self.mbits = mbits
        self._native = None

    def native(self) -> Tensor:
        if self._native is None:
            self._native = ops.fp6_repack(self.fpx_data, 1 + self.ebits + self.mbits)
        return self._native

    def __tensor_flatten__(self):
        return ["fpx_data", "scale"], [self.ebits, self.mbits]

    @classmethod
    def __tensor_unflatten__(cls, tensor_data_dict, tensor_attributes, outer_size=None, outer_stride=None):
        return cls(tensor_data_dict["fpx_data"], tensor_data_dict["scale"], *tensor_attributes)

    @classmethod
    def from_float(cls, input_float: Tensor, ebits: int, mbits: int):
        fpx_data, scale = to_scaled_tc_fpx(input_float, ebits, mbits)
        return cls(fpx_data, scale, ebits, mbits)

    def dequantize(self, output_dtype=None):
        output_dtype = output_dtype or torch.get_default_dtype()
        return from_scaled_tc_fpx(self.fpx_data, self.ebits, self.mbits, self.scale).to(output_dtype)

    def __repr__(self):
        return (f"{self.__class__.__name__}(dtype=fp{1 + self.ebits + self.mbits}_e{self.ebits}m{self.mbits}, "
                f"shape={tuple(self.shape)}, device={self.device}, requires_grad={self.requires_grad})")

    def _apply_fn_to_data(self, fn):
        return self.__class__(fn(self.fpx_data), fn(self.scale), self.ebits, self.mbits)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = {} if kwargs is None else kwargs
        handler = _ATEN_OP_OR_TORCH_FN_TABLE[cls].get(func)
        if handler is not None:
            return handler(*args, **kwargs)
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **kwargs)

    @classmethod
    def __torch_dispatch__(cls, func, types, args, kwargs):
        handler = _ATEN_OP_OR_TORCH_FN_TABLE[cls].get(func)
        if handler is not None:
            return handler(func, *args, **(kwargs or {}))
        raise NotImplementedError(f"{cls.__name__} dispatch: attempting to run {func}, this is not supported")


@QuantLlmLinearWeight.implements(torch.nn.functional.linear)
def _(*args, **kwargs):
    act, weight = args[0], args[1]
    bias = args[2] if len(args) >= 3 else kwargs.get("bias")
    assert isinstance(weight, QuantLlmLinearWeight)
    out_dim, in_dim = weight.shape
    act_2d = act.reshape(-1, in_dim).half()
    # the reference picks a split-K factor from a table tuned for NVIDIA SM counts (:212-345, :427-431);
    # the gfx950 kernel sizes its own K split from the shape, so no table is consulted here
    out = ops.fp6_linear_native(weight.ebits, weight.mbits, act_2d, weight.native(), weight.scale)
    if bias is not None:
        out += bias
    return out.view(*act.shape[:-1], out_dim).to(act.dtype)


@QuantLlmLinearWeight.implements(torch.ops.aten.detach.default)
def _(func, *args, **kwargs):
    return return_and_correct_aliasing(func, args, kwargs, args[0]._apply_fn_to_data(torch.detach))


@QuantLlmLinearWeight.implements(torch.ops.aten.clone.default)
def _(func, *args, **kwargs):
    return return_and_correct_aliasing(func, args, kwargs, args[0]._apply_fn_to_data(torch.clone))


def quant_llm_fpx_weight_only(ebits: int, mbits: int):
    """Weights whose shape the kernel cannot take (in % 64 or out % 256) are left in floating point."""

    def apply_quant_llm(weight: Tensor) -> Tensor:
        out_dim, in_dim = weight.shape
        if (in_dim % 64 != 0) or (out_dim % 256 != 0):
            return weight
        return QuantLlmLinearWeight.from_float(weight, ebits, mbits)

    return apply_quant_llm


def fp6_llm_weight_only():
    return quant_llm_fpx_weight_only(3, 2)
