"""Model-rewrite API: swap the weights of nn.Linear modules for quantized tensor subclasses.

Mirrors torchao/quantization/quant_api.py: `quantize` (:262-318) walks the module tree
(`_replace_with_custom_fn_if_matches_filter`, :146-176) and replaces each matching Linear's weight with
`apply_tensor_subclass(weight)`; `int4_weight_only` (:362-387) builds that function for uint4 groupwise
asymmetric quantization.  `quantize_` is the in-place spelling later releases use.
"""
from typing import Callable, Optional

import torch

from .quant_primitives import MappingType, ZeroPointDomain

__all__ = ["quantize", "quantize_", "int4_weight_only", "int8_weight_only", "fp6_llm_weight_only",
           "change_linear_weights_to_int4_woqtensors", "change_linear_weights_to_int8_woqtensors",
           "quant_llm_fpx_weight_only"]


def _replace_with_custom_fn_if_matches_filter(model, replacement_fn, filter_fn, cur_fqn=""):
    """Depth-first: replace every module for which filter_fn(module, fqn) holds by replacement_fn(module)."""
    if filter_fn(model, cur_fqn[:-1]):
        return replacement_fn(model)
    for name, child in model.named_children():
        new_child = _replace_with_custom_fn_if_matches_filter(child, replacement_fn, filter_fn, f"{cur_fqn}{name}.")
        if new_child is not child:
            setattr(model, name, new_child)
    return model


def _is_linear(mod, *args):
    """nn.Linear whose weight is not already a quantized subclass (a weight shared by several modules
    is quantized once)."""
    from ..dtypes import AffineQuantizedTensor
    from ..prototype.quant_llm import QuantLlmLinearWeight

    return (
        isinstance(mod, torch.nn.Linear)
        and hasattr(mod, "weight")
        and not isinstance(mod.weight, (AffineQuantizedTensor, QuantLlmLinearWeight))
    )


def _get_linear_subclass_inserter(constructor):
    def insert_subclass(lin):
        lin.weight = torch.nn.Parameter(constructor(lin.weight), requires_grad=False)
        return lin

    return insert_subclass


def quantize(model: torch.nn.Module, apply_tensor_subclass: Callable[[torch.Tensor], torch.Tensor],
             filter_fn: Optional[Callable[[torch.nn.Module, str], bool]] = None,
             set_inductor_config: bool = True) -> torch.nn.Module:
    """Convert the weight of the linear modules selected by `filter_fn` (default: every nn.Linear) with
    `apply_tensor_subclass` and return the model.

        m = quantize(m, int4_weight_only(group_size=64))

    `set_inductor_config` is accepted for signature compatibility; nothing here uses inductor."""
    _replace_with_custom_fn_if_matches_filter(
        model,
        _get_linear_subclass_inserter(apply_tensor_subclass),
        _is_linear if filter_fn is None else filter_fn,
    )
    return model


def quantize_(model, apply_tensor_subclass, filter_fn=None, set_inductor_config: bool = True) -> None:
    """In-place form of `quantize`."""
    quantize(model, apply_tensor_subclass, filter_fn, set_inductor_config)


def int4_weight_only(group_size=128, inner_k_tiles=8):
    """uint4 weight-only asymmetric per-group quantization, float zero point, packed for the gfx950
    kernels.  `group_size` in {256, 128, 64, 32}; `inner_k_tiles` is accepted and ignored (it tunes
    the tensor-core layout this library does not use)."""
    if group_size not in (32, 64, 128, 256):
        raise ValueError(f"group_size must be one of 256, 128, 64, 32, got {group_size}")

    def apply_int4_weight_only_quant(weight):
        from ..dtypes import to_affine_quantized

        return to_affine_quantized(
            weight, MappingType.ASYMMETRIC, (1, group_size), torch.int32, 0, 15, 1e-6,
            zero_point_dtype=torch.bfloat16, preserve_zero=False, zero_point_domain=ZeroPointDomain.FLOAT,
            extended_layout="gfx950_wave_tiled", inner_k_tiles=inner_k_tiles)

    return apply_int4_weight_only_quant


def int8_weight_only():
    """int8 weight-only symmetric per-channel quantization (reference :390-405): one bf16 scale per output row,
    zero point 0, codes kept in the plain [N, K] layout, which the gfx950 kernel reads in place."""

    def apply_int8wo_quant(weight):
        from ..dtypes import to_affine_quantized

        return to_affine_quantized(weight, MappingType.SYMMETRIC, (1, weight.shape[1]), torch.int8,
                                   eps=torch.finfo(torch.float32).eps, zero_point_dtype=torch.int64)

    return apply_int8wo_quant


def quant_llm_fpx_weight_only(ebits: int, mbits: int):
    from ..prototype.quant_llm import quant_llm_fpx_weight_only as impl

    return impl(ebits, mbits)


def fp6_llm_weight_only():
    return quant_llm_fpx_weight_only(3, 2)


def change_linear_weights_to_int4_woqtensors(model, groupsize=128, inner_k_tiles=8, filter_fn=None):
    """Legacy entry point (reference quant_api.py:119-141): every linear weight becomes the legacy
    `Int4WeightOnlyQuantizedLinearWeight` tensor subclass (subclass.py:394-601), in place.  The reference refuses
    to run it on PyTorch >= 2.4 in favour of `quantize_`; it works here on any version."""
    from .subclass import Int4WeightOnlyQuantizedLinearWeight

    def is_plain_linear(mod, *args):
        return _is_linear(mod, *args) and not isinstance(mod.weight, Int4WeightOnlyQuantizedLinearWeight)

    def swap(lin):
        lin.weight = torch.nn.Parameter(
            Int4WeightOnlyQuantizedLinearWeight.from_float(lin.weight, groupsize=groupsize, inner_k_tiles=inner_k_tiles),
            requires_grad=False)
        return lin

    _replace_with_custom_fn_if_matches_filter(model, swap, is_plain_linear if filter_fn is None else filter_fn)


def change_linear_weights_to_int8_woqtensors(model, filter_fn=None, **kwargs):
    """Legacy entry point (reference quant_api.py:103-117): per-channel int8 weight-only on every linear, in place;
    maps to `quantize_(model, int8_weight_only())`."""
    quantize_(model, int8_weight_only(), filter_fn)
