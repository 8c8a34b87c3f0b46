"""Dispatch tables and the layout registry of the tensor subclasses.

Same plugin seam as torchao/dtypes/utils.py:12-65: `_implements` registers a handler for a torch
function or aten op on a subclass, `_register_layout_cls` maps a layout name to the constructor that
builds the layout tensor from plain (int_data, scale, zero_point).
"""
from collections import defaultdict
from typing import Callable, Dict

# subclass -> {torch function or aten overload -> handler}
_ATEN_OP_OR_TORCH_FN_TABLE: Dict[type, Dict[Callable, Callable]] = defaultdict(dict)
# subclass -> {layout name -> LayoutClass.from_plain}
_LAYOUT_CONSTRUCTOR_TABLE: Dict[type, Dict[str, Callable]] = defaultdict(dict)


def _implements(cls, aten_ops_or_torch_fns):
    """Decorator: use the function as the handler of one or several ops for `cls`."""
    if not isinstance(aten_ops_or_torch_fns, (list, tuple)):
        aten_ops_or_torch_fns = [aten_ops_or_torch_fns]

    def decorator(func):
        for op in aten_ops_or_torch_fns:
            _ATEN_OP_OR_TORCH_FN_TABLE[cls][op] = func
        return func

    return decorator


def _register_layout_cls(cls, extended_layout: str, *aliases: str):
    """Decorator: register a layout class under `extended_layout` (and optional alias names)."""

    def decorator(layout_cls):
        layout_cls.extended_layout = extended_layout
        for name in (extended_layout, *aliases):
            _LAYOUT_CONSTRUCTOR_TABLE[cls][name] = layout_cls.from_plain
        return layout_cls

    return decorator


def _get_layout_tensor_constructor(cls, extended_layout: str) -> Callable:
    if cls not in _LAYOUT_CONSTRUCTOR_TABLE:
        raise ValueError(f"no registered layout class constructor for: {cls}")
    if extended_layout not in _LAYOUT_CONSTRUCTOR_TABLE[cls]:
        raise ValueError(f"extended_layout: {extended_layout} is not supported yet for {cls}")
    return _LAYOUT_CONSTRUCTOR_TABLE[cls][extended_layout]
