"""Plumbing shared by the tensor subclasses: op routing tables, the layout registry and a wrapper-subclass base.

The plugin seam is the reference's (torchao/dtypes/utils.py:12-65): `_implements` registers a handler for a torch
function or aten overload on a subclass, `_register_layout_cls` maps a layout name to the constructor that builds the
layout tensor from plain (int_data, scale, zero_point), `_get_layout_tensor_constructor` looks it up.

`PackedWeightBase` is this package's own: a wrapper subclass that names its inner tensors and plain attributes once
(`_inner`, `_plain`) and gets flattening, rebuilding under a per-tensor map (detach, clone, device moves) and the
routing of torch functions / aten overloads through the tables from those two tuples.
"""
from collections import defaultdict
from typing import Callable, Dict, Iterable, Tuple

import torch
from torch.utils._python_dispatch import return_and_correct_aliasing

# subclass -> {torch function or aten overload -> handler}
_ATEN_OP_OR_TORCH_FN_TABLE: Dict[type, Dict[Callable, Callable]] = defaultdict(dict)
# subclass -> {layout name -> LayoutClass.from_plain}
_LAYOUT_CONSTRUCTOR_TABLE: Dict[type, Dict[str, Callable]] = defaultdict(dict)


def _as_ops(one_or_many) -> Iterable[Callable]:
    return one_or_many if isinstance(one_or_many, (list, tuple)) else (one_or_many,)


def _implements(cls, aten_ops_or_torch_fns):
    """`@_implements(cls, op)` / `@_implements(cls, [op, ...])`: the decorated function serves those ops for `cls`."""
    table = _ATEN_OP_OR_TORCH_FN_TABLE[cls]

    def register(handler):
        table.update((op, handler) for op in _as_ops(aten_ops_or_torch_fns))
        return handler

    return register


def _register_layout_cls(cls, extended_layout: str, *aliases: str):
    """`@_register_layout_cls(cls, name, *aliases)`: the decorated layout class builds `cls`'s layout tensors of that
    name (the aliases let state written under the reference's layout names resolve to this package's classes)."""
    table = _LAYOUT_CONSTRUCTOR_TABLE[cls]

    def register(layout_cls):
        layout_cls.extended_layout = extended_layout
        table.update((name, layout_cls.from_plain) for name in (extended_layout, *aliases))
        return layout_cls

    return register


def _get_layout_tensor_constructor(cls, extended_layout: str) -> Callable:
    table = _LAYOUT_CONSTRUCTOR_TABLE.get(cls)
    if table is None:
        raise ValueError(f"no registered layout class constructor for: {cls}")
    try:
        return table[extended_layout]
    except KeyError:
        raise ValueError(f"extended_layout: {extended_layout} is not supported yet for {cls}") from None


class PackedWeightBase(torch.Tensor):
    """A weight whose storage is a few inner tensors plus plain attributes, constructed as `cls(*inner, *plain)`.

    Subclasses set `_inner` (attribute names of the tensors, in constructor order) and `_plain` (names of the other
    constructor arguments).  Everything that only moves or copies the storage is derived from those: the flatten
    protocol (`torch.save` / `load_state_dict(assign=True)` / compile), `_apply_fn_to_data`, and the aten overloads
    that alias or copy (`detach`, `clone`).  Other ops go through the handlers registered with `cls.implements`."""

    _inner: Tuple[str, ...] = ()
    _plain: Tuple[str, ...] = ()
    implements = classmethod(_implements)

    def _inner_tensors(self):
        return tuple(getattr(self, name) for name in self._inner)

    def _plain_attrs(self):
        return tuple(getattr(self, name) for name in self._plain)

    def __tensor_flatten__(self):
        return list(self._inner), list(self._plain_attrs())

    @classmethod
    def __tensor_unflatten__(cls, tensor_data_dict, tensor_attributes, outer_size=None, outer_stride=None):
        return cls(*(tensor_data_dict[name] for name in cls._inner), *tensor_attributes)

    def _apply_fn_to_data(self, fn):
        return type(self)(*(fn(t) for t in self._inner_tensors()), *self._plain_attrs())

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        handler = _ATEN_OP_OR_TORCH_FN_TABLE[cls].get(func)
        if handler is not None:
            return handler(*args, **(kwargs or {}))
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **(kwargs or {}))

    _STORAGE_ONLY = {torch.ops.aten.detach.default: torch.detach, torch.ops.aten.clone.default: torch.clone}

    @classmethod
    def __torch_dispatch__(cls, func, types, args, kwargs):
        kwargs = kwargs or {}
        handler = _ATEN_OP_OR_TORCH_FN_TABLE[cls].get(func)
        if handler is not None:
            return handler(func, *args, **kwargs)
        per_tensor = cls._STORAGE_ONLY.get(func)
        if per_tensor is not None:
            return return_and_correct_aliasing(func, args, kwargs, args[0]._apply_fn_to_data(per_tensor))
        raise NotImplementedError(f"{cls.__name__} dispatch: attempting to run {func}, this is not supported")
