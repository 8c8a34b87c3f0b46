"""Small helpers shared by the host code (counterparts of torchao/utils.py:81-165)."""
import itertools
from functools import reduce
from math import gcd

import torch
import torch.nn.utils.parametrize as parametrize

__all__ = ["find_multiple", "get_model_size_in_bytes", "unwrap_tensor_subclass"]


def find_multiple(n: int, *args: int) -> int:
    """Smallest multiple of lcm(args) that is >= n (torchao/utils.py:81-85)."""
    k = reduce(lambda x, y: x * y // gcd(x, y), args + (1,))
    return n if n % k == 0 else n + k - (n % k)


def get_model_size_in_bytes(model, ignore_embeddings: bool = False) -> int:
    """Bytes of all parameters and buffers; tensor subclasses count their inner tensors
    (torchao/utils.py:87-111).  This is the model size the decode GB/s figure multiplies by tok/s."""

    def flat_size(t):
        if hasattr(t, "__tensor_flatten__"):
            return sum(flat_size(getattr(t, name)) for name in t.__tensor_flatten__()[0])
        return t.numel() * t.element_size()

    total = 0
    for _, child in model.named_children():
        if isinstance(child, torch.nn.Embedding) and ignore_embeddings:
            continue
        for p in itertools.chain(child.parameters(recurse=False), child.buffers(recurse=False)):
            total += flat_size(p)
        total += get_model_size_in_bytes(child, ignore_embeddings)
    return total


class UnwrapTensorSubclass(torch.nn.Module):
    """Parametrization that stores a (nested) tensor subclass as its plain inner tensors and rebuilds
    it on access (torchao/utils.py:113-146); lets export / AOT tooling see only plain tensors."""

    def forward(self, *tensors):
        todo = list(tensors)
        for tp, meta, names in reversed(self.rebuild_stack):
            n = len(names)
            inner = dict(zip(names, todo[-n:]))
            todo = todo[:-n] if n else todo
            todo.append(tp.__tensor_unflatten__(inner, meta, None, None))
        assert len(todo) == 1
        return todo[0]

    def right_inverse(self, tensor):
        assert type(tensor) is not torch.Tensor
        self.rebuild_stack = []
        plain = []
        todo = [tensor]
        while todo:
            obj = todo.pop()
            names, meta = obj.__tensor_flatten__()
            self.rebuild_stack.append((type(obj), meta, names))
            nested = []
            for name in names:
                val = getattr(obj, name)
                if type(val) is torch.Tensor:
                    plain.append(val)
                else:
                    nested.append(val)
            assert len(nested) == 0 or len(nested) == len(names), "mixed plain / nested inner tensors"
            todo.extend(nested)
        return plain


def unwrap_tensor_subclass(model, filter_fn=None):
    """Replace subclass weights of nn.Linear modules by parametrizations over plain tensors
    (torchao/utils.py:148-165)."""
    for _, child in model.named_children():
        w = getattr(child, "weight", None)
        if (isinstance(child, torch.nn.Linear) and w is not None and type(w) is not torch.Tensor
                and type(w) is not torch.nn.Parameter and isinstance(w, torch.Tensor)):
            parametrize.register_parametrization(child, "weight", UnwrapTensorSubclass())
        unwrap_tensor_subclass(child)
    return model
