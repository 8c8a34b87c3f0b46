"""The legacy int4 weight-only tensor subclass (reference torchao/quantization/subclass.py:394-601).

`Int4WeightOnlyQuantizedLinearWeight.from_float(w, groupsize, inner_k_tiles)` keeps the reference's constructor,
attribute names (`int_data`, `scales_and_zeros`, `transposed`, `groupsize`, `inner_k_tiles`) and accessors
(`dequantize`, `int_repr`, `q_params`, `to_qtensor_components`), because that is what state dicts and user code of the
legacy flow refer to.  What the attributes hold differs where the hardware does:

  int_data          int32 [ceil(N/16), Kp/128, 64, 4]   the wave64 tile order of the HIP kernels (the reference holds the
                                                        tensor-core order [N/8, K/(16 ikt), 32, ikt/2]; inner_k_tiles is
                                                        accepted and ignored)
  scales_and_zeros  bf16 [K/g, N, 2]                     the reference's buffer, same shape and bits

The codes and (scale, zero) pairs are the tinygemm groupwise ones (get_groupwise_affine_qparams /
groupwise_affine_quantize_tensor_from_qparams), computed by the HIP primitives.  The linear runs
torch.ops.torchao.int4wo_linear; `dequantize()` is the dequantize kernel, not a matmul with the identity.
"""
import torch
from torch.utils._python_dispatch import return_and_correct_aliasing

from ..dtypes.utils import _ATEN_OP_OR_TORCH_FN_TABLE, _implements
from .utils import groupwise_affine_quantize_tensor, unpack_tinygemm_scales_and_zeros

__all__ = ["Int4WeightOnlyQuantizedLinearWeight"]

aten = torch.ops.aten


def _interleaved(scales_and_zeros, groupsize):
    from .GPTQ import interleave_scales_and_zeros

    return interleave_scales_and_zeros(scales_and_zeros, groupsize)


class Int4WeightOnlyQuantizedLinearWeight(torch.Tensor):
    """Groupwise asymmetric int4 weight of a linear; `shape` is the logical [out_features, in_features]
    (or its transpose when `transposed`)."""

    @staticmethod
    def __new__(cls, int_data, scales_and_zeros, transposed, shape, groupsize=128, inner_k_tiles=8, dtype=None, **kwargs):
        kwargs["device"] = int_data.device
        kwargs["dtype"] = scales_and_zeros.dtype if dtype is None else dtype
        kwargs["layout"] = kwargs.get("layout", torch.strided)
        kwargs["requires_grad"] = False
        return torch.Tensor._make_wrapper_subclass(cls, shape, **kwargs)  # type: ignore[attr-defined]

    def __init__(self, int_data, scales_and_zeros, transposed, shape, groupsize=128, inner_k_tiles=8, dtype=None, **kwargs):
        self.int_data = int_data
        self.scales_and_zeros = scales_and_zeros
        self.transposed = transposed
        self.groupsize = groupsize
        self.inner_k_tiles = inner_k_tiles
        self._qparams = None   # the kernels' interleaved (scale | zero << 16) words, built on first use

    # ------------------------------------------------------------------ construction
    @classmethod
    def to_qtensor_components(cls, input_float, groupsize=128, inner_k_tiles=8):
        """(packed codes, scales_and_zeros, transposed, groupsize, inner_k_tiles) of a float weight
        [out_features, in_features], the reference's 5-tuple (:583-601); in_features is zero-extended to a whole number of groups (the reference pads to
        1024: its kernel needs it, these do not)."""
        assert groupsize in (256, 128, 64, 32), f"groupsize {groupsize} not supported"
        assert inner_k_tiles in (8, 4, 2), f"inner_k_tiles {inner_k_tiles} not supported"
        assert input_float.dim() == 2
        N, K = input_float.shape
        Kg = (K + groupsize - 1) // groupsize * groupsize
        w = input_float.to(torch.bfloat16)
        if Kg != K:
            w = torch.nn.functional.pad(w, (0, Kg - K))
        codes, scales_and_zeros = groupwise_affine_quantize_tensor(w, 4, groupsize, dtype=torch.bfloat16)
        scales, zeros = unpack_tinygemm_scales_and_zeros(scales_and_zeros)
        packed, _ = torch.ops.torchao.int4wo_pack(codes, scales.reshape(N, -1).contiguous(), zeros.reshape(N, -1).contiguous(), groupsize)
        return packed, scales_and_zeros, False, groupsize, inner_k_tiles

    @classmethod
    def from_float(cls, input_float, groupsize=128, inner_k_tiles=8, dtype=None):
        """Legacy conversion entry point (reference :551-571)."""
        if dtype is None:
            dtype = input_float.dtype
        int_data, scales_and_zeros, transposed, groupsize, inner_k_tiles = cls.to_qtensor_components(
            input_float, groupsize, inner_k_tiles)
        return cls(int_data, scales_and_zeros, transposed, input_float.shape, groupsize, inner_k_tiles, dtype=dtype)

    # ------------------------------------------------------------------ accessors
    def _interleaved_qparams(self):
        if self._qparams is None:
            self._qparams = _interleaved(self.scales_and_zeros, self.groupsize)
        return self._qparams

    def _logical(self):
        """(out_features, in_features)"""
        return (self.shape[1], self.shape[0]) if self.transposed else (self.shape[0], self.shape[1])

    @staticmethod
    def _quantized_op(act_mat, w_qtensor, bias):
        """act_mat @ dequant(w)^T (+ bias), computed in bf16, returned in the activation dtype (reference :441-467)."""
        N, K = w_qtensor._logical()
        orig = act_mat.size()
        x = act_mat.reshape(-1, orig[-1]).to(torch.bfloat16)
        Kg = w_qtensor.scales_and_zeros.shape[0] * w_qtensor.groupsize
        if Kg != K:
            x = torch.nn.functional.pad(x, (0, Kg - K))
        fused_bias = bias if bias is not None and bias.dtype is torch.bfloat16 else None
        y = torch.ops.torchao.int4wo_linear(x.contiguous(), w_qtensor.int_data, w_qtensor._interleaved_qparams(),
                                            w_qtensor.groupsize, N, fused_bias, False)
        y = y.reshape(*orig[:-1], N)
        if bias is not None and fused_bias is None:
            y = y + bias
        return y.to(act_mat.dtype)

    def dequantize(self):
        N, K = self._logical()
        Kg = self.scales_and_zeros.shape[0] * self.groupsize
        w = torch.ops.torchao.int4wo_dequantize(self.int_data, self._interleaved_qparams(), N, Kg, self.groupsize)[:, :K]
        w = w.t() if self.transposed else w
        return w.to(self.dtype)

    def int_repr(self):
        return self.int_data

    def q_params(self):
        scales, zero_points = unpack_tinygemm_scales_and_zeros(self.scales_and_zeros)
        return {"q_scales": scales, "q_zero_points": zero_points}

    def half(self):
        return self.to(torch.float16)

    def __repr__(self):
        return (f"{self.__class__.__name__}(shape={tuple(self.shape)}, groupsize={self.groupsize}, "
                f"transposed={self.transposed}, device={self.device}, dtype={self.dtype})")

    # ------------------------------------------------------------------ tensor plumbing
    def _with(self, int_data, scales_and_zeros, transposed=None, shape=None, dtype=None):
        return self.__class__(int_data, scales_and_zeros, self.transposed if transposed is None else transposed,
                              self.shape if shape is None else shape, self.groupsize, self.inner_k_tiles,
                              dtype=self.dtype if dtype is None else dtype)

    def _apply_fn_to_data(self, fn):
        return self._with(fn(self.int_data), fn(self.scales_and_zeros))

    def to(self, *args, **kwargs):
        device, dtype, _, _ = torch._C._nn._parse_to(*args, **kwargs)
        device = self.device if device is None else device
        return self._with(self.int_data.to(device), self.scales_and_zeros.to(device), dtype=dtype)

    def __tensor_flatten__(self):
        return ["int_data", "scales_and_zeros"], (self.transposed, self.groupsize, self.inner_k_tiles, self.dtype, self.shape)

    @classmethod
    def __tensor_unflatten__(cls, tensor_data_dict, attributes, outer_size=None, outer_stride=None):
        transposed, groupsize, inner_k_tiles, dtype, shape = attributes
        return cls(tensor_data_dict["int_data"], tensor_data_dict["scales_and_zeros"], transposed,
                   shape if outer_size is None else outer_size, groupsize, inner_k_tiles, dtype=dtype)

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
        raise NotImplementedError(f"Int4WeightOnlyQuantizedLinearWeight dispatch: attempting to run {func}, this is not supported")


def _implements_legacy(ops):
    return _implements(Int4WeightOnlyQuantizedLinearWeight, ops)


@_implements_legacy(torch.nn.functional.linear)
def _legacy_linear(*args, **kwargs):
    act, w = args[0], args[1]
    bias = args[2] if len(args) > 2 else kwargs.get("bias")
    assert not w.transposed, "F.linear expects the weight as [out_features, in_features]"
    return w._quantized_op(act, w, bias)


@_implements_legacy([aten.mm.default, aten.addmm.default])
def _legacy_mm(func, *args, **kwargs):
    if func is aten.addmm.default:
        bias, act, w = args[0], args[1], args[2]
    else:
        bias, act, w = None, args[0], args[1]
    assert w.transposed, "mm / addmm expect the weight transposed: x @ w.t()"
    return w._quantized_op(act, w, bias)


@_implements_legacy([aten.detach.default])
def _legacy_detach(func, *args, **kwargs):
    return return_and_correct_aliasing(func, args, kwargs, args[0]._apply_fn_to_data(torch.detach))


@_implements_legacy([aten.clone.default])
def _legacy_clone(func, *args, **kwargs):
    return return_and_correct_aliasing(func, args, kwargs, args[0]._apply_fn_to_data(torch.clone))


@_implements_legacy([aten._to_copy.default])
def _legacy_to_copy(func, *args, **kwargs):
    return return_and_correct_aliasing(func, args, kwargs, args[0].to(*args[1:], **kwargs)._apply_fn_to_data(torch.clone))


@_implements_legacy([aten.t.default])
def _legacy_t(func, *args, **kwargs):
    w = args[0]
    new = w._with(w.int_data, w.scales_and_zeros, transposed=not w.transposed, shape=w.shape[::-1])
    return return_and_correct_aliasing(func, args, kwargs, new)
