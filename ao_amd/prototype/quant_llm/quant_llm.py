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

from ... import ops
from ...dtypes.utils import PackedWeightBase

__all__ = ["to_scaled_tc_fpx", "from_scaled_tc_fpx", "QuantLlmLinearWeight", "quant_llm_fpx_weight_only",
           "fp6_llm_weight_only"]

# the formats the reference kernel dispatches (torchao/csrc/cuda/fp6_llm/fp6_linear.cu:173-184)
_FORMATS = {(3, 2), (2, 3), (2, 2), (3, 1)}


def _check_fp6(ebits: int, mbits: int):
    if (ebits, mbits) not in _FORMATS:
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


class QuantLlmLinearWeight(PackedWeightBase):
    """Weight of a linear layer stored as packed FPx bytes + fp16 row scales (reference :348-417: same constructor
    arguments, attribute names and serialised state).

    `fpx_data` / `scale` are the reference's interchange format bit for bit; the wave64 kernel reads a rearrangement
    of the same bits that is made on first use (`native()`) and is never part of the state."""

    _inner = ("fpx_data", "scale")
    _plain = ("ebits", "mbits")

    @staticmethod
    def __new__(cls, fpx_data: Tensor, scale: Tensor, ebits: int, mbits: int):
        torch._check(fpx_data.dim() == 2 and fpx_data.dtype is torch.uint8,
                     lambda: f"fpx_data must be a 2d uint8 tensor, got {fpx_data.dtype} with {fpx_data.dim()} dims")
        rows, row_bytes = fpx_data.shape
        logical = (rows, row_bytes * 8 // (1 + ebits + mbits))   # the floating-point weight this stands for
        return Tensor._make_wrapper_subclass(cls, logical, device=fpx_data.device, requires_grad=False)

    def __init__(self, fpx_data: Tensor, scale: Tensor, ebits: int, mbits: int):
        self.fpx_data, self.scale, self.ebits, self.mbits = fpx_data, scale, ebits, mbits
        self._native = None

    @property
    def nbits(self) -> int:
        return 1 + self.ebits + self.mbits

    def native(self) -> Tensor:
        """The kernel's tile order of `fpx_data`, built once per tensor object."""
        if self._native is None:
            self._native = ops.fp6_repack(self.fpx_data, self.nbits)
        return self._native

    @classmethod
    def from_float(cls, input_float: Tensor, ebits: int, mbits: int):
        return cls(*to_scaled_tc_fpx(input_float, ebits, mbits), ebits, mbits)

    def dequantize(self, output_dtype=None):
        values = from_scaled_tc_fpx(self.fpx_data, self.ebits, self.mbits, self.scale)
        return values.to(torch.get_default_dtype() if output_dtype is None else output_dtype)

    def __repr__(self):
        return (f"{type(self).__name__}(dtype=fp{self.nbits}_e{self.ebits}m{self.mbits}, shape={tuple(self.shape)}, "
                f"device={self.device}, requires_grad={self.requires_grad})")


@QuantLlmLinearWeight.implements(torch.nn.functional.linear)
def _fpx_linear(act, weight, bias=None):
    """fp16 product on the HIP kernel whatever the activation's dtype, result in that dtype (reference :419-445; its
    split-K factor comes from a table tuned for NVIDIA SM counts, :212-345, while the gfx950 kernel sizes its own K
    split from the shape)."""
    assert isinstance(weight, QuantLlmLinearWeight)
    out_features, in_features = weight.shape
    rows = act.reshape(-1, in_features).to(torch.float16)
    out = ops.fp6_linear_native(weight.ebits, weight.mbits, rows, weight.native(), weight.scale)
    if bias is not None:
        out += bias
    return out.view(*act.shape[:-1], out_features).to(act.dtype)


def quant_llm_fpx_weight_only(ebits: int, mbits: int):
    """Weights whose shape the kernel cannot take (in % 64 or out % 256) are left in floating point."""

    def apply_quant_llm(weight: Tensor) -> Tensor:
        out_features, in_features = weight.shape
        if in_features % 64 or out_features % 256:
            return weight
        return QuantLlmLinearWeight.from_float(weight, ebits, mbits)

    return apply_quant_llm


def fp6_llm_weight_only():
    return quant_llm_fpx_weight_only(3, 2)
