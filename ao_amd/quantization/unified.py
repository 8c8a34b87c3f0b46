"""The two quantizer interfaces of the module-swap flows (reference torchao/quantization/unified.py:15-37)."""
import abc

import torch


class Quantizer(abc.ABC):
    """One call: `quantize(model, ...)` returns the quantized model."""

    @abc.abstractmethod
    def quantize(self, model: torch.nn.Module, *args, **kwargs) -> torch.nn.Module:
        ...


class TwoStepQuantizer:
    """`prepare(model)` inserts what calibration or training needs, `convert(model)` produces the quantized model."""

    @abc.abstractmethod
    def prepare(self, model: torch.nn.Module, *args, **kwargs) -> torch.nn.Module:
        ...

    def convert(self, model: torch.nn.Module, *args, **kwargs) -> torch.nn.Module:
        ...
