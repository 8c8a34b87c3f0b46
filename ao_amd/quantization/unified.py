"""Quantizer base classes (reference torchao/quantization/unified.py:15-37)."""
from abc import ABC, abstractmethod
from typing import Any

import torch


class Quantizer(ABC):
    """One-step flow: `quantize(model)` returns the quantized model."""

    @abstractmethod
    def quantize(self, model: torch.nn.Module, *args: Any, **kwargs: Any) -> torch.nn.Module:
        pass


class TwoStepQuantizer:
    """Flow with a calibration or training phase between `prepare` and `convert`."""

    @abstractmethod
    def prepare(self, model: torch.nn.Module, *args: Any, **kwargs: Any) -> torch.nn.Module:
        pass

    def convert(self, model: torch.nn.Module, *args: Any, **kwargs: Any) -> torch.nn.Module:
        pass
