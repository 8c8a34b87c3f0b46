"""ao_amd: MI355X (gfx950) implementation of torchao's weight-only quantized linear path.

    from ao_amd import quantize_, int4_weight_only
    quantize_(model, int4_weight_only(group_size=64))

The public surface mirrors torchao 0.3.1 (torchao/__init__.py:31-41): `quantize` / `quantize_`,
`int4_weight_only`, `fp6_llm_weight_only`, the `quantization`, `dtypes`, `ops` and `prototype.quant_llm`
sub-packages.  Everything runs in hand-written HIP kernels; tensors must be on the GPU.
"""
__version__ = "0.1.0"

from . import dtypes, ops, quantization  # noqa: F401
from .quantization import (  # noqa: F401
    fp6_llm_weight_only,
    int4_weight_only,
    int8_weight_only,
    quant_llm_fpx_weight_only,
    quantize,
    quantize_,
)

__all__ = ["dtypes", "ops", "quantization", "quantize", "quantize_", "int4_weight_only", "int8_weight_only", "fp6_llm_weight_only",
           "quant_llm_fpx_weight_only"]
