"""Import alias: `torchao` resolves to `ao_amd`, so code written against torchao 0.3.1 runs unchanged on the HIP kernels.

    from torchao.quantization import quantize_, int4_weight_only
    import torchao; torchao.ops.quant_llm_linear(...)

Every `torchao.<sub>` module below IS the `ao_amd.<sub>` module (same object in sys.modules), the names follow
torchao/__init__.py:31-41 and the sub-packages the int4 / FP6 weight-only path touches.  This directory only takes
effect when it is importable ahead of (or instead of) an installed torchao: put the repository root on sys.path.
"""
import importlib
import sys

import ao_amd

__version__ = ao_amd.__version__

_SUBMODULES = [
    "quantization", "quantization.quant_api", "quantization.quant_primitives", "quantization.GPTQ", "quantization.unified",
    "quantization.utils", "dtypes", "dtypes.affine_quantized_tensor", "dtypes.utils", "ops", "utils", "prototype",
    "prototype.quant_llm", "prototype.quant_llm.quant_llm", "prototype.hqq", "prototype.hqq.hqq_tinygemm_linear",
    "prototype.hqq.mixed_mm", "_models", "_models.llama", "_models.llama.model", "_models.llama.generate",
]
for _name in _SUBMODULES:
    _mod = importlib.import_module("ao_amd." + _name)
    sys.modules[__name__ + "." + _name] = _mod
    if "." not in _name:
        globals()[_name] = _mod

from ao_amd import *  # noqa: E402,F401,F403
from ao_amd import __all__  # noqa: E402,F401
