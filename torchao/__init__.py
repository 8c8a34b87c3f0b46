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

import pkgutil


def _submodules():
    """every module of the ao_amd package tree (packages before their members), private helpers excluded"""
    names = []
    for info in pkgutil.walk_packages(ao_amd.__path__, "ao_amd."):
        rel = info.name[len("ao_amd."):]
        if any(part.startswith("_") and part != "_models" for part in rel.split(".")) or rel.startswith(("csrc", "lib")):
            continue
        names.append(rel)
    return names


for _name in _submodules():
    _mod = importlib.import_module("ao_amd." + _name)
    sys.modules[__name__ + "." + _name] = _mod
    if "." not in _name:
        globals()[_name] = _mod

from ao_amd import *  # noqa: E402,F401,F403
from ao_amd import __all__  # noqa: E402,F401
