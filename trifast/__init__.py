"""Drop-in import name: ``import trifast`` resolves to the MI355X implementation.

``trifast.triangle_attention`` and the submodules ``trifast.torch``,
``trifast.utils``, ``trifast.equiv``, ``trifast.tune`` mirror the reference package layout
(reference src/trifast/__init__.py:1-3); the code lives in ``trifast_amd``.
"""

import sys as _sys

import trifast_amd as _impl
from trifast_amd import equiv as _equiv_mod
from trifast_amd import torch as _torch_mod
from trifast_amd import tuner as _tuner_mod
from trifast_amd import utils as _utils_mod
from trifast_amd.torch import triangle_attention

__version__ = _impl.__version__

# submodule aliases: `import trifast.torch`, `from trifast.utils import gen_tensors`
for _name, _mod in (("torch", _torch_mod), ("utils", _utils_mod), ("autotune", _tuner_mod), ("equiv", _equiv_mod)):
    _sys.modules[f"{__name__}.{_name}"] = _mod
    globals()[_name] = _mod

__all__ = ["triangle_attention"]
