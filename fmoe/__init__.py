r"""``import fmoe`` for code written against FasterMoE's package name.

Every module of :mod:`fastermoe_amd` that has a counterpart in the reference's ``fmoe``
package (fmoe/__init__.py:5-7, fmoe/functions.py, fmoe/fused_functions.py, fmoe/layers.py,
fmoe/transformer.py, fmoe/distributed.py, fmoe/gates/*) is registered under the reference's
module path, so ``from fmoe.gates import GShardGate``, ``from fmoe.functions import
prepare_forward`` or ``import fmoe.gates.utils`` resolve to the MI355X implementation.  The
modules are the same objects, not copies: ``fmoe.layers is fastermoe_amd.layers``.
"""
import importlib
import sys

import fastermoe_amd as _impl
from fastermoe_amd import DistributedGroupedDataParallel, FMoE, FMoELinear, FMoETransformerMLP

_MODULES = ("layers", "transformer", "functions", "fused_functions", "distributed", "gates", "gates.base_gate",
            "gates.naive_gate", "gates.gshard_gate", "gates.switch_gate", "gates.zero_gate", "gates.noisy_gate",
            "gates.utils")
for _name in _MODULES:
    _mod = importlib.import_module("fastermoe_amd." + _name)
    sys.modules[__name__ + "." + _name] = _mod
    if "." not in _name:
        globals()[_name] = _mod
del _name, _mod

__all__ = ["FMoE", "FMoELinear", "FMoETransformerMLP", "DistributedGroupedDataParallel"]
