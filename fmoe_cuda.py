r"""``import fmoe_cuda`` (also ``import fmoe_cuda as fmoe_native``, fmoe/gates/utils.py:6): the
operator module the reference builds from cuda/fmoe_cuda.cpp:105-130, served here by
:mod:`fastermoe_amd.fmoe_native` on top of ``libfmoe_hip.so``.  The module object is the same."""
import sys

from fastermoe_amd import fmoe_native as _native

sys.modules[__name__] = _native
