r"""fastermoe_amd: the single-GPU Mixture-of-Experts path of FasterMoE's ``fmoe``
package on MI355X (gfx950), with hand-written HIP kernels behind the same
Python API (fmoe/__init__.py:5-7).  ``import fastermoe_amd as fmoe``."""
from .layers import FMoE, FMoELinear
from .transformer import FMoETransformerMLP
from .distributed import DistributedGroupedDataParallel

__all__ = ["FMoE", "FMoELinear", "FMoETransformerMLP", "DistributedGroupedDataParallel"]
