r"""Gates (fmoe/gates/__init__.py).  The topology-aware, neighbour and BASE-layer
gates of the reference need several workers and are not part of this package."""
from .zero_gate import ZeroGate
from .naive_gate import NaiveGate
from .noisy_gate import NoisyGate
from .gshard_gate import GShardGate
from .switch_gate import SwitchGate
