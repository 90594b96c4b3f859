r"""State shared by all gates (interface of fmoe/gates/base_gate.py:8-25).

A gate maps token rows to ``(top_k_idx, top_k_score)``.  Gates that balance the experts leave an
auxiliary loss behind with :meth:`set_loss`; the training loop collects it with :meth:`get_loss`."""
import torch.nn as nn


class BaseGate(nn.Module):
    def __init__(self, num_expert: int, world_size: int):
        super().__init__()
        self.num_expert, self.world_size = num_expert, world_size
        self.tot_expert = num_expert * world_size   # experts over all workers
        self.loss = None                            # auxiliary loss of the last forward, if any

    def forward(self, x):
        raise NotImplementedError(f"{type(self).__name__} has no forward: BaseGate only holds the shared state")

    def set_loss(self, loss):
        self.loss = loss

    def get_loss(self, clear: bool = True):
        r"""The loss left by the last forward (``None`` without one); ``clear`` forgets it."""
        kept = self.loss
        self.loss = None if clear else kept
        return kept
