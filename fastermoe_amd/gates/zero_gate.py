r"""Gate that sends everything to expert 0 (fmoe/gates/zero_gate.py:11-30)."""
import torch

from .base_gate import BaseGate


class ZeroGate(BaseGate):
    def __init__(self, _1, num_expert, world_size, top_k=2):
        super().__init__(num_expert, world_size)
        self.top_k = top_k

    def forward(self, inp):
        idx = torch.zeros(inp.shape[0] * self.top_k, dtype=torch.int64, device=inp.device)
        score = torch.ones(inp.shape[0] * self.top_k, device=inp.device) / self.top_k
        return idx, score.reshape(-1, 1, self.top_k)
