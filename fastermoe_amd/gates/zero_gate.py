r"""Gate that names expert 0 for every choice of every token, with equal scores
(behaviour of fmoe/gates/zero_gate.py:11-30); a fixture for tests of the layer."""
import torch

from .base_gate import BaseGate


class ZeroGate(BaseGate):
    def __init__(self, d_model, num_expert, world_size, top_k=2):
        # d_model is accepted for the common constructor signature gate(d_model, num_expert, world_size, top_k)
        super().__init__(num_expert, world_size)
        self.top_k = top_k

    def forward(self, inp):
        n_tokens, k = inp.shape[0], self.top_k
        # a FLAT index tensor [n_tokens * k] and float32 scores [n_tokens, 1, k], as the reference returns
        idx = inp.new_zeros(n_tokens * k, dtype=torch.int64)
        score = torch.full((n_tokens, 1, k), 1.0, device=inp.device) / k
        return idx, score
