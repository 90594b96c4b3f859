r"""Top-k of a linear layer (fmoe/gates/naive_gate.py:11-42)."""
import torch.nn as nn

from ..functions import gate_topk
from .base_gate import BaseGate


class NaiveGate(BaseGate):
    r"""Returns the top-k expert indices and, as the score, the RAW top-k logits:
    the reference computes a softmax over them and then returns the logits
    (fmoe/gates/naive_gate.py:38-42), and so does this gate."""

    def __init__(self, d_model, num_expert, world_size, top_k=2):
        super().__init__(num_expert, world_size)
        self.gate = nn.Linear(d_model, self.tot_expert)
        self.top_k = top_k

    def forward(self, inp, return_all_scores=False):
        logits = self.gate(inp)
        # torch.topk(sorted=False) in the reference; here one kernel that also leaves the expert
        # histogram and the positions for the layer's routing step (order of the k choices: by logit)
        top_idx, top_val = gate_topk(logits, self.top_k)
        top_val = top_val.view(-1, self.top_k)
        if return_all_scores:
            return top_idx, top_val, logits
        return top_idx, top_val
