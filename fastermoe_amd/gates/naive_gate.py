r"""Top-k of a linear layer (fmoe/gates/naive_gate.py:11-42)."""
import torch.nn as nn

from ..functions import gate_linear_topk, gate_topk
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
        # torch.topk(sorted=False) in the reference; here one kernel that also leaves the expert
        # histogram and the positions for the layer's routing step (order of the k choices: by logit)
        if return_all_scores:
            logits = self.gate(inp)
            top_idx, top_val = gate_topk(logits, self.top_k)
            return top_idx, top_val.view(-1, self.top_k), logits
        # nobody asks for the logits: for small expert counts the linear layer runs inside the same
        # kernel and they never reach memory
        top_idx, top_val = gate_linear_topk(inp, self.gate, self.top_k)
        return top_idx, top_val.view(-1, self.top_k)
