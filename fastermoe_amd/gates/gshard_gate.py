r"""GShard top-2 gate with capacity and random second-expert routing
(fmoe/gates/gshard_gate.py:11-46)."""
import math

import torch
import torch.nn.functional as F

from .naive_gate import NaiveGate
from .utils import limit_by_capacity


class GShardGate(NaiveGate):
    def __init__(self, d_model, num_expert, world_size, topk=2, capacity=(1.2, 2.4),
                 random_routing=True):
        assert topk == 2, "topk should be 2 in gshard"
        super().__init__(d_model, num_expert, world_size, top_k=2)
        self.capacity = capacity
        # the reference stores True whatever is passed (gshard_gate.py:17)
        self.random_routing = True

    def forward(self, x):
        topk_idx, topk_val, logits = super().forward(x, return_all_scores=True)

        n_tokens = logits.shape[0]
        top1_idx = topk_idx.view(-1, self.top_k)[:, 0]
        c_e = torch.scatter_add(
            torch.zeros(self.tot_expert, device=top1_idx.device), 0, top1_idx,
            torch.ones_like(top1_idx, dtype=torch.float)) / n_tokens
        m_e = torch.mean(F.softmax(logits, dim=1), dim=0)
        self.set_loss(torch.mean(c_e * m_e) * (self.num_expert ** 2))

        cap_rate = self.capacity[0 if self.training else 1]
        capacity = math.ceil(cap_rate * x.shape[0])
        _new_lec, _new_gec, topk_idx = limit_by_capacity(
            topk_idx, self.num_expert, self.world_size, capacity)

        if self.random_routing:
            rand_routing_prob = torch.rand(logits.size(0), device=x.device)
            mask = 2 * topk_val[:, 1] < rand_routing_prob
            topk_idx[:, 1].masked_fill_(mask, -1)
        return topk_idx, topk_val
