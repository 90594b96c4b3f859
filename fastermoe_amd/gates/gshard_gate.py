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

        # Balance loss.  The reference derives "top_k" as topk_idx.shape[0] // n_tokens, which is 1
        # for the [n_tokens, 2] index tensor, so its "top-1" list is the flattened list of BOTH
        # choices of every token (gshard_gate.py:23-31): c_e is the number of (token, choice)
        # slots that name expert e, over the number of tokens.
        n_tokens = logits.shape[0]
        c_e = torch.bincount(topk_idx.reshape(-1), minlength=self.tot_expert).to(torch.float) / n_tokens
        m_e = F.softmax(logits, dim=1).mean(dim=0)
        self.set_loss((c_e * m_e).mean() * (self.num_expert ** 2))

        cap_rate = self.capacity[0 if self.training else 1]
        capacity = math.ceil(cap_rate * x.shape[0])
        _new_lec, _new_gec, topk_idx = limit_by_capacity(
            topk_idx, self.num_expert, self.world_size, capacity)

        if self.random_routing:
            rand_routing_prob = torch.rand(logits.size(0), device=x.device)
            mask = 2 * topk_val[:, 1] < rand_routing_prob
            topk_idx[:, 1].masked_fill_(mask, -1)
        return topk_idx, topk_val
