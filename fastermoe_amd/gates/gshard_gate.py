r"""GShard top-2 gate: balance loss, per-expert capacity, random drop of the second choice
(behaviour of fmoe/gates/gshard_gate.py:11-46)."""
import torch

from .naive_gate import NaiveGate
from .utils import capacity_of, limit_by_capacity


class GShardGate(NaiveGate):
    def __init__(self, d_model, num_expert, world_size, topk=2, capacity=(1.2, 2.4),
                 random_routing=True):
        if topk != 2:
            raise AssertionError("topk should be 2 in gshard")
        super().__init__(d_model, num_expert, world_size, top_k=2)
        self.capacity = capacity
        # the reference stores True whatever is passed (gshard_gate.py:17)
        self.random_routing = True

    def _balance_loss(self, topk_idx, logits):
        # The reference derives "top_k" as topk_idx.shape[0] // n_tokens, which is 1 for the
        # [n_tokens, 2] index tensor, so its "top-1" list is the flattened list of BOTH choices of
        # every token (gshard_gate.py:23-31): c_e is the number of (token, choice) slots that name
        # expert e over the number of tokens, m_e the mean softmax probability of expert e.
        n_tokens = logits.shape[0]
        c_e = torch.bincount(topk_idx.reshape(-1), minlength=self.tot_expert).to(torch.float) / n_tokens
        m_e = torch.softmax(logits, dim=1).mean(dim=0)
        return (c_e * m_e).mean() * (self.num_expert ** 2)

    def forward(self, x):
        topk_idx, topk_val, logits = super().forward(x, return_all_scores=True)
        self.set_loss(self._balance_loss(topk_idx, logits))

        cap = capacity_of(self.capacity, self.training, x.shape[0])
        topk_idx = limit_by_capacity(topk_idx, self.num_expert, self.world_size, cap)[2]

        if self.random_routing:
            # the second choice survives with probability min(1, 2 * its score)
            draw = torch.rand(logits.shape[0], device=x.device)
            topk_idx[:, 1].masked_fill_(draw > 2 * topk_val[:, 1], -1)
        return topk_idx, topk_val
