r"""Capacity helpers of the gates (fmoe/gates/utils.py:9-26)."""
import math

import torch

from .. import fmoe_native
from ..functions import count_by_gate


def limit_by_capacity(topk_idx, num_expert, world_size, capacity):
    r"""Caps every expert at ``capacity`` slots and rewrites the gate indices of the
    slots that do not fit to -1 (slots with the lowest flat index win).
    Returns ``(new_local_expert_count, new_global_expert_count, pruned_idx)``.
    The reference unpacks three values from ``count_by_gate``'s five
    (fmoe/gates/utils.py:14); the five-tuple is what is used here."""
    with torch.no_grad():
        cap = torch.full((num_expert,), int(capacity), dtype=torch.int32, device=topk_idx.device)
        _pos, _lec, _all_ec, gec, _all_gec = count_by_gate(topk_idx, num_expert, world_size,
                                                           require_pos=False)
        new_gec = fmoe_native.limit_by_capacity(gec, cap, num_expert, world_size)
        new_lec = new_gec  # one worker: nothing to exchange
        pruned = fmoe_native.prune_gate_by_capacity(topk_idx.contiguous(), new_lec.to(torch.int32),
                                                    num_expert, world_size)
    return new_lec, new_gec, pruned


def capacity_of(rates, training, n_tokens):
    r"""Slots an expert may take: ``rates = (train, eval)`` factors of the token count, rounded up
    (fmoe/gates/gshard_gate.py:36-37, switch_gate.py:40-41)."""
    return math.ceil(rates[0 if training else 1] * n_tokens)
