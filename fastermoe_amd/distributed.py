r"""Placeholder for the reference's ``fmoe.distributed`` (fmoe/distributed.py:11-121).

Gradient synchronisation across data-parallel groups needs several processes and
is outside the single-GPU path this package implements; the name is kept so that
``from fastermoe_amd import DistributedGroupedDataParallel`` resolves."""
import torch.nn as nn


class DistributedGroupedDataParallel(nn.Module):
    def __init__(self, module, *args, **kwargs):
        super().__init__()
        raise NotImplementedError(
            "DistributedGroupedDataParallel: multi-process training is not part of "
            "fastermoe_amd (single-GPU MoE path only)")
