r"""MoE modules with the constructor and forward signatures of the reference's
``fmoe.layers`` (fmoe/layers.py), for one worker."""
import math
import os

import torch
import torch.nn as nn

from . import fmoe_native
from .functions import (AllGather, MaskRestore, MaskSelect, MOECache, MOECombine, MOEGather, MOEGatherCombine,
                        MOELinear, MOEScatter, Slice, _PendingCounts, _prepare_forward_ex, _route_launch,
                        _single_worker, ensure_comm, mask_index)
from .gates import NaiveGate


class FMoELinear(nn.Module):
    r"""``num_expert`` linear layers applied to consecutive row segments of the
    input in one grouped GEMM (fmoe/layers.py:16-67).  ``weight`` is
    ``[num_expert, out_feat, in_feat]``, ``bias`` ``[num_expert, out_feat]``."""

    def __init__(self, num_expert: int, in_feat: int, out_feat: int, bias: bool = True, rank: int = 0):
        super().__init__()
        self.num_expert = num_expert
        self.in_feat = in_feat
        self.out_feat = out_feat
        self.rank = rank
        self.weight = nn.Parameter(torch.empty(num_expert, out_feat, in_feat))
        if bias:
            self.bias = nn.Parameter(torch.zeros(num_expert, out_feat))
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()

    def forward(self, inp, fwd_expert_count):
        return MOELinear.apply(inp, fwd_expert_count, self.weight, self.bias)

    def extra_repr(self) -> str:
        return "num_expert={}, in_features={}, out_features={}, bias={}, rank={}".format(
            self.num_expert, self.in_feat, self.out_feat, self.bias is not None, self.rank)

    def reset_parameters(self):
        # Kaiming-uniform over the whole 3-D tensor, bias left at zero
        # (fmoe/layers.py:62-67)
        torch.nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))


def mark_module_parallel_comm(module, comm):
    r"""Tags every parameter with the data-parallel group it is synchronised in
    (fmoe/layers.py:70-76)."""
    for p in module.parameters():
        setattr(p, "dp_comm", comm)


def _own_expert_path(expert_fn, experts):
    """True when ``expert_fn`` is :meth:`FMoE.expert_fn` itself (not overridden, not replaced on the
    instance) and ``experts`` is this package's ``_Expert`` with its own ``forward``: only then may
    the layer skip handing rows and counts through ``expert_fn``."""
    from .transformer import _Expert
    return (getattr(expert_fn, "__func__", None) is FMoE.expert_fn
            and isinstance(experts, _Expert) and type(experts).forward is _Expert.forward)


def _fmoe_general_global_forward(inp, gate, expert_fn, policy_fn, experts, num_expert, world_size,
                                 fused, enable_fuse=False, combine_score=None):
    r"""Route, scatter, run the experts, gather (fmoe/layers.py:79-149).  Returns
    ``(rows in slot order [N*top_k, d], stored_models)``.

    With ``combine_score`` (the gate scores ``[N, top_k]``; not in the reference) the
    gather and the score-weighted sum over each token's ``top_k`` rows run as one pass
    over the experts' output where it lies, and the first result is ``[N, d]``."""
    from .fused_functions import MOEForward

    topk = gate.shape[1] if gate.dim() == 2 else 1
    # On the GPU, with one gate index per (token, k) pair and this package's own expert module
    # behind the layer's own expert_fn, nothing between the gate and the combine needs the expert
    # counts on the host:
    #   * unfused: the grouped GEMMs take the row segments from a table the device builds from the
    #     routing's counts, and the first of them reads the token rows through `pos` in its loader;
    #   * fused pipeline: the counts are read back asynchronously and waited for inside the
    #     pipeline call's binding, where the chunk bounds are computed.
    # Any other expert_fn or expert module gets what the reference gives it: exactly the routed
    # rows and CPU counts it can read (fmoe/layers.py:117-140).
    own = (inp.is_cuda and gate.is_cuda and inp.dim() == 2 and inp.shape[0] > 0
           and gate.numel() == inp.shape[0] * topk and fused and _own_expert_path(expert_fn, experts))
    if own:
        _single_worker(world_size, "count_by_gate")
        counts_dev, pos_buf, slot_to_row = _route_launch(gate, num_expert)
        if not enable_fuse:
            x = experts.routed_forward(inp, pos_buf, slot_to_row, counts_dev, topk)
            if x is not None:
                stored_models = torch.zeros(world_size * num_expert, dtype=torch.bool)
                if combine_score is not None:
                    return MOEGatherCombine.apply(x, slot_to_row, combine_score, inp.shape[0], topk), stored_models
                return MOEGather.apply(x, pos_buf, None, None, stored_models, inp.shape[0] * topk, world_size,
                                       slot_to_row), stored_models
            own = False
    if own:
        # fused pipeline: its sorted buffers hold one row per slot, the routed rows first
        counts_cpu = _PendingCounts(counts_dev).counts_cpu
        pos = pos_buf
        local_expert_count = global_expert_count = all_expert_count = all_global_expert_count = counts_cpu
        fwd_expert_count = counts_cpu
    else:
        (pos, local_expert_count, global_expert_count, all_expert_count, all_global_expert_count,
         fwd_expert_count), slot_to_row = _prepare_forward_ex(gate, num_expert, world_size)

    out_batch_size = inp.shape[0] * topk

    # MOECache (fmoe/functions.py:122-194) decides which experts to shadow on other workers; with
    # one worker it is the identity, so its results are written down directly (the autograd node
    # and its views would only add host time between the routing's read-back and the first GEMM)
    _single_worker(world_size, "MOECache")
    models = [[experts]] if fused else [experts]
    stored_models = torch.zeros(world_size * num_expert, dtype=torch.bool)
    fwd_batch_size = int(pos.shape[0])

    if combine_score is not None and slot_to_row.numel() != out_batch_size:
        raise ValueError("combine_score needs one gate index per (token, k) pair")
    if enable_fuse:
        # (the fused entry point takes pos and top_k; the token index pos // topk is not materialised)
        x = MOEForward.apply(inp, models, None, pos, local_expert_count, global_expert_count,
                             stored_models, fwd_batch_size, out_batch_size, world_size, slot_to_row,
                             combine_score is None)
        if combine_score is not None:
            x = MOEGatherCombine.apply(x, slot_to_row, combine_score, inp.shape[0], topk)
        return x, stored_models

    # ZeroGate hands back N*top_k indices as a 1-D tensor, so the slot count can
    # exceed the token count; the per-token reduction only applies when it does not.
    per_token = slot_to_row if slot_to_row.numel() == inp.shape[0] * topk else None
    x = MOEScatter.apply(inp, pos // topk, local_expert_count, global_expert_count, stored_models,
                         fwd_batch_size, world_size, per_token, topk)
    x = expert_fn(x, models, fwd_expert_count, num_expert)
    if combine_score is not None:
        return MOEGatherCombine.apply(x, slot_to_row, combine_score, inp.shape[0], topk), stored_models
    x = MOEGather.apply(x, pos, local_expert_count, global_expert_count, stored_models,
                        out_batch_size, world_size,
                        slot_to_row if slot_to_row.numel() == out_batch_size else None)
    return x, stored_models


class FMoE(nn.Module):
    r"""General MoE layer (fmoe/layers.py:151-326).

    * ``num_expert``: experts on this worker; ``world_size`` must be 1 here.
    * ``top_k``: experts per token; ``gate``: a class from :mod:`fastermoe_amd.gates`.
    * ``expert``: a module class (or list of classes) instantiated per expert and
      called on row slices; ``None`` means the subclass provides a fused
      ``self.experts`` taking ``(rows, fwd_expert_count)``.
    * ``enable_fuse`` (or ``FMOE_ENABLE_FUSE=1``): run scatter, the expert MLP and
      gather as one chunked, stream-overlapped pipeline.
    """

    def __init__(self, num_expert=32, d_model=1024, world_size=1, mp_group=None, moe_group=None,
                 top_k=2, gate=NaiveGate, expert=None, gate_hook=None, policy_fn=None, mask=None,
                 mask_dict=None, enable_fuse=False):
        super().__init__()
        if world_size != 1:
            raise NotImplementedError("fastermoe_amd implements the single-GPU path: world_size must be 1")
        self.d_model, self.top_k, self.world_size = d_model, top_k, world_size
        self.mp_group, self.moe_group = mp_group, moe_group
        self.mp_size, self.mp_rank = (1, 0) if mp_group is None else (mp_group.size(), mp_group.rank())
        if self.mp_size != 1:
            raise NotImplementedError("model-parallel groups larger than 1 are not supported")

        # `expert`: one module class for every expert, a list with one class per expert (its length
        # then is the expert count), or None when the sub-class sets a fused `self.experts` itself
        classes = expert if type(expert) is list else (None if expert is None else [expert] * num_expert)
        self.experts_fused = classes is None
        if classes is not None:
            num_expert = len(classes)
            self.experts = nn.ModuleList([cls(d_model) for cls in classes])
        self.num_expert = num_expert

        self.gate = gate(d_model, num_expert, world_size, top_k)
        self.policy_fn = policy_fn
        if hasattr(self.gate, "stored_models"):   # gates that shadow experts take the policy too
            self.gate.policy_fn = policy_fn
        self.gate_hook, self.mask, self.mask_dict = gate_hook, mask, mask_dict

        self.enable_fuse = enable_fuse or os.environ.get("FMOE_ENABLE_FUSE", "0") == "1"
        if self.enable_fuse and not self.experts_fused:
            raise AssertionError("enable_fuse needs the fused experts module of a sub-class")

    def expert_fn(self, inp, models, fwd_expert_count, num_expert):
        r"""Runs the experts on expert-sorted rows (fmoe/layers.py:222-255): the fused expert
        module in one call, or one module per expert on its segment of the rows.  One worker, so
        ``fwd_expert_count`` is a single row of counts and ``models`` holds this worker's experts."""
        if fwd_expert_count.numel() != num_expert or len(models) != 1:
            raise NotImplementedError("expert_fn: one worker only")
        experts = models[0]
        if not experts:
            raise ValueError(f"Experts is {experts} yet counts is {fwd_expert_count}")
        if self.experts_fused:
            return experts[0](inp, fwd_expert_count.view(-1))
        sizes = [int(n) for n in fwd_expert_count.view(-1).tolist()]
        if sum(sizes) > inp.shape[0]:
            raise ValueError(f"expert counts {sizes} add up to more than the {inp.shape[0]} rows given")
        # split (not slices): its backward is one concatenation, not a zero-filled copy per expert
        pieces = inp.split(sizes + [inp.shape[0] - sum(sizes)], dim=0)
        out = [experts[i](piece) for i, piece in enumerate(pieces[:-1])]
        if pieces[-1].shape[0]:
            out.append(out[0].new_zeros(pieces[-1].shape[0], *out[0].shape[1:]) if out else pieces[-1])
        return torch.cat(out, dim=0)

    def mark_parallel_comm(self, expert_dp_comm="none"):
        r"""Tags the experts' parameters with ``expert_dp_comm`` and the gate's with "moe"
        (fmoe/layers.py:257-270); sub-classes call it at the end of their constructor."""
        experts = getattr(self, "experts", None)
        if experts is not None:
            for module in (experts if isinstance(experts, list) else [experts]):
                mark_module_parallel_comm(module, expert_dp_comm)
        mark_module_parallel_comm(self.gate, "moe")

    def _mask_kernels_apply(self, inp, gate_top_k_idx, gate_score):
        """The index-kernel form of the mask path needs GPU tensors, one gate index and one score per
        (token, k) pair and mask_dict values that are one row of d_model each."""
        n = inp.shape[0]
        return (inp.is_cuda and inp.is_floating_point() and inp.dtype != torch.float64
                and torch.is_tensor(gate_score) and gate_score.dtype == inp.dtype
                and gate_top_k_idx.numel() == gate_score.numel() == n * self.top_k
                and self.mask.numel() == n
                and all(torch.is_tensor(v) and v.numel() == self.d_model for v in self.mask_dict.values())
                and os.environ.get("FMOE_MASK_KERNELS", "1") != "0")

    def _forward_masked(self, inp, gate_top_k_idx, gate_score):
        r"""fmoe/layers.py:288-322 without boolean indexing: the kept tokens' rows, gate indices and
        scores are gathered over an index built by one routing call, go through the experts and the
        folded combine, and one kernel restores the token order, writing
        ``sum_j score[t,j] * mask_dict[mask[t]]`` for the masked tokens (all ``top_k`` slots of a
        masked token hold the same ``mask_dict`` row)."""
        n, k, d = inp.shape[0], self.top_k, self.d_model
        mask = self.mask.view(-1).to(inp.device)
        keep_idx, token_to_row = mask_index(mask)
        score = gate_score.reshape(n, k)
        inp_k = MaskSelect.apply(inp, keep_idx, token_to_row)
        score_k = MaskSelect.apply(score, keep_idx, token_to_row)
        idx_k = fmoe_native.gather_rows(gate_top_k_idx.reshape(n, k).contiguous().view(torch.float64),
                                        keep_idx).view(torch.int64)
        if os.environ.get("FMOE_FOLD_COMBINE", "1") != "0":
            y_k, _ = _fmoe_general_global_forward(
                inp_k, idx_k, self.expert_fn, self.policy_fn, self.experts, self.num_expert, self.world_size,
                self.experts_fused, self.enable_fuse, score_k)
        else:
            rows, _ = _fmoe_general_global_forward(
                inp_k, idx_k, self.expert_fn, self.policy_fn, self.experts, self.num_expert, self.world_size,
                self.experts_fused, self.enable_fuse)
            y_k = MOECombine.apply(rows.reshape(-1, d), score_k.reshape(-1, 1, k), inp_k.shape[0], k)
        # which mask_dict row a masked token takes (-1: its mask value has no entry -> zero row)
        keys = sorted(int(key) for key in self.mask_dict)
        fill = fill_row = scale = None
        if keys:
            fill = torch.cat([self.mask_dict[key].reshape(1, d) for key in keys]).to(device=inp.device, dtype=inp.dtype)
            lut = torch.full((max(keys) + 2,), -1, dtype=torch.int64, device=inp.device)
            lut[torch.tensor(keys, device=inp.device)] = torch.arange(len(keys), device=inp.device)
            lut[0] = -1
            fill_row = lut[mask.clamp(min=0, max=max(keys) + 1)]
            scale = score.sum(dim=-1).contiguous()
        return MaskRestore.apply(y_k, keep_idx, token_to_row, scale, fill, fill_row)

    def forward(self, inp):
        r"""Gate, route through the experts, and combine each token's ``top_k``
        expert outputs with the gate scores (fmoe/layers.py:272-326)."""
        if self.world_size > 1:
            ensure_comm(inp, self.moe_group)
        if self.mp_size > 1:
            inp = Slice.apply(inp, self.mp_rank, self.mp_size, self.mp_group)

        gate_top_k_idx, gate_score = self.gate(inp)
        if self.gate_hook is not None:
            self.gate_hook(gate_top_k_idx, gate_score, None)

        masked = self.mask is not None and self.mask_dict is not None
        if masked and self._mask_kernels_apply(inp, gate_top_k_idx, gate_score):
            x = self._forward_masked(inp, gate_top_k_idx, gate_score)
            if self.mp_size > 1:
                x = AllGather.apply(x, self.mp_rank, self.mp_size, self.mp_group)
            return x
        if masked:
            mask = self.mask.view(-1)
            inp = inp[mask == 0, :]
            gate_top_k_idx = gate_top_k_idx[mask == 0, :]

        # Without a mask the gather and the combine with the gate scores are one pass
        # (FMOE_FOLD_COMBINE=0 keeps them apart, as in the reference).
        fold = (not masked and inp.is_cuda and inp.is_floating_point() and torch.is_tensor(gate_score)
                and gate_score.dtype == inp.dtype and gate_top_k_idx.dim() == 2
                and gate_score.numel() == gate_top_k_idx.numel() == inp.shape[0] * self.top_k
                and os.environ.get("FMOE_FOLD_COMBINE", "1") != "0")
        fwd, _stored_models = _fmoe_general_global_forward(
            inp, gate_top_k_idx, self.expert_fn, self.policy_fn, self.experts, self.num_expert,
            self.world_size, self.experts_fused, self.enable_fuse,
            gate_score.reshape(inp.shape[0], self.top_k) if fold else None)
        if fold:
            if self.mp_size > 1:
                fwd = AllGather.apply(fwd, self.mp_rank, self.mp_size, self.mp_group)
            return fwd

        if masked:
            fwd = fwd.view(-1, self.top_k, self.d_model)
            x = torch.zeros(mask.shape[0], self.top_k, self.d_model, device=fwd.device, dtype=fwd.dtype)
            x[mask == 0] = fwd
            for k, v in self.mask_dict.items():
                x[mask == k] = v
        else:
            x = fwd.view(-1, self.top_k, self.d_model)

        gate_score = gate_score.view(x.shape[0], 1, self.top_k)
        if x.is_cuda and gate_score.dtype == x.dtype and x.is_floating_point():
            # the bmm of fmoe/layers.py:321-322 as a streaming kernel
            x = MOECombine.apply(x.reshape(-1, self.d_model), gate_score, x.shape[0], self.top_k)
        else:
            x = torch.bmm(gate_score, x).reshape(-1, self.d_model)

        if self.mp_size > 1:
            x = AllGather.apply(x, self.mp_rank, self.mp_size, self.mp_group)
        return x
