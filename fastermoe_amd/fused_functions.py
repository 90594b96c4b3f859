r"""Fused MoE forward (fmoe/fused_functions.py): scatter, the two-linear expert MLP
and gather as one chunked, stream-overlapped pipeline.

Differences from the reference, all deliberate: the activation is the expert
module's own (exact GELU, ReLU or none) instead of a hard-coded ReLU
(cuda/fused_compute.cuh:20-44), biases are honoured, and the weight gradients
flow through autograd instead of being written into ``param.grad`` from C++
(cuda/fused_compute.cu:94-105).
"""
import os

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.autograd import Function

from . import _lib, fmoe_native


def _activation_code(act):
    if act is None or isinstance(act, nn.Identity):
        return _lib.ACT_NONE
    if isinstance(act, nn.ReLU) or act in (F.relu, torch.relu):
        return _lib.ACT_RELU
    if isinstance(act, nn.GELU):
        if getattr(act, "approximate", "none") != "none":
            raise NotImplementedError("the fused path implements the exact (erf) GELU only")
        return _lib.ACT_GELU
    if act is F.gelu:
        return _lib.ACT_GELU
    raise NotImplementedError(
        f"the fused expert pipeline supports GELU, ReLU or no activation, got {act!r}; "
        "use enable_fuse=False for other activations")


def fuse_chunks():
    r"""Number of pipeline chunks: ``FMOE_FUSE_GRAN`` when set (the variable of
    cuda/fused_compute.cu:21-28, whose default there is 4); unset: 0, which lets the library take
    up to 4 chunks but no more than leave every chunk enough tiles to fill the chip."""
    gran = os.environ.get("FMOE_FUSE_GRAN")
    return 0 if gran is None else max(1, int(gran))


class _FusedExpertMLP(Function):
    @staticmethod
    def forward(ctx, inp, w1, b1, w2, b2, pos, slot_to_row, expert_count, top_k, activation, n_chunks,
                slot_order=True):
        inp = inp.contiguous()
        out, buf_in, buf_pre, buf_mid = fmoe_native.fused_mlp_forward(
            inp, pos, slot_to_row, expert_count, w1, b1, w2, b2, top_k, activation, n_chunks, slot_order)
        # without a sorted copy of the input (the first GEMM gathered the rows itself) the backward
        # rebuilds one from the input, which autograd keeps alive anyway
        ctx.save_for_backward(pos, slot_to_row, expert_count, w1, b1, w2, b2, buf_in if buf_in is not None else inp,
                              buf_pre, buf_mid)
        ctx.moe_args = inp.shape[0], top_k, activation, n_chunks, slot_order, buf_in is None
        return out

    @staticmethod
    def backward(ctx, grad_out):
        pos, slot_to_row, expert_count, w1, b1, w2, b2, buf_in, buf_pre, buf_mid = ctx.saved_tensors
        n_tokens, top_k, activation, n_chunks, slot_order, regather = ctx.moe_args
        grad_inp, gw1, gb1, gw2, gb2 = fmoe_native.fused_mlp_backward(
            grad_out.contiguous(), pos, slot_to_row, expert_count, w1, b1, w2, b2,
            None if regather else buf_in, buf_pre, buf_mid,
            n_tokens, top_k, activation, n_chunks, slot_order, inp=buf_in if regather else None)
        return grad_inp, gw1, gb1, gw2, gb2, None, None, None, None, None, None, None


class MOEForward:
    r"""Drop-in for the reference's ``MOEForward`` autograd Function
    (fmoe/fused_functions.py:12-61): ``MOEForward.apply(...)`` takes the same
    arguments (plus an optional ``slot_to_row``) and returns the rows in slot
    order.  ``models[0][0]`` is the fused expert module (two ``FMoELinear`` and an
    activation)."""

    @staticmethod
    def apply(inp, models, pos_s, pos_g, local_expert_count, global_expert_count, stored_models,
              fwd_batch_size, out_batch_size, world_size, slot_to_row=None, slot_order=True):
        r"""``slot_order=False`` (not in the reference): skip the copy back to slot order and
        return the experts' output rows in expert-sorted order, for
        :class:`fastermoe_amd.functions.MOEGatherCombine`."""
        if world_size != 1:
            raise NotImplementedError("MOEForward: one worker only")
        experts = models[0][0]
        top_k = out_batch_size // max(inp.shape[0], 1) if inp.shape[0] else 1
        if slot_to_row is None or slot_to_row.numel() != out_batch_size:
            slot_to_row = fmoe_native.invert_index(pos_g, out_batch_size)
        act = _activation_code(experts.activation)
        return _FusedExpertMLP.apply(inp, experts.htoh4.weight, experts.htoh4.bias, experts.h4toh.weight,
                                     experts.h4toh.bias, pos_g, slot_to_row,
                                     # (the very tensor object when it is flat: a pending read-back rides on it)
                                     global_expert_count if global_expert_count.dim() == 1 else global_expert_count.view(-1),
                                     top_k, act, fuse_chunks(), slot_order)
