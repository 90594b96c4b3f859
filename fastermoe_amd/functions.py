r"""Autograd Functions and routing helpers of the MoE layer, with the interface of
the reference's ``fmoe.functions`` (fmoe/functions.py), on top of
:mod:`fastermoe_amd.fmoe_native`.

Single worker only: ``world_size > 1`` (token all-to-all, dynamic shadowing) is
outside this package and raises ``NotImplementedError``.
"""
import torch
from torch.autograd import Function

from . import fmoe_native


def _single_worker(world_size, what):
    if world_size != 1:
        raise NotImplementedError(
            f"{what}: world_size={world_size}; this package implements the single-GPU "
            "path only (no global exchange, no dynamic shadowing)")


def ensure_comm(t, comm):
    """fmoe/functions.py:14-17 binds an NCCL communicator; nothing to do for one worker."""
    return None


class GateTopK(Function):
    r"""``torch.topk`` of the gate logits (and, with ``score_mode`` 1, the softmax over the selected
    logits) of fmoe/gates/naive_gate.py:26-42 with the routing of ``count_by_gate`` computed in
    the same launches.  Returns ``(topk_idx [N,k], topk_score [N,k])``; the routing result rides
    on ``topk_idx`` (``_fmoe_route``) and is picked up by :func:`_route` when the layer is handed
    this very tensor, unmodified."""

    @staticmethod
    def forward(ctx, logits, top_k, score_mode):
        logits = logits.contiguous()
        idx, score, cnt, pos_buf, s2r = fmoe_native.gate_topk_route(logits, top_k, score_mode)
        ctx.save_for_backward(idx, score)
        ctx.moe_args = logits.shape[1], score_mode
        ctx.mark_non_differentiable(idx)
        idx._fmoe_route = (idx._version, logits.shape[1], cnt, pos_buf, s2r)
        return idx, score

    @staticmethod
    def backward(ctx, _grad_idx, grad_score):
        idx, score = ctx.saved_tensors
        n_expert, score_mode = ctx.moe_args
        return fmoe_native.gate_topk_backward(grad_score.contiguous(), score, idx, n_expert, score_mode), None, None


class GateLinearTopK(Function):
    r"""``nn.Linear`` -> ``torch.topk`` (-> softmax) of fmoe/gates/naive_gate.py:26-42 and the routing of
    ``count_by_gate`` in one call that keeps the logits on chip.  Returns ``(topk_idx, topk_score)`` like
    :class:`GateTopK`; the routing rides on ``topk_idx``.  Backward: the sparse gradient of the logits
    (``fmoe_gate_topk_backward``), then the linear layer's own backward as two skinny library products."""

    @staticmethod
    def forward(ctx, x, weight, bias, top_k, score_mode):
        x = x.contiguous()
        weight = weight.contiguous()
        idx, score, cnt, pos_buf, s2r = fmoe_native.gate_linear_topk_route(x, weight, bias, top_k, score_mode)
        ctx.save_for_backward(x, weight, idx, score)
        ctx.moe_args = score_mode, bias is not None
        ctx.mark_non_differentiable(idx)
        idx._fmoe_route = (idx._version, weight.shape[0], cnt, pos_buf, s2r)
        return idx, score

    @staticmethod
    def backward(ctx, _grad_idx, grad_score):
        x, weight, idx, score = ctx.saved_tensors
        score_mode, has_bias = ctx.moe_args
        g = fmoe_native.gate_topk_backward(grad_score.contiguous(), score, idx, weight.shape[0], score_mode)
        grad_x = g @ weight if ctx.needs_input_grad[0] else None
        grad_w = g.t() @ x if ctx.needs_input_grad[1] else None
        grad_b = g.float().sum(dim=0).to(g.dtype) if has_bias and ctx.needs_input_grad[2] else None
        return grad_x, grad_w, grad_b, None, None


def gate_linear_topk(x, linear, top_k, score_mode=0):
    r"""Top-k indices and scores of ``linear(x)`` for an ``nn.Linear`` gate: one fused call when the
    shape is taken (CUDA tensors, at most 64 experts, ``top_k`` 1, 2, 4 or 8, rows of whole 16-byte
    chunks; ``FMOE_GATE_LINEAR_FUSED=0`` switches it off), else the layer followed by :func:`gate_topk`."""
    import os
    w, b = linear.weight, linear.bias
    if (x.is_cuda and x.dim() == 2 and w.is_cuda and w.dtype == x.dtype and (b is None or b.dtype == x.dtype)
            and os.environ.get("FMOE_GATE_LINEAR_FUSED", "1") != "0"
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and fmoe_native.gate_linear_supported(x.shape[1], w.shape[0], top_k, x.dtype)):
        return GateLinearTopK.apply(x, w, b, top_k, score_mode)
    return gate_topk(linear(x), top_k, score_mode)


class NoisyTopK(Function):
    r"""The training-mode selection of the noisy top-k gate (fmoe/gates/noisy_gate.py:113-144) after
    its two linear products: ``(topk_idx [N,k], gates [N,k], load [E])`` from the clean logits, the raw
    noise widths and a draw of N(0,1) noise, with the routing of ``count_by_gate`` riding on ``topk_idx``.
    ``load`` is the smooth estimate of tokens per expert (float32); both ``gates`` and ``load`` are
    differentiable with respect to ``clean`` and ``raw``."""

    @staticmethod
    def forward(ctx, clean, raw, noise, top_k, eps):
        clean, raw, noise = clean.contiguous(), raw.contiguous(), noise.contiguous()
        idx, gates, load, thr_val, thr_idx, cnt, pos_buf, s2r = fmoe_native.noisy_gate_forward(clean, raw, noise, top_k, eps)
        ctx.save_for_backward(clean, raw, noise, idx, gates, thr_val, thr_idx)
        ctx.moe_args = top_k, eps
        ctx.mark_non_differentiable(idx)
        idx._fmoe_route = (idx._version, clean.shape[1], cnt, pos_buf, s2r)
        return idx, gates, load

    @staticmethod
    def backward(ctx, _grad_idx, grad_gates, grad_load):
        clean, raw, noise, idx, gates, thr_val, thr_idx = ctx.saved_tensors
        top_k, eps = ctx.moe_args
        if grad_gates is None:
            grad_gates = torch.zeros_like(gates)
        if grad_load is None:
            grad_load = torch.zeros(clean.shape[1], dtype=torch.float32, device=clean.device)
        g_clean, g_raw = fmoe_native.noisy_gate_backward(clean, raw, noise, top_k, eps, idx, gates, thr_val, thr_idx,
                                                         grad_gates.contiguous(), grad_load.float().contiguous())
        return g_clean, g_raw, None, None, None


def gate_topk(logits, top_k, score_mode=0):
    r"""Top-k indices and scores of ``logits [N, E]``: the HIP gate kernel when it takes the shape
    (CUDA tensor, 16/32-bit floats, ``top_k`` 1, 2, 4 or 8), ``torch.topk``
    otherwise.  ``score_mode`` 0: the selected logits; 1: their softmax over the ``top_k``."""
    if logits.is_cuda and logits.dim() == 2 and fmoe_native.gate_topk_supported(logits.shape[1], top_k, logits.dtype):
        idx, score = GateTopK.apply(logits, top_k, score_mode)
        # autograd hands back a new Python object for the index tensor: carry the routing over
        return idx, score
    val, idx = torch.topk(logits, k=top_k, dim=-1, largest=True, sorted=False)
    return idx, (torch.softmax(val, dim=-1) if score_mode == 1 else val)


def _route_launch(gate, num_expert):
    """Enqueues the routing of ``gate`` (or picks up the one its :class:`GateTopK` call made) and
    returns the device tensors ``(counts [E], pos_buf [n_slots], slot_to_row [n_slots])``; nothing
    is read back.  ``pos_buf`` holds the routed slots first and -1 after them."""
    with torch.no_grad():
        cached = getattr(gate, "_fmoe_route", None)
        if cached is not None and cached[0] == gate._version and cached[1] == num_expert:
            return cached[2:]
        return fmoe_native.route(gate.contiguous(), num_expert)


def _route(gate, num_expert, world_size):
    """(pos, counts, slot_to_row): one fused routing call and ONE device-to-host
    read (the counts), instead of the histogram / cumsum / ``.item()`` /
    placement sequence of fmoe/functions.py:19-42.  An index tensor that comes
    straight from :class:`GateTopK` carries its routing with it."""
    _single_worker(world_size, "count_by_gate")
    counts, pos_buf, slot_to_row = _route_launch(gate, num_expert)
    with torch.no_grad():
        counts_cpu = counts.cpu()
        pos = pos_buf[: int(counts_cpu.sum())]
    return pos, counts, counts_cpu, slot_to_row


class _PendingCounts:
    """The expert counts on their way to the host: an asynchronous copy into pinned memory that
    starts right behind the routing kernels.  ``counts_cpu`` is the CPU tensor the counts will be
    in; it carries this object as ``_fmoe_pending``, and whoever reads its values calls
    :meth:`wait` first (``fmoe_native`` does, just before a launch that needs them), so that all
    host work up to that point runs while the GPU is still busy with whatever precedes the
    routing, instead of after it.  Only the fused pipeline of this package's own expert module is
    handed such a tensor: it goes to the bindings unread."""

    # (thread, device, n_expert) -> [pinned int64 buffer, the _PendingCounts whose copy is in it or None]
    _staging = {}

    def __init__(self, counts):
        import threading
        key = (threading.get_ident(), counts.device.index, counts.numel())
        slot = self._staging.get(key)
        if slot is None:
            slot = self._staging[key] = [torch.empty(counts.numel(), dtype=torch.int64, pin_memory=True), None]
        elif slot[1] is not None:
            slot[1].wait()   # an earlier read-back that nobody has waited for yet still owns the buffer
        self._buf = slot[0]
        self._slot = slot
        self._done = False
        self.counts_cpu = torch.empty(counts.numel(), dtype=torch.int64)
        self.counts_cpu._fmoe_pending = self
        # the copy and the event go to the current stream of the counts' device, whichever device is current
        with torch.cuda.device(counts.device), torch.no_grad():
            self._buf.copy_(counts, non_blocking=True)
            self._event = torch.cuda.Event()
            self._event.record(torch.cuda.current_stream(counts.device))
        slot[1] = self

    def wait(self):
        if not self._done:
            self._event.synchronize()
            self.counts_cpu.copy_(self._buf)
            self._done = True
            if self._slot[1] is self:
                self._slot[1] = None
        return self.counts_cpu


def count_by_gate(gate, num_expert, world_size, require_pos=True):
    """fmoe/functions.py:19-42.  Returns ``(pos, local_expert_count,
    all_expert_count, global_expert_count, all_global_expert_count)``; with one
    worker the four count tensors are the same int64 ``[num_expert]`` tensor."""
    _single_worker(world_size, "count_by_gate")
    with torch.no_grad():
        if not require_pos:
            cnt32 = torch.zeros(num_expert, device=gate.device, dtype=torch.int32)
            fmoe_native.expert_count(gate.contiguous(), cnt32)
            counts = cnt32.long()
            pos = None
        else:
            pos, counts, _, _ = _route(gate, num_expert, world_size)
    return pos, counts, counts, counts, counts


def _prepare_forward_ex(gate, num_expert, world_size):
    pos, counts, counts_cpu, slot_to_row = _route(gate, num_expert, world_size)
    return (pos, counts_cpu, counts_cpu, counts_cpu, counts_cpu, counts_cpu.clone()), slot_to_row


def prepare_forward(gate, num_expert, world_size):
    r"""fmoe/functions.py:45-69: ``(pos, local_expert_count, global_expert_count,
    all_expert_count, all_global_expert_count, fwd_expert_count)`` with ``pos`` on
    the device and the counts on the CPU."""
    return _prepare_forward_ex(gate, num_expert, world_size)[0]


def _local_scatter(inp, pos):
    """fmoe/functions.py:72-74 (index_select)."""
    return fmoe_native.gather_rows(inp.contiguous(), pos)


def _local_gather(inp, pos, out_batch_size, maybe_overlap=True):
    """fmoe/functions.py:77-84: zero-fill then index_add_ (``maybe_overlap``) or
    index_copy_."""
    inp = inp.contiguous()
    if maybe_overlap:
        return fmoe_native.index_add_rows(inp, pos, out_batch_size)
    inverse = fmoe_native.invert_index(pos, out_batch_size)
    return fmoe_native.gather_rows(inp, inverse)


class MOECache(Function):
    r"""fmoe/functions.py:122-194.  The reference decides here which experts to
    shadow on other workers and raises for one worker; with one worker there is
    nothing to shadow, so this is the identity: ``models = [[experts]]``,
    ``stored_models`` all False, counts unchanged."""

    @staticmethod
    def forward(ctx, inp, all_expert_count, all_global_expert_count, local_expert_count,
                global_expert_count, fwd_expert_count, policy_fn, experts, batch_size, d_model,
                topk, num_expert, world_size, fused):
        _single_worker(world_size, "MOECache")
        stored_models = torch.zeros(world_size * num_expert, dtype=torch.bool)
        models = [[experts]] if fused else [experts]
        ctx.mark_non_differentiable(stored_models, fwd_expert_count)
        return inp.view_as(inp), models, stored_models, fwd_expert_count, int(fwd_expert_count.sum().item())

    @staticmethod
    def backward(ctx, grad_inp, *unused):
        return (grad_inp,) + (None,) * 13


class MOEScatter(Function):
    r"""Token rows -> expert-sorted rows (fmoe/functions.py:196-248).  ``pos`` is
    the token index of every sorted row (``pos // top_k``).  The two trailing
    arguments are optional extras: given ``slot_to_row`` and ``top_k`` the
    backward sums each token's ``top_k`` rows directly instead of going through
    the general index-add."""

    @staticmethod
    def forward(ctx, inp, pos, local_expert_count, global_expert_count, stored_models,
                fwd_batch_size, world_size, slot_to_row=None, top_k=None):
        _single_worker(world_size, "MOEScatter")
        buf = _local_scatter(inp, pos)
        ctx.moe_args = inp.shape[0], top_k
        ctx.save_for_backward(pos, slot_to_row)
        return buf

    @staticmethod
    def backward(ctx, grad_buf):
        pos, slot_to_row = ctx.saved_tensors
        n_tokens, top_k = ctx.moe_args
        grad_buf = grad_buf.contiguous()
        if slot_to_row is not None:
            grad_in = fmoe_native.reduce_slots(grad_buf, slot_to_row, n_tokens, top_k)
        else:
            grad_in = _local_gather(grad_buf, pos, n_tokens)
        return grad_in, None, None, None, None, None, None, None, None


class MOELinear(Function):
    r"""Per-expert linear over expert-sorted rows (fmoe/functions.py:251-275)."""

    @staticmethod
    def forward(ctx, global_input_buf, fwd_expert_count, weight, bias=None):
        global_input_buf = global_input_buf.contiguous()
        out = fmoe_native.linear_forward(global_input_buf, fwd_expert_count, weight, bias)
        ctx.save_for_backward(global_input_buf, fwd_expert_count, weight, bias)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        input_buf, fwd_expert_count, weight, bias = ctx.saved_tensors
        grad_in, grad_w, grad_b = fmoe_native.linear_backward(
            grad_out.contiguous(), input_buf, fwd_expert_count, weight, bias)
        return grad_in, None, grad_w, grad_b


class MOEExpertMLP(Function):
    r"""``Linear -> activation -> Linear`` of fmoe/transformer.py:22-30 over expert-sorted rows as
    one autograd node, so that the activation runs in the first GEMM's epilogue and its
    derivative in the epilogue of the second linear's data gradient, instead of as elementwise
    kernels over ``[rows, d_hidden]`` of their own.  ``activation`` is an ``ACT_*`` code
    (exact GELU, ReLU or none).  Not in the reference; same results as the three modules."""

    @staticmethod
    def forward(ctx, inp, fwd_expert_count, w1, b1, w2, b2, activation):
        from . import _lib
        inp = inp.contiguous()
        keep_pre = activation == _lib.ACT_GELU  # ReLU's derivative can be read off the output
        mid, pre = fmoe_native.linear_act_forward(inp, fwd_expert_count, w1, b1, activation, keep_pre)
        out = fmoe_native.linear_forward(mid, fwd_expert_count, w2, b2)
        ctx.save_for_backward(inp, fwd_expert_count, w1, b1, w2, b2, pre, mid)
        ctx.activation = activation
        return out

    @staticmethod
    def backward(ctx, grad_out):
        inp, fwd_expert_count, w1, b1, w2, b2, pre, mid = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        g_pre = fmoe_native.linear_dact_backward(grad_out, fwd_expert_count, w2, pre if pre is not None else mid,
                                                 ctx.activation)
        gw2, gb2 = fmoe_native.linear_weight_backward(grad_out, mid, fwd_expert_count, w2, b2)
        g_inp, gw1, gb1 = fmoe_native.linear_backward(g_pre, inp, fwd_expert_count, w1, b1)
        return g_inp, None, gw1, gb1, gw2, gb2, None


class MOERoutedMLP(Function):
    r"""``MOEScatter`` -> ``Linear -> activation -> Linear`` (fmoe/functions.py:196-248,
    fmoe/transformer.py:22-30) over the rows as the routing kernels left them, with nothing read
    back to the host: the first GEMM reads token row ``pos_buf[r] // top_k`` for sorted row ``r``
    in its loader (no scattered copy), and all GEMMs take the experts' row segments from
    ``table``, the device-side segment table of the routing's counts.  Returns the experts' output
    in expert-sorted order, one row per slot (``[n_slots, d_model]``; the rows past the routed
    ones are not written), for :class:`MOEGatherCombine` / :class:`MOEGather`.  The backward makes
    the sorted copy of the input that the first linear's weight gradient contracts over.
    Not in the reference; same results as ``MOEScatter`` + the three modules."""

    @staticmethod
    def forward(ctx, inp, w1, b1, w2, b2, pos_buf, slot_to_row, table, top_k, activation):
        from . import _lib
        inp = inp.contiguous()
        n_slots = pos_buf.numel()
        keep_pre = activation == _lib.ACT_GELU  # ReLU's derivative can be read off the output
        in_loader = inp.numel() * inp.element_size() < (1 << 31)
        src = inp if in_loader else fmoe_native.gather_rows(inp, pos_buf, index_div=top_k)
        mid, pre = fmoe_native.linear_forward_dev(src, w1, b1, table, n_slots, activation, keep_pre,
                                                  row_index=pos_buf if in_loader else None, index_div=top_k)
        out, _ = fmoe_native.linear_forward_dev(mid, w2, b2, table, n_slots)
        ctx.save_for_backward(inp, w1, b1, w2, b2, pos_buf, slot_to_row, table, pre, mid)
        ctx.moe_args = top_k, activation
        return out

    @staticmethod
    def backward(ctx, grad_out):
        inp, w1, b1, w2, b2, pos_buf, slot_to_row, table, pre, mid = ctx.saved_tensors
        top_k, activation = ctx.moe_args
        n_slots = pos_buf.numel()
        grad_out = grad_out.contiguous()
        g_pre = fmoe_native.linear_dgrad_dev(grad_out, w2, table, n_slots, pre if pre is not None else mid, activation)
        gw2, gb2 = fmoe_native.linear_wgrad_dev(grad_out, mid, w2, table, n_slots, b2 is not None)
        g_inp = None
        if ctx.needs_input_grad[0]:
            g_rows = fmoe_native.linear_dgrad_dev(g_pre, w1, table, n_slots)
            g_inp = fmoe_native.reduce_slots(g_rows, slot_to_row, inp.shape[0], top_k)
        rows = fmoe_native.gather_rows(inp, pos_buf, index_div=top_k)
        gw1, gb1 = fmoe_native.linear_wgrad_dev(g_pre, rows, w1, table, n_slots, b1 is not None)
        return g_inp, gw1, gb1, gw2, gb2, None, None, None, None, None


class MOEGather(Function):
    r"""Expert-sorted rows -> slot order, zero rows for dropped slots
    (fmoe/functions.py:278-330).  ``slot_to_row`` (optional extra) is the inverse
    of ``pos``; without it the inverse is rebuilt from ``pos``."""

    @staticmethod
    def forward(ctx, global_output_buf, pos, local_expert_count, global_expert_count,
                stored_models, local_batch_size, world_size, slot_to_row=None):
        _single_worker(world_size, "MOEGather")
        buf = global_output_buf.contiguous()
        if slot_to_row is None:
            slot_to_row = fmoe_native.invert_index(pos, local_batch_size)
        out = fmoe_native.gather_rows(buf, slot_to_row, local_batch_size)
        ctx.save_for_backward(pos)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        (pos,) = ctx.saved_tensors
        return _local_scatter(grad_out, pos), None, None, None, None, None, None, None


class MOECombine(Function):
    r"""``torch.bmm(gate_score[N,1,k], x[N,k,d])`` of fmoe/layers.py:321-322 as one
    streaming kernel (fp32 accumulation, one rounding) with its backward."""

    @staticmethod
    def forward(ctx, x, gate_score, n_tokens, top_k):
        x = x.contiguous()
        gate_score = gate_score.contiguous()
        ctx.save_for_backward(x, gate_score)
        ctx.moe_args = n_tokens, top_k, gate_score.shape
        return fmoe_native.combine_forward(x, gate_score, n_tokens, top_k)

    @staticmethod
    def backward(ctx, grad_out):
        x, gate_score = ctx.saved_tensors
        n_tokens, top_k, score_shape = ctx.moe_args
        grad_x, grad_score = fmoe_native.combine_backward(grad_out.contiguous(), x, gate_score, n_tokens, top_k)
        return grad_x, grad_score.view(score_shape), None, None


class MOEGatherCombine(Function):
    r"""``MOEGather`` (fmoe/functions.py:285-312) and the ``bmm`` with the gate scores
    (fmoe/layers.py:321-322) as one pass over the experts' output in expert-sorted
    order: ``out[t] = sum_j score[t,j] * rows[slot_to_row[t*k+j]]``; dropped slots
    (``slot_to_row < 0``) contribute zero, as the zero rows of ``_local_gather`` do."""

    @staticmethod
    def forward(ctx, rows, slot_to_row, gate_score, n_tokens, top_k):
        rows = rows.contiguous()
        gate_score = gate_score.contiguous()
        ctx.save_for_backward(rows, slot_to_row, gate_score)
        ctx.moe_args = n_tokens, top_k, gate_score.shape
        return fmoe_native.gather_combine_forward(rows, slot_to_row, gate_score, n_tokens, top_k)

    @staticmethod
    def backward(ctx, grad_out):
        rows, slot_to_row, gate_score = ctx.saved_tensors
        n_tokens, top_k, score_shape = ctx.moe_args
        grad_rows, grad_score = fmoe_native.gather_combine_backward(grad_out.contiguous(), rows, slot_to_row,
                                                                    gate_score, n_tokens, top_k)
        return grad_rows, None, grad_score.view(score_shape), None, None


def mask_index(mask):
    r"""For FMoE's ``mask`` (fmoe/layers.py:288-293): ``(keep_idx, token_to_row)`` -- the indices of
    the tokens whose mask is 0 (what ``inp[mask == 0]`` selects, here in descending token order)
    and, per token, its row among the kept ones (-1 for masked tokens).  One routing call with a
    single "expert" and one device-to-host read (the number of kept tokens), no boolean indexing."""
    with torch.no_grad():
        key = (mask.reshape(-1) != 0).to(torch.int64).neg_()        # 0: keep, -1: masked
        counts, pos_buf, token_to_row = fmoe_native.route(key, 1)
        keep_idx = pos_buf[: int(counts.cpu()[0])]
    return keep_idx, token_to_row


class MaskSelect(Function):
    r"""``rows[keep_idx]``: the rows of the kept tokens (``inp[mask == 0, :]``, fmoe/layers.py:292);
    the backward puts the gradient rows back and leaves zero rows for masked tokens."""

    @staticmethod
    def forward(ctx, rows, keep_idx, token_to_row):
        ctx.save_for_backward(token_to_row)
        return fmoe_native.gather_rows(rows.contiguous(), keep_idx)

    @staticmethod
    def backward(ctx, grad_rows):
        (token_to_row,) = ctx.saved_tensors
        return fmoe_native.gather_rows(grad_rows.contiguous(), token_to_row), None, None


class MaskRestore(Function):
    r"""Back to the full token order (fmoe/layers.py:305-317, with the combine of :322 already
    applied to the kept tokens): ``out[t] = kept[token_to_row[t]]`` for kept tokens and
    ``scale[t] * fill[fill_row[t]]`` for a masked token whose mask value has a ``mask_dict`` entry
    (``scale`` = the sum of the token's gate scores, since every one of its ``top_k`` slots holds
    the same ``mask_dict`` value), zero rows otherwise.  ``fill`` may be ``None``."""

    @staticmethod
    def forward(ctx, kept, keep_idx, token_to_row, scale, fill, fill_row):
        ctx.save_for_backward(keep_idx, token_to_row, scale, fill, fill_row)
        return fmoe_native.mask_restore(kept.contiguous(), token_to_row, scale, fill, fill_row, token_to_row.numel())

    @staticmethod
    def backward(ctx, grad_out):
        keep_idx, token_to_row, scale, fill, fill_row = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        grad_kept = fmoe_native.gather_rows(grad_out, keep_idx)
        grad_scale = grad_fill = None
        if fill is not None and scale is not None and ctx.needs_input_grad[3]:
            grad_scale = fmoe_native.mask_scale_grad(grad_out, token_to_row, fill, fill_row)
        if fill is not None and ctx.needs_input_grad[4]:
            # a mask_dict value that is trained: rare, plain torch
            masked = (token_to_row < 0) & (fill_row >= 0)
            w = scale.float() if scale is not None else torch.ones_like(fill_row, dtype=torch.float32)
            contrib = (grad_out.float() * (w * masked).unsqueeze(1))
            grad_fill = torch.zeros(fill.shape, dtype=torch.float32, device=fill.device).index_add_(
                0, fill_row.clamp(min=0), contrib).to(fill.dtype)
        return grad_kept, None, None, grad_scale, grad_fill, None


class AllGather(Function):
    r"""fmoe/functions.py:333-349 (model-parallel group); one worker only."""

    @staticmethod
    def forward(ctx, inp, rank, world_size, group):
        _single_worker(world_size, "AllGather")
        return inp.view_as(inp)

    @staticmethod
    def backward(ctx, grad_out):
        return grad_out, None, None, None


class Slice(Function):
    r"""fmoe/functions.py:352-375 (model-parallel group); one worker only."""

    @staticmethod
    def forward(ctx, inp, rank, world_size, group):
        _single_worker(world_size, "Slice")
        return inp.view_as(inp)

    @staticmethod
    def backward(ctx, grad_out):
        return grad_out, None, None, None
