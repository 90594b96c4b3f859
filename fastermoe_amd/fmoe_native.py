"""Operator module with the interface of the reference's ``fmoe_cuda`` extension
(cuda/fmoe_cuda.cpp:105-130), backed by ``libfmoe_hip.so``.

Every function validates its tensors (Python exceptions instead of the
reference's ``exit()``), allocates outputs with torch, and enqueues the HIP
kernels on torch's current stream through the C ABI.  Nothing here computes on
the CPU and nothing falls back to torch operators.
"""
import ctypes

import torch

from . import _lib
from ._lib import check

_DTYPES = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16,
           torch.float64: _lib.F64}


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _dev(name, t, dtype=None):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise ValueError(f"{name} must be a CUDA (HIP) tensor, got device {t.device}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must have dtype {dtype}, got {t.dtype}")
    return t


def _host_counts(name, t, n=None):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.is_cuda:
        raise ValueError(f"{name} must be a CPU tensor (it is read on the host)")
    if t.dtype != torch.int64:
        raise TypeError(f"{name} must have dtype torch.int64, got {t.dtype}")
    # counts that are still on their way from the device (an asynchronous read-back started by the
    # layer) are waited for here, at the last moment before the host reads them
    pending = getattr(t, "_fmoe_pending", None)
    if pending is not None:
        pending.wait()
    t = t.contiguous().view(-1)
    if n is not None and t.numel() != n:
        raise ValueError(f"{name} has {t.numel()} entries, expected {n}")
    return t


def _float_dtype(name, t):
    if t.dtype not in _DTYPES:
        raise TypeError(f"{name}: unsupported dtype {t.dtype}")
    return _DTYPES[t.dtype]


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


# ---- routing ----------------------------------------------------------------

def expert_count(gate_idx, expert_count):
    """expert_count[e] += number of entries of gate_idx equal to e (-1 skipped).
    fmoe_cuda.expert_count, cuda/local_exchange.cu:22-32."""
    _dev("gate_idx", gate_idx, torch.int64)
    _dev("expert_count", expert_count, torch.int32)
    lib = _lib.load()
    with torch.cuda.device(gate_idx.device):
        check(lib.fmoe_expert_count(_ptr(gate_idx), _ptr(expert_count), gate_idx.numel(),
                                    expert_count.numel(), _stream(gate_idx)))


def assign_pos(cum_count, gate, pos):
    """Fills ``pos`` with the slot indices grouped by expert; ``cum_count`` (int32
    inclusive cumsum) is left as the exclusive cumsum.
    fmoe_cuda.assign_pos, cuda/local_exchange.cu:5-20."""
    _dev("cum_count", cum_count, torch.int32)
    _dev("gate", gate, torch.int64)
    _dev("pos", pos, torch.int64)
    lib = _lib.load()
    n, e = gate.numel(), cum_count.numel()
    with torch.cuda.device(gate.device):
        ws = _workspace(lib.fmoe_routing_workspace_bytes(n, e), gate.device)
        check(lib.fmoe_assign_pos(_ptr(cum_count), _ptr(gate), _ptr(pos), pos.numel(), n, e, _ptr(ws), ws.numel(),
                                  _stream(gate)))


def route(gate, n_expert):
    """One call for what fmoe/functions.py:19-42 does in several: returns
    ``(expert_count int64 [E], pos_buf int64 [n_slots], slot_to_row int64 [n_slots])``,
    all on the device.  Only the first ``expert_count.sum()`` entries of
    ``pos_buf`` are meaningful."""
    _dev("gate", gate, torch.int64)
    lib = _lib.load()
    n = gate.numel()
    with torch.cuda.device(gate.device):
        cnt = torch.empty(n_expert, dtype=torch.int64, device=gate.device)
        pos = torch.empty(n, dtype=torch.int64, device=gate.device)
        s2r = torch.empty(n, dtype=torch.int64, device=gate.device)
        ws = _workspace(lib.fmoe_routing_workspace_bytes(n, n_expert), gate.device)
        check(lib.fmoe_route(_ptr(gate), n, n_expert, _ptr(cnt), _ptr(pos), _ptr(s2r), _ptr(ws), ws.numel(),
                             _stream(gate)))
    return cnt, pos, s2r


def gate_topk_supported(n_expert, top_k, dtype):
    """Whether :func:`gate_topk_route` takes this gate shape (else: torch.topk and :func:`route`)."""
    return (top_k in (1, 2, 4, 8) and top_k <= n_expert <= 8192
            and dtype in (torch.float32, torch.bfloat16, torch.float16))


def gate_topk_route(logits, top_k, score_mode=0):
    """Top-k of ``logits [N, E]`` with the routing bookkeeping in the same launches.  Returns
    ``(topk_idx int64 [N,k], topk_score [N,k], expert_count int64 [E], pos_buf int64 [N*k],
    slot_to_row int64 [N*k])``; ``score_mode`` 0 returns the selected logits as scores, 1 their
    softmax over the k selected."""
    _dev("logits", logits)
    if logits.dim() != 2:
        raise ValueError(f"logits must be [n_tokens, n_expert], got {tuple(logits.shape)}")
    n, e = logits.shape
    if not gate_topk_supported(e, top_k, logits.dtype):
        raise ValueError(f"gate_topk_route does not take n_expert={e}, top_k={top_k}, dtype={logits.dtype}")
    dt = _float_dtype("logits", logits)
    lib = _lib.load()
    dev = logits.device
    with torch.cuda.device(dev):
        idx = torch.empty(n, top_k, dtype=torch.int64, device=dev)
        score = torch.empty(n, top_k, dtype=logits.dtype, device=dev)
        cnt = torch.empty(e, dtype=torch.int64, device=dev)
        pos = torch.empty(n * top_k, dtype=torch.int64, device=dev)
        s2r = torch.empty(n * top_k, dtype=torch.int64, device=dev)
        ws = _workspace(lib.fmoe_routing_workspace_bytes(n * top_k, e), dev)
        check(lib.fmoe_gate_topk_route(_ptr(logits), n, e, top_k, dt, score_mode, _ptr(idx), _ptr(score), _ptr(cnt),
                                       _ptr(pos), _ptr(s2r), _ptr(ws), ws.numel(), _stream(logits)))
    return idx, score, cnt, pos, s2r


def gate_linear_supported(d_model, n_expert, top_k, dtype):
    """Whether :func:`gate_linear_topk_route` takes this gate (else: the linear layer and :func:`gate_topk_route`)."""
    return dtype in _DTYPES and _lib.load().fmoe_gate_linear_supported(int(d_model), int(n_expert), int(top_k),
                                                                       _DTYPES[dtype]) == 1


def gate_linear_topk_route(x, weight, bias, top_k, score_mode=0):
    """``gate_topk_route(x @ weight.T + bias, ...)`` without the logits ever reaching memory: the gate's
    linear layer, its top-k, the scores and the routing in one call.  ``weight`` is ``[E, d_model]``
    (``nn.Linear.weight``), ``bias`` ``[E]`` or ``None``.  Same results tuple as :func:`gate_topk_route`."""
    dt = _rows("x", x)
    _dev("weight", weight, x.dtype)
    if weight.dim() != 2 or weight.shape[1] != x.shape[1]:
        raise ValueError(f"weight must be [n_expert, {x.shape[1]}], got {tuple(weight.shape)}")
    n, d = x.shape
    e = weight.shape[0]
    if bias is not None:
        _dev("bias", bias, x.dtype)
        if tuple(bias.shape) != (e,):
            raise ValueError(f"bias must be [{e}], got {tuple(bias.shape)}")
    if not gate_linear_supported(d, e, top_k, x.dtype):
        raise ValueError(f"gate_linear_topk_route does not take d_model={d}, n_expert={e}, top_k={top_k}, dtype={x.dtype}")
    lib = _lib.load()
    dev = x.device
    with torch.cuda.device(dev):
        idx = torch.empty(n, top_k, dtype=torch.int64, device=dev)
        score = torch.empty(n, top_k, dtype=x.dtype, device=dev)
        cnt = torch.empty(e, dtype=torch.int64, device=dev)
        pos = torch.empty(n * top_k, dtype=torch.int64, device=dev)
        s2r = torch.empty(n * top_k, dtype=torch.int64, device=dev)
        ws = _workspace(lib.fmoe_routing_workspace_bytes(n * top_k, e), dev)
        check(lib.fmoe_gate_linear_topk_route(_ptr(x), _ptr(weight), _ptr(bias), n, d, e, top_k, dt, score_mode, _ptr(idx),
                                              _ptr(score), _ptr(cnt), _ptr(pos), _ptr(s2r), _ptr(ws), ws.numel(),
                                              _stream(x)))
    return idx, score, cnt, pos, s2r


def noisy_gate_supported(n_expert, top_k, dtype):
    """Whether :func:`noisy_gate_forward` takes this gate shape."""
    return top_k in (1, 2, 4, 8) and top_k < n_expert <= 2048 and dtype in (torch.float32, torch.bfloat16, torch.float16)


def noisy_gate_forward(clean, raw, noise, top_k, eps):
    """Noisy top-k gating after the two linear products (training mode).  Returns ``(topk_idx [N,k],
    gates [N,k], load float32 [E], thr_val, thr_idx, expert_count, pos_buf, slot_to_row)``;
    ``thr_val`` / ``thr_idx`` are what :func:`noisy_gate_backward` needs."""
    dt = _rows("clean", clean)
    _dev("raw", raw, clean.dtype)
    _dev("noise", noise, clean.dtype)
    if raw.shape != clean.shape or noise.shape != clean.shape:
        raise ValueError("clean, raw and noise must have the same shape [n_tokens, n_expert]")
    n, e = clean.shape
    if not noisy_gate_supported(e, top_k, clean.dtype):
        raise ValueError(f"noisy_gate_forward does not take n_expert={e}, top_k={top_k}, dtype={clean.dtype}")
    lib = _lib.load()
    dev = clean.device
    n_blocks = max(1, -(-n * top_k // 2048))
    with torch.cuda.device(dev):
        idx = torch.empty(n, top_k, dtype=torch.int64, device=dev)
        gates = torch.empty(n, top_k, dtype=clean.dtype, device=dev)
        thr_val = torch.empty(n, 2, dtype=torch.float32, device=dev)
        thr_idx = torch.empty(n, 2, dtype=torch.int32, device=dev)
        partial = torch.zeros(n_blocks, e, dtype=torch.float32, device=dev)
        cnt = torch.empty(e, dtype=torch.int64, device=dev)
        pos = torch.empty(n * top_k, dtype=torch.int64, device=dev)
        s2r = torch.empty(n * top_k, dtype=torch.int64, device=dev)
        ws = _workspace(lib.fmoe_routing_workspace_bytes(n * top_k, e), dev)
        check(lib.fmoe_noisy_gate_forward(_ptr(clean), _ptr(raw), _ptr(noise), float(eps), n, e, top_k, dt, _ptr(idx),
                                          _ptr(gates), _ptr(thr_val), _ptr(thr_idx), _ptr(partial), _ptr(cnt), _ptr(pos),
                                          _ptr(s2r), _ptr(ws), ws.numel(), _stream(clean)))
        load = partial.sum(dim=0)
    return idx, gates, load, thr_val, thr_idx, cnt, pos, s2r


def noisy_gate_backward(clean, raw, noise, top_k, eps, topk_idx, gates, thr_val, thr_idx, grad_gates, grad_load):
    """Gradients of ``clean`` and ``raw`` ``[N, E]`` from those of the gates ``[N, k]`` and the load ``[E]``."""
    dt = _rows("clean", clean)
    _dev("grad_gates", grad_gates, clean.dtype)
    _dev("grad_load", grad_load, torch.float32)
    n, e = clean.shape
    grad_clean, grad_raw = torch.empty_like(clean), torch.empty_like(clean)
    with torch.cuda.device(clean.device):
        check(_lib.load().fmoe_noisy_gate_backward(_ptr(clean), _ptr(raw), _ptr(noise), float(eps), n, e, top_k, dt,
                                                   _ptr(topk_idx), _ptr(gates), _ptr(thr_val), _ptr(thr_idx),
                                                   _ptr(grad_gates), _ptr(grad_load), _ptr(grad_clean), _ptr(grad_raw),
                                                   _stream(clean)))
    return grad_clean, grad_raw


def gate_topk_backward(grad_score, score, topk_idx, n_expert, score_mode=0):
    """Gradient of the top-k scores with respect to the logits, ``[N, E]``."""
    _dev("grad_score", grad_score)
    _dev("topk_idx", topk_idx, torch.int64)
    n, k = topk_idx.shape
    dt = _float_dtype("grad_score", grad_score)
    if score_mode == 1:
        _dev("score", score, grad_score.dtype)
    grad_logits = torch.empty(n, n_expert, dtype=grad_score.dtype, device=grad_score.device)
    with torch.cuda.device(grad_score.device):
        check(_lib.load().fmoe_gate_topk_backward(_ptr(grad_score), _ptr(score if score_mode == 1 else None),
                                                  _ptr(topk_idx), _ptr(grad_logits), n, n_expert, k, dt, score_mode,
                                                  _stream(grad_score)))
    return grad_logits


def limit_by_capacity(expert_count, capacity, n_expert, n_worker):
    """fmoe_cuda.limit_by_capacity, cuda/balancing.cu:7-20."""
    _dev("expert_count", expert_count, torch.int64)
    _dev("capacity", capacity, torch.int32)
    if expert_count.numel() != n_expert * n_worker:
        raise ValueError("expert_count must have n_expert * n_worker entries")
    if capacity.numel() != n_expert:
        raise ValueError("capacity must have n_expert entries")
    lib = _lib.load()
    out = torch.empty_like(expert_count)
    with torch.cuda.device(expert_count.device):
        check(lib.fmoe_limit_by_capacity(_ptr(expert_count), _ptr(capacity), _ptr(out), n_expert, n_worker,
                                         _stream(expert_count)))
    return out


def prune_gate_by_capacity(gate_idx, expert_count, n_expert, n_worker):
    """fmoe_cuda.prune_gate_by_capacity, cuda/balancing.cu:22-37."""
    _dev("gate_idx", gate_idx, torch.int64)
    _dev("expert_count", expert_count, torch.int32)
    if expert_count.numel() != n_expert * n_worker:
        raise ValueError("expert_count must have n_expert * n_worker entries")
    lib = _lib.load()
    out = torch.empty_like(gate_idx)
    n, e = gate_idx.numel(), expert_count.numel()
    with torch.cuda.device(gate_idx.device):
        ws = _workspace(lib.fmoe_routing_workspace_bytes(n, e), gate_idx.device)
        check(lib.fmoe_prune_gate_by_capacity(_ptr(gate_idx), _ptr(out), _ptr(expert_count), n, e, _ptr(ws),
                                              ws.numel(), _stream(gate_idx)))
    return out


# ---- row permutes -------------------------------------------------------------

def _rows(name, t):
    _dev(name, t)
    if t.dim() != 2:
        raise ValueError(f"{name} must be 2-D [rows, features], got shape {tuple(t.shape)}")
    return _float_dtype(name, t)


def gather_rows(inp, index, n_out=None, index_div=1):
    """out[r] = inp[index[r] // index_div] (zero row where index[r] < 0)."""
    dt = _rows("inp", inp)
    _dev("index", index, torch.int64)
    n_out = index.numel() if n_out is None else n_out
    out = torch.empty(n_out, inp.shape[1], dtype=inp.dtype, device=inp.device)
    with torch.cuda.device(inp.device):
        if index_div == 1:
            check(_lib.load().fmoe_gather_rows(_ptr(inp), _ptr(index), _ptr(out), n_out, inp.shape[0], inp.shape[1],
                                               dt, _stream(inp)))
        else:
            check(_lib.load().fmoe_gather_rows_div(_ptr(inp), _ptr(index), int(index_div), _ptr(out), n_out,
                                                   inp.shape[0], inp.shape[1], dt, _stream(inp)))
    return out


def invert_index(pos, n_out):
    """inverse[pos[i]] = i, -1 elsewhere."""
    _dev("pos", pos, torch.int64)
    inv = torch.empty(n_out, dtype=torch.int64, device=pos.device)
    with torch.cuda.device(pos.device):
        check(_lib.load().fmoe_invert_index(_ptr(pos), pos.numel(), _ptr(inv), n_out, _stream(pos)))
    return inv


def reduce_slots(inp, slot_to_row, n_tokens, top_k):
    """out[t] = sum over the token's top_k slots of inp[slot_to_row[slot]]."""
    dt = _rows("inp", inp)
    _dev("slot_to_row", slot_to_row, torch.int64)
    if slot_to_row.numel() != n_tokens * top_k:
        raise ValueError("slot_to_row must have n_tokens * top_k entries")
    out = torch.empty(n_tokens, inp.shape[1], dtype=inp.dtype, device=inp.device)
    with torch.cuda.device(inp.device):
        check(_lib.load().fmoe_reduce_slots(_ptr(inp), _ptr(slot_to_row), _ptr(out), n_tokens, top_k,
                                            inp.shape[0], inp.shape[1], dt, _stream(inp)))
    return out


def index_add_rows(inp, index, n_out):
    """zeros(n_out, d).index_add_(0, index, inp), summed in a fixed order."""
    dt = _rows("inp", inp)
    _dev("index", index, torch.int64)
    if index.numel() != inp.shape[0]:
        raise ValueError("index must have one entry per row of inp")
    lib = _lib.load()
    out = torch.empty(n_out, inp.shape[1], dtype=inp.dtype, device=inp.device)
    with torch.cuda.device(inp.device):
        ws = _workspace(lib.fmoe_index_add_workspace_bytes(inp.shape[0], n_out), inp.device)
        check(lib.fmoe_index_add_rows(_ptr(inp), _ptr(index), _ptr(out), inp.shape[0], n_out, inp.shape[1], dt,
                                      _ptr(ws), ws.numel(), _stream(inp)))
    return out


def mask_restore(src, token_to_row, scale, fill, fill_row, n_tokens):
    """out[t] = src[token_to_row[t]] for kept tokens, scale[t] * fill[fill_row[t]] for masked tokens
    that have a fill row, zero otherwise.  ``fill`` may be ``None`` (no fill rows at all)."""
    dt = _rows("src", src)
    _dev("token_to_row", token_to_row, torch.int64)
    n_fill = 0
    if fill is not None:
        _dev("fill", fill, src.dtype)
        _dev("fill_row", fill_row, torch.int64)
        n_fill = fill.shape[0]
        if scale is not None:
            _dev("scale", scale, src.dtype)
    out = torch.empty(n_tokens, src.shape[1], dtype=src.dtype, device=src.device)
    with torch.cuda.device(src.device):
        check(_lib.load().fmoe_mask_restore(_ptr(src), _ptr(token_to_row), _ptr(scale if fill is not None else None),
                                            _ptr(fill), _ptr(fill_row if fill is not None else None), _ptr(out),
                                            n_tokens, src.shape[0], n_fill, src.shape[1], dt, _stream(src)))
    return out


def mask_scale_grad(grad_out, token_to_row, fill, fill_row):
    """Per-token dot product of the output gradient with the token's fill row (masked tokens only)."""
    dt = _rows("grad_out", grad_out)
    _dev("fill", fill, grad_out.dtype)
    grad_scale = torch.empty(grad_out.shape[0], dtype=grad_out.dtype, device=grad_out.device)
    with torch.cuda.device(grad_out.device):
        check(_lib.load().fmoe_mask_scale_grad(_ptr(grad_out), _ptr(token_to_row), _ptr(fill), _ptr(fill_row),
                                               _ptr(grad_scale), grad_out.shape[0], fill.shape[0], grad_out.shape[1],
                                               dt, _stream(grad_out)))
    return grad_scale


# ---- score-weighted combine ---------------------------------------------------------

def combine_forward(x, score, n_tokens, top_k):
    """out[t] = sum_j score[t,j] * x[t*top_k+j]  (torch.bmm(score[N,1,k], x[N,k,d]))."""
    dt = _rows("x", x)
    _dev("score", score, x.dtype)
    if x.shape[0] != n_tokens * top_k or score.numel() != n_tokens * top_k:
        raise ValueError("x must have n_tokens*top_k rows and score n_tokens*top_k entries")
    out = torch.empty(n_tokens, x.shape[1], dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        check(_lib.load().fmoe_combine_forward(_ptr(x), _ptr(score), _ptr(out), n_tokens, top_k, x.shape[1], dt,
                                               _stream(x)))
    return out


def combine_backward(grad_out, x, score, n_tokens, top_k):
    """Returns (grad_x [N*top_k, d], grad_score [N, top_k])."""
    dt = _rows("x", x)
    _dev("grad_out", grad_out, x.dtype)
    _dev("score", score, x.dtype)
    if tuple(grad_out.shape) != (n_tokens, x.shape[1]):
        raise ValueError(f"grad_out must be [{n_tokens}, {x.shape[1]}]")
    grad_x = torch.empty_like(x)
    grad_score = torch.empty(n_tokens, top_k, dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        check(_lib.load().fmoe_combine_backward(_ptr(grad_out), _ptr(x), _ptr(score), _ptr(grad_x), _ptr(grad_score),
                                                n_tokens, top_k, x.shape[1], dt, _stream(x)))
    return grad_x, grad_score


def gather_combine_forward(rows, slot_to_row, score, n_tokens, top_k):
    """out[t] = sum_j score[t,j] * rows[slot_to_row[t*top_k+j]] (dropped slots, index < 0,
    contribute nothing): MOEGather's copy to slot order and the bmm in one pass."""
    dt = _rows("rows", rows)
    _dev("score", score, rows.dtype)
    _dev("slot_to_row", slot_to_row, torch.int64)
    if slot_to_row.numel() != n_tokens * top_k or score.numel() != n_tokens * top_k:
        raise ValueError("slot_to_row and score must have n_tokens*top_k entries")
    out = torch.empty(n_tokens, rows.shape[1], dtype=rows.dtype, device=rows.device)
    with torch.cuda.device(rows.device):
        check(_lib.load().fmoe_gather_combine_forward(_ptr(rows), _ptr(slot_to_row), _ptr(score), _ptr(out), n_tokens,
                                                      top_k, rows.shape[0], rows.shape[1], dt, _stream(rows)))
    return out


def gather_combine_backward(grad_out, rows, slot_to_row, score, n_tokens, top_k):
    """Returns (grad_rows [n_rows, d] in expert-sorted order, grad_score [N, top_k])."""
    dt = _rows("rows", rows)
    _dev("grad_out", grad_out, rows.dtype)
    _dev("score", score, rows.dtype)
    _dev("slot_to_row", slot_to_row, torch.int64)
    if tuple(grad_out.shape) != (n_tokens, rows.shape[1]):
        raise ValueError(f"grad_out must be [{n_tokens}, {rows.shape[1]}]")
    if slot_to_row.numel() != n_tokens * top_k or score.numel() != n_tokens * top_k:
        raise ValueError("slot_to_row and score must have n_tokens*top_k entries")
    grad_rows = torch.empty_like(rows)
    grad_score = torch.empty(n_tokens, top_k, dtype=rows.dtype, device=rows.device)
    with torch.cuda.device(rows.device):
        check(_lib.load().fmoe_gather_combine_backward(_ptr(grad_out), _ptr(rows), _ptr(slot_to_row), _ptr(score),
                                                       _ptr(grad_rows), _ptr(grad_score), n_tokens, top_k,
                                                       rows.shape[0], rows.shape[1], dt, _stream(rows)))
    return grad_rows, grad_score


# ---- per-expert linear ----------------------------------------------------------

def _check_linear(input_buf, expert_count, weight, bias):
    """Shapes and dtypes first, the counts last: reading them may have to wait for their read-back.
    ``input_buf`` may hold more rows than the counts add up to (a buffer sized for every slot, of
    which the routed ones come first): the rows past the counted ones are neither read nor written."""
    dt = _rows("input_buf", input_buf)
    _dev("weight", weight, input_buf.dtype)
    if weight.dim() != 3:
        raise ValueError(f"weight must be [num_expert, out_feat, in_feat], got {tuple(weight.shape)}")
    n_expert, out_feat, in_feat = weight.shape
    if input_buf.shape[1] != in_feat:
        raise ValueError(f"input_buf has {input_buf.shape[1]} features, weight expects {in_feat}")
    if bias is not None:
        _dev("bias", bias, input_buf.dtype)
        if tuple(bias.shape) != (n_expert, out_feat):
            raise ValueError(f"bias must be [{n_expert}, {out_feat}], got {tuple(bias.shape)}")
    return dt, n_expert, out_feat, in_feat


def _linear_counts(input_buf, expert_count, n_expert):
    cnt = _host_counts("expert_count", expert_count, n_expert)
    total = int(cnt.sum())
    if total > input_buf.shape[0]:
        raise ValueError(f"expert_count sums to {total} but input_buf has {input_buf.shape[0]} rows")
    return cnt


def linear_forward(input_buf, expert_count, weight, bias=None):
    """Y[seg_e] = X[seg_e] @ W_e^T (+ b_e).  fmoe_cuda.linear_forward,
    cuda/parallel_linear.cu:5-49; ``expert_count`` is a CPU int64 tensor."""
    dt, n_expert, out_feat, in_feat = _check_linear(input_buf, expert_count, weight, bias)
    out = torch.empty(input_buf.shape[0], out_feat, dtype=input_buf.dtype, device=input_buf.device)
    cnt = _linear_counts(input_buf, expert_count, n_expert)
    with torch.cuda.device(input_buf.device):
        check(_lib.load().fmoe_linear_forward(_ptr(input_buf), _ptr(weight), _ptr(bias), _ptr(out),
                                              ctypes.c_void_p(cnt.data_ptr()), n_expert, in_feat, out_feat, dt,
                                              _stream(input_buf)))
    return out


def linear_backward(grad_output_buf, input_buf, expert_count, weight, bias=None):
    """Returns [grad_input, grad_weight, grad_bias].  fmoe_cuda.linear_backward,
    cuda/parallel_linear.cu:52-94.  ``grad_bias`` is computed only when ``bias``
    is given (the reference returns an uninitialised tensor otherwise); without
    bias it is ``None``."""
    dt, n_expert, out_feat, in_feat = _check_linear(input_buf, expert_count, weight, bias)
    cnt = _linear_counts(input_buf, expert_count, n_expert)
    _dev("grad_output_buf", grad_output_buf, input_buf.dtype)
    if tuple(grad_output_buf.shape) != (input_buf.shape[0], out_feat):
        raise ValueError(f"grad_output_buf must be [{input_buf.shape[0]}, {out_feat}]")
    grad_in = torch.empty_like(input_buf)
    grad_w = torch.empty_like(weight)
    grad_b = torch.empty(n_expert, out_feat, dtype=input_buf.dtype, device=input_buf.device) \
        if bias is not None else None
    with torch.cuda.device(input_buf.device):
        check(_lib.load().fmoe_linear_backward(_ptr(grad_output_buf), _ptr(input_buf), _ptr(weight), _ptr(grad_in),
                                               _ptr(grad_w), _ptr(grad_b), ctypes.c_void_p(cnt.data_ptr()),
                                               n_expert, in_feat, out_feat, dt, _stream(input_buf)))
    return [grad_in, grad_w, grad_b]


def linear_act_forward(input_buf, expert_count, weight, bias, activation, keep_pre=True):
    """``pre = X @ W_e^T + b_e`` per expert segment and ``y = act(pre)`` in one grouped GEMM
    (the activation runs in its epilogue).  Returns ``(y, pre)``; ``pre`` is ``None`` when
    ``keep_pre`` is false.  ``activation`` is an ``ACT_*`` code of :mod:`fastermoe_amd._lib`."""
    dt, n_expert, out_feat, in_feat = _check_linear(input_buf, expert_count, weight, bias)
    if activation not in (_lib.ACT_NONE, _lib.ACT_RELU, _lib.ACT_GELU):
        raise ValueError(f"unknown activation code {activation}")
    new = lambda: torch.empty(input_buf.shape[0], out_feat, dtype=input_buf.dtype, device=input_buf.device)
    y = new()
    pre = new() if keep_pre else None
    cnt = _linear_counts(input_buf, expert_count, n_expert)
    with torch.cuda.device(input_buf.device):
        check(_lib.load().fmoe_linear_act_forward(_ptr(input_buf), _ptr(weight), _ptr(bias), _ptr(pre), _ptr(y),
                                                  ctypes.c_void_p(cnt.data_ptr()), n_expert, in_feat, out_feat, dt,
                                                  activation, _stream(input_buf)))
    return y, pre


def linear_dact_backward(grad_output_buf, expert_count, weight, pre, activation):
    """``(grad_y @ W_e) * act'(pre)`` per expert segment: the data gradient of a linear whose input
    was ``act(pre)``, taken with respect to ``pre``.  ``weight`` is ``[E, out_feat, in_feat]``,
    ``pre`` ``[rows, in_feat]``."""
    if weight.dim() != 3:
        raise ValueError(f"weight must be [num_expert, out_feat, in_feat], got {tuple(weight.shape)}")
    n_expert, out_feat, in_feat = weight.shape
    dt = _rows("grad_output_buf", grad_output_buf)
    _dev("weight", weight, grad_output_buf.dtype)
    if grad_output_buf.shape[1] != out_feat:
        raise ValueError(f"grad_output_buf has {grad_output_buf.shape[1]} features, weight produces {out_feat}")
    cnt = _host_counts("expert_count", expert_count, n_expert)
    if int(cnt.sum()) > grad_output_buf.shape[0]:
        raise ValueError("expert_count sums to more rows than grad_output_buf has")
    if activation != _lib.ACT_NONE:
        _dev("pre", pre, grad_output_buf.dtype)
        if tuple(pre.shape) != (grad_output_buf.shape[0], in_feat):
            raise ValueError(f"pre must be [{grad_output_buf.shape[0]}, {in_feat}]")
    grad_x = torch.empty(grad_output_buf.shape[0], in_feat, dtype=grad_output_buf.dtype, device=grad_output_buf.device)
    with torch.cuda.device(grad_output_buf.device):
        check(_lib.load().fmoe_linear_dact_backward(_ptr(grad_output_buf), _ptr(weight),
                                                    _ptr(pre if activation != _lib.ACT_NONE else None), _ptr(grad_x),
                                                    ctypes.c_void_p(cnt.data_ptr()), n_expert, in_feat, out_feat, dt,
                                                    activation, _stream(grad_output_buf)))
    return grad_x


def linear_weight_backward(grad_output_buf, input_buf, expert_count, weight, bias=None):
    """The weight (and bias) half of :func:`linear_backward`: ``[grad_weight, grad_bias]``."""
    dt, n_expert, out_feat, in_feat = _check_linear(input_buf, expert_count, weight, bias)
    cnt = _linear_counts(input_buf, expert_count, n_expert)
    _dev("grad_output_buf", grad_output_buf, input_buf.dtype)
    if tuple(grad_output_buf.shape) != (input_buf.shape[0], out_feat):
        raise ValueError(f"grad_output_buf must be [{input_buf.shape[0]}, {out_feat}]")
    grad_w = torch.empty_like(weight)
    grad_b = torch.empty(n_expert, out_feat, dtype=input_buf.dtype, device=input_buf.device) \
        if bias is not None else None
    with torch.cuda.device(input_buf.device):
        check(_lib.load().fmoe_linear_backward(_ptr(grad_output_buf), _ptr(input_buf), _ptr(weight), None,
                                               _ptr(grad_w), _ptr(grad_b), ctypes.c_void_p(cnt.data_ptr()),
                                               n_expert, in_feat, out_feat, dt, _stream(input_buf)))
    return [grad_w, grad_b]


# ---- per-expert linear over a segment table in device memory ------------------------------

def segment_table(expert_count, rows_cap):
    """The row segments of ``expert_count`` (int64 ``[E]``, on the device) as the int32 table the
    ``*_dev`` products read: built by one small kernel, nothing is read back.  ``rows_cap`` bounds
    the sum of the counts (counts beyond it are clamped)."""
    _dev("expert_count", expert_count, torch.int64)
    lib = _lib.load()
    n_expert = expert_count.numel()
    nbytes = lib.fmoe_segment_table_bytes(int(rows_cap), n_expert)
    with torch.cuda.device(expert_count.device):
        table = torch.empty(nbytes // 4, dtype=torch.int32, device=expert_count.device)
        check(lib.fmoe_segment_table_build(_ptr(expert_count), n_expert, int(rows_cap), _ptr(table), nbytes,
                                           _stream(expert_count)))
    return table


def linear_dev_supported(in_feat, out_feat, dtype):
    """Whether the ``*_dev`` products take this shape (else: the host-count entry points)."""
    return dtype in _DTYPES and _lib.load().fmoe_linear_dev_supported(int(in_feat), int(out_feat), _DTYPES[dtype]) == 1


def _dev_workspace(contraction, dt, device):
    """The caller-side workspace of the row-ragged ``*_dev`` products (``None`` when this contraction is
    never split); torch's caching allocator hands the same block back call after call."""
    import os
    nbytes = _lib.load().fmoe_linear_dev_workspace_bytes(int(contraction), dt)
    if nbytes == 0 or os.environ.get("FMOE_DEV_SPLIT", "1") == "0":
        return None
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def _check_table(table, n_expert, rows_cap):
    _dev("segment_table", table, torch.int32)
    need = _lib.load().fmoe_segment_table_bytes(int(rows_cap), int(n_expert)) // 4
    if table.numel() < need:
        raise ValueError(f"segment_table has {table.numel()} entries, {need} needed for {rows_cap} rows / {n_expert} experts")


def linear_forward_dev(x, weight, bias, table, rows_cap, activation=_lib.ACT_NONE, keep_pre=False,
                       row_index=None, index_div=1):
    """``y = act(x @ W_e^T + b_e)`` per expert segment of ``table``; returns ``(y, pre)`` with ``pre``
    the pre-activation when ``keep_pre``.  With ``row_index`` (int64 ``[rows_cap]``) sorted row ``r`` is
    read from ``x[row_index[r] // index_div]`` in the GEMM's loader.  Outputs have ``rows_cap`` rows,
    of which only the table's rows are written."""
    dt = _rows("x", x)
    _dev("weight", weight, x.dtype)
    if weight.dim() != 3 or weight.shape[2] != x.shape[1]:
        raise ValueError(f"weight must be [num_expert, out_feat, {x.shape[1]}], got {tuple(weight.shape)}")
    n_expert, out_feat, in_feat = weight.shape
    if bias is not None:
        _dev("bias", bias, x.dtype)
        if tuple(bias.shape) != (n_expert, out_feat):
            raise ValueError(f"bias must be [{n_expert}, {out_feat}], got {tuple(bias.shape)}")
    _check_table(table, n_expert, rows_cap)
    if row_index is not None:
        _dev("row_index", row_index, torch.int64)
        if row_index.numel() < rows_cap:
            raise ValueError("row_index must have one entry per row")
    elif x.shape[0] < rows_cap:
        raise ValueError(f"x has {x.shape[0]} rows, rows_cap is {rows_cap}")
    new = lambda: torch.empty(rows_cap, out_feat, dtype=x.dtype, device=x.device)
    y = new()
    pre = new() if keep_pre else None
    with torch.cuda.device(x.device):
        ws = _dev_workspace(in_feat, dt, x.device)
        check(_lib.load().fmoe_linear_forward_dev(_ptr(x), _ptr(row_index), int(index_div), x.shape[0], _ptr(weight),
                                                  _ptr(bias), _ptr(pre), _ptr(y), _ptr(table), n_expert, int(rows_cap),
                                                  in_feat, out_feat, dt, activation, _ptr(ws),
                                                  0 if ws is None else ws.numel(), _stream(x)))
    return y, pre


def linear_dgrad_dev(grad_y, weight, table, rows_cap, pre=None, activation=_lib.ACT_NONE):
    """``(grad_y @ W_e) * act'(pre)`` per expert segment of ``table`` (no activation: the plain
    data gradient)."""
    dt = _rows("grad_y", grad_y)
    _dev("weight", weight, grad_y.dtype)
    if weight.dim() != 3 or weight.shape[1] != grad_y.shape[1]:
        raise ValueError(f"weight must be [num_expert, {grad_y.shape[1]}, in_feat], got {tuple(weight.shape)}")
    n_expert, out_feat, in_feat = weight.shape
    _check_table(table, n_expert, rows_cap)
    if grad_y.shape[0] < rows_cap:
        raise ValueError(f"grad_y has {grad_y.shape[0]} rows, rows_cap is {rows_cap}")
    if activation != _lib.ACT_NONE:
        _dev("pre", pre, grad_y.dtype)
        if pre.dim() != 2 or pre.shape[0] < rows_cap or pre.shape[1] != in_feat:
            raise ValueError(f"pre must be [>= {rows_cap}, {in_feat}]")
    grad_x = torch.empty(rows_cap, in_feat, dtype=grad_y.dtype, device=grad_y.device)
    with torch.cuda.device(grad_y.device):
        ws = _dev_workspace(out_feat, dt, grad_y.device)
        check(_lib.load().fmoe_linear_dgrad_dev(_ptr(grad_y), _ptr(weight),
                                                _ptr(pre if activation != _lib.ACT_NONE else None), _ptr(grad_x),
                                                _ptr(table), n_expert, int(rows_cap), in_feat, out_feat, dt, activation,
                                                _ptr(ws), 0 if ws is None else ws.numel(), _stream(grad_y)))
    return grad_x


def linear_wgrad_dev(grad_y, x, weight, table, rows_cap, with_bias):
    """``[grad_weight, grad_bias]`` of a per-expert linear over the segments of ``table``
    (``grad_bias`` is ``None`` unless ``with_bias``); ``weight`` only gives the shape."""
    dt = _rows("x", x)
    _dev("grad_y", grad_y, x.dtype)
    n_expert, out_feat, in_feat = weight.shape
    if x.shape[1] != in_feat or grad_y.shape[1] != out_feat or x.shape[0] < rows_cap or grad_y.shape[0] < rows_cap:
        raise ValueError(f"x must be [>= {rows_cap}, {in_feat}] and grad_y [>= {rows_cap}, {out_feat}]")
    _check_table(table, n_expert, rows_cap)
    grad_w = torch.empty(n_expert, out_feat, in_feat, dtype=x.dtype, device=x.device)
    grad_b = torch.empty(n_expert, out_feat, dtype=x.dtype, device=x.device) if with_bias else None
    with torch.cuda.device(x.device):
        check(_lib.load().fmoe_linear_wgrad_dev(_ptr(grad_y), _ptr(x), _ptr(grad_w), _ptr(grad_b), _ptr(table), n_expert,
                                                int(rows_cap), in_feat, out_feat, dt, _stream(x)))
    return grad_w, grad_b


# ---- fused expert MLP (chunked, stream-overlapped pipeline) -------------------------

def _mlp_params(w1, b1, w2, b2, activation):
    dt = _float_dtype("w1", _dev("w1", w1))
    _dev("w2", w2, w1.dtype)
    if w1.dim() != 3 or w2.dim() != 3:
        raise ValueError("w1 / w2 must be [num_expert, out_feat, in_feat]")
    n_expert, d_hidden, d_model = w1.shape
    if tuple(w2.shape) != (n_expert, d_model, d_hidden):
        raise ValueError(f"w2 must be [{n_expert}, {d_model}, {d_hidden}], got {tuple(w2.shape)}")
    for name, b, width in (("b1", b1, d_hidden), ("b2", b2, d_model)):
        if b is not None:
            _dev(name, b, w1.dtype)
            if tuple(b.shape) != (n_expert, width):
                raise ValueError(f"{name} must be [{n_expert}, {width}]")
    if dt == _lib.F64:
        raise TypeError("the fused expert MLP supports float32, bfloat16 and float16")
    if activation not in (_lib.ACT_NONE, _lib.ACT_RELU, _lib.ACT_GELU):
        raise ValueError(f"unknown activation code {activation}")
    prm = _lib.MlpParams(w1.data_ptr(), b1.data_ptr() if b1 is not None else None, w2.data_ptr(),
                         b2.data_ptr() if b2 is not None else None, n_expert, d_model, d_hidden, dt, activation)
    return prm, n_expert, d_model, d_hidden


def fused_mlp_forward(inp, pos, slot_to_row, expert_count, w1, b1, w2, b2, top_k, activation, n_chunks,
                      slot_order=True):
    """scatter -> Linear -> activation -> Linear -> gather as one pipelined call.
    Returns ``(out [N*top_k, d], buf_in, buf_pre or None, buf_mid)``; the three
    buffers are what the backward needs.  ``buf_in`` is ``None`` when the first GEMM read the
    token rows through ``pos`` in its loader (no sorted copy of the input exists; the backward
    makes one from ``inp``).  With ``slot_order=False`` the copy to slot order is skipped and
    ``out`` is the experts' output in expert-sorted order, ``[n_rows, d]``."""
    import os
    prm, n_expert, d_model, d_hidden = _mlp_params(w1, b1, w2, b2, activation)
    _dev("inp", inp, w1.dtype)
    _dev("pos", pos, torch.int64)
    _dev("slot_to_row", slot_to_row, torch.int64)
    if inp.dim() != 2 or inp.shape[1] != d_model:
        raise ValueError(f"inp must be [n_tokens, {d_model}]")
    # ``pos`` may be the whole position buffer (one entry per slot, the routed slots first): the buffers
    # then hold a row per slot and the counts say how many of them are used.  The counts are read last:
    # they may still be on their way from the device.
    n_tokens, cap = inp.shape[0], pos.numel()
    if slot_to_row.numel() != n_tokens * top_k:
        raise ValueError("slot_to_row must have n_tokens * top_k entries")
    new = lambda r, c: torch.empty(r, c, dtype=inp.dtype, device=inp.device)
    lib = _lib.load()
    in_loader = (os.environ.get("FMOE_FOLD_SCATTER", "1") != "0" and cap > 0
                 and lib.fmoe_fused_scatter_in_loader(ctypes.byref(prm), _ptr(inp), n_tokens) == 1)
    buf_in = None if in_loader else new(cap, d_model)
    buf_mid, buf_out = new(cap, d_hidden), new(cap, d_model)
    buf_pre = new(cap, d_hidden) if activation == _lib.ACT_GELU else None
    out = new(n_tokens * top_k, d_model) if slot_order else None
    cnt = _host_counts("expert_count", expert_count, n_expert)
    n_rows = int(cnt.sum())
    if n_rows > cap:
        raise ValueError(f"expert_count sums to {n_rows} but pos has {cap} entries")
    with torch.cuda.device(inp.device):
        check(lib.fmoe_fused_mlp_forward(
            ctypes.byref(prm), _ptr(inp), _ptr(pos), _ptr(slot_to_row), ctypes.c_void_p(cnt.data_ptr()),
            n_tokens, top_k, n_rows, _ptr(buf_in), _ptr(buf_pre), _ptr(buf_mid), _ptr(buf_out), _ptr(out),
            n_chunks, _stream(inp)))
    return (out if slot_order else buf_out), buf_in, buf_pre, buf_mid


def fused_mlp_backward(grad_out, pos, slot_to_row, expert_count, w1, b1, w2, b2, buf_in, buf_pre, buf_mid,
                       n_tokens, top_k, activation, n_chunks, slot_order=True, inp=None):
    """Backward of :func:`fused_mlp_forward`.  Returns
    ``(grad_inp, grad_w1, grad_b1, grad_w2, grad_b2)`` (bias grads ``None``
    without biases).  For ReLU the post-activation buffer doubles as the
    pre-activation (same sign pattern).  With ``slot_order=False``, ``grad_out``
    is already in expert-sorted order, ``[n_rows, d]``.  ``buf_in=None``: the forward kept no
    sorted copy of the input; it is rebuilt here from ``inp`` ``[n_tokens, d]``."""
    prm, n_expert, d_model, d_hidden = _mlp_params(w1, b1, w2, b2, activation)
    _dev("grad_out", grad_out, w1.dtype)
    cnt = _host_counts("expert_count", expert_count, n_expert)
    n_rows, cap = int(cnt.sum()), pos.numel()   # pos may be the whole position buffer (see the forward)
    if n_rows > cap:
        raise ValueError(f"expert_count sums to {n_rows} but pos has {cap} entries")
    want = (n_tokens * top_k, d_model) if slot_order else (cap, d_model)
    if tuple(grad_out.shape) != want:
        raise ValueError(f"grad_out must be [{want[0]}, {want[1]}]")
    pre = buf_pre if buf_pre is not None else buf_mid
    dev, dty = grad_out.device, grad_out.dtype
    new = lambda *s: torch.empty(*s, dtype=dty, device=dev)
    regather = buf_in is None
    if regather:
        if inp is None:
            raise ValueError("fused_mlp_backward: neither buf_in nor inp")
        _dev("inp", inp, w1.dtype)
        buf_in = new(cap, d_model)
    g_out = new(cap, d_model) if slot_order else grad_out
    g_mid, g_in = new(cap, d_hidden), new(cap, d_model)
    grad_inp = new(n_tokens, d_model)
    grad_w1, grad_w2 = torch.empty_like(w1), torch.empty_like(w2)
    grad_b1 = torch.empty_like(b1) if b1 is not None else None
    grad_b2 = torch.empty_like(b2) if b2 is not None else None
    with torch.cuda.device(dev):
        check(_lib.load().fmoe_fused_mlp_backward(
            ctypes.byref(prm), _ptr(grad_out if slot_order else None), _ptr(pos), _ptr(slot_to_row),
            ctypes.c_void_p(cnt.data_ptr()),
            n_tokens, top_k, n_rows, _ptr(inp if regather else None), _ptr(buf_in), _ptr(pre), _ptr(buf_mid),
            _ptr(g_out), _ptr(g_mid), _ptr(g_in),
            _ptr(grad_inp), _ptr(grad_w1), _ptr(grad_b1), _ptr(grad_w2), _ptr(grad_b2), n_chunks,
            _stream(grad_out)))
    return grad_inp, grad_w1, grad_b1, grad_w2, grad_b2


def _fuse_chunks():
    import os
    gran = os.environ.get("FMOE_FUSE_GRAN")
    return 0 if gran is None else max(1, int(gran))  # 0: the library chooses


def _unpack_params(params, has_bias):
    expert = params[0][0]
    if has_bias:
        w1, b1, w2, b2 = expert
    else:
        w1, w2 = expert[0], expert[len(expert) // 2]
        b1 = b2 = None
    return w1, b1, w2, b2


def fused_forward(input_buf, params, local_expert_count, global_expert_count, stored_models,
                  global_batch_size, n_workers, has_bias):
    """fmoe_cuda.fused_forward (cuda/fused_compute.cu:12-62) for one worker:
    ``input_buf`` is already expert-sorted, the activation is ReLU as in the
    reference kernel (cuda/fused_compute.cuh:20-44).  Returns
    ``[output_buf, global_input_buf, global_middle_buf, global_output_buf]``."""
    if n_workers != 1:
        raise NotImplementedError("fused_forward: one worker only")
    w1, b1, w2, b2 = _unpack_params(params, has_bias)
    rows = input_buf.shape[0]
    ident = torch.arange(rows, dtype=torch.int64, device=input_buf.device)
    input_buf = input_buf.contiguous()
    out, buf_in, _pre, buf_mid = fused_mlp_forward(input_buf, ident, ident, global_expert_count,
                                                   w1, b1, w2, b2, 1, _lib.ACT_RELU, _fuse_chunks())
    # global_input_buf of the reference: with the identity permutation it is the input itself
    return [out, buf_in if buf_in is not None else input_buf, buf_mid, out]


def fused_backward(input_buf, params, middle_buf, output_buf, grad_out, local_expert_count,
                   global_expert_count, inp, stored_models, global_batch_size, buf_batch_size,
                   n_workers, has_bias):
    """fmoe_cuda.fused_backward (cuda/fused_compute.cu:64-131) for one worker.
    Returns ``[grad_in]`` and, like the reference, leaves the weight gradients
    in ``param.grad`` -- ADDED to an existing ``.grad`` (the reference overwrites
    it on its first pipeline step, cuda/fused_compute.cuh:123)."""
    if n_workers != 1:
        raise NotImplementedError("fused_backward: one worker only")
    w1, b1, w2, b2 = _unpack_params(params, has_bias)
    rows = input_buf.shape[0]
    ident = torch.arange(rows, dtype=torch.int64, device=input_buf.device)
    grad_in, gw1, gb1, gw2, gb2 = fused_mlp_backward(
        grad_out.contiguous(), ident, ident, global_expert_count, w1, b1, w2, b2, input_buf, None, middle_buf,
        rows, 1, _lib.ACT_RELU, _fuse_chunks())
    for prm, g in ((w1, gw1), (b1, gb1), (w2, gw2), (b2, gb2)):
        if prm is None:
            continue
        if prm.grad is None:
            prm.grad = g
        else:
            prm.grad.add_(g)
    return [grad_in]
