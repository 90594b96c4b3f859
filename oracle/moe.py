"""Brute-force MoE MLP oracle (torch, CPU).

TEST INFRASTRUCTURE ONLY (see the package docstring).

``brute_force_moe_mlp`` restates the reference's ``BruteForceMoELinear.forward``
(tests/moe.py:30-49): every token is repeated ``top_k`` times, each expert takes
the rows whose gate index names it (boolean mask), applies
``Linear -> activation -> Linear`` with its own weights and biases, and the
``top_k`` results of a token are combined with ``bmm`` by the gate scores.
One deliberate difference: rows whose gate index is -1 (dropped by a capacity
gate) are ZERO, not uninitialised (``torch.empty`` at tests/moe.py:34), because
the layer under test zero-fills them (fmoe/functions.py:78).

Gradients come from torch autograd on this forward, as in the reference's tests
(tests/test_numerical.py:45-46: ``out.mean().backward()``).

Pinning (tests/test_oracle.py): against a dense one-hot formulation that shares
no code with the masked loop (einsum over all experts, then select), against a
hand-worked 2-token case, and against ``torch.nn.Linear``/``nn.Sequential`` when
there is a single expert.  ``moe_mlp_forward_backward_per_expert`` (the same
forward with the textbook backward written out, one expert at a time, for shapes
whose float64 autograd graph would not fit in memory) is pinned against the
autograd version on small shapes.
"""
import time

import torch
import torch.nn.functional as F


def resolve_activation(activation):
    if callable(activation):
        return activation
    if activation == "gelu":
        return F.gelu
    if activation == "relu":
        return F.relu
    raise ValueError(activation)


def brute_force_moe_mlp(inp, gate_idx, gate_score, w1, b1, w2, b2, activation, top_k):
    """inp [N,d]; gate_idx int64 [N,k] or [N*k]; gate_score [N,k];
    w1 [E,h,d], b1 [E,h] or None, w2 [E,d,h], b2 [E,d] or None -> [N,d]."""
    act = resolve_activation(activation)
    d_model = inp.shape[1]
    rep = inp.repeat_interleave(repeats=top_k, dim=0)
    gate_long = gate_idx.long().reshape(-1)
    o = torch.zeros(rep.shape[0], d_model, dtype=inp.dtype, device=inp.device)
    for i in range(w1.shape[0]):
        idx = gate_long == i
        x = rep[idx]
        x = x @ w1[i].t()
        if b1 is not None:
            x = x + b1[i]
        x = act(x)
        x = x @ w2[i].t()
        if b2 is not None:
            x = x + b2[i]
        o[idx] = x
    score = gate_score.reshape(-1, 1, top_k).to(o.dtype)
    return torch.bmm(score, o.view(-1, top_k, d_model)).reshape(-1, d_model)


def moe_mlp_forward_backward(inp, gate_idx, gate_score, w1, b1, w2, b2, activation, top_k,
                             dtype=torch.float64, loss="mean"):
    """Runs the oracle in ``dtype`` with autograd and returns a dict with
    ``out, grad_inp, grad_w1, grad_b1, grad_w2, grad_b2`` (biases may be None)."""
    def leaf(t):
        return None if t is None else t.detach().to("cpu", dtype).clone().requires_grad_(True)
    x, W1, B1, W2, B2 = leaf(inp), leaf(w1), leaf(b1), leaf(w2), leaf(b2)
    score = gate_score.detach().to("cpu", dtype)
    out = brute_force_moe_mlp(x, gate_idx.detach().cpu(), score, W1, B1, W2, B2, activation, top_k)
    (out.mean() if loss == "mean" else out.sum()).backward()
    g = lambda t: None if t is None else t.grad
    return {"out": out.detach(), "grad_inp": x.grad, "grad_w1": W1.grad, "grad_b1": g(B1),
            "grad_w2": W2.grad, "grad_b2": g(B2)}


def moe_mlp_forward_backward_per_expert(inp, gate_idx, gate_score, w1, b1, w2, b2, activation, top_k,
                                        grad_out=None, grad_dtype=torch.float64):
    """Same results as ``moe_mlp_forward_backward`` (float64, ``out.mean()`` as the loss
    unless ``grad_out`` [N,d] is given), computed one expert at a time with the backward of
    ``Linear -> activation -> Linear`` and of the score-weighted sum written out, so that
    only one expert's weights are held in float64 at a time.  ``activation``: "gelu"
    (exact) or "relu".  Gate scores get no gradient here.  The weight gradients are stored
    in ``grad_dtype`` (float32 halves the memory of very large layers)."""
    f64 = torch.float64
    x = inp.detach().to("cpu", f64)
    n, d = x.shape
    idx = gate_idx.detach().cpu().long().reshape(-1)
    score = gate_score.detach().to("cpu", f64).reshape(-1)
    g_out = torch.full((n, d), 1.0 / (n * d), dtype=f64) if grad_out is None else grad_out.detach().to("cpu", f64)
    out = torch.zeros(n, d, dtype=f64)
    res = {"out": out, "grad_inp": torch.zeros(n, d, dtype=f64),
           "grad_w1": torch.zeros(w1.shape, dtype=grad_dtype), "grad_w2": torch.zeros(w2.shape, dtype=grad_dtype),
           "grad_b1": None if b1 is None else torch.zeros(b1.shape, dtype=f64),
           "grad_b2": None if b2 is None else torch.zeros(b2.shape, dtype=f64)}
    for e in range(w1.shape[0]):
        slots = torch.nonzero(idx == e).reshape(-1)
        if slots.numel() == 0:
            continue
        tok = slots // top_k
        W1, W2 = w1[e].detach().to("cpu", f64), w2[e].detach().to("cpu", f64)
        xe = x[tok]
        pre = xe @ W1.t()
        if b1 is not None:
            pre = pre + b1[e].detach().to("cpu", f64)
        if activation == "gelu":
            cdf = 0.5 * (1.0 + torch.erf(pre / 2.0 ** 0.5))
            mid = pre * cdf
            dact = cdf + pre * torch.exp(-0.5 * pre * pre) / (2.0 * torch.pi) ** 0.5
        elif activation == "relu":
            mid = pre.clamp_min(0.0)
            dact = (pre > 0).to(f64)
        else:
            raise ValueError(activation)
        y = mid @ W2.t()
        if b2 is not None:
            y = y + b2[e].detach().to("cpu", f64)
        sc = score[slots].unsqueeze(1)
        out.index_add_(0, tok, sc * y)
        gy = sc * g_out[tok]
        res["grad_w2"][e] = gy.t() @ mid
        g_pre = (gy @ W2) * dact
        res["grad_w1"][e] = g_pre.t() @ xe
        if b2 is not None:
            res["grad_b2"][e] = gy.sum(0)
        if b1 is not None:
            res["grad_b1"][e] = g_pre.sum(0)
        res["grad_inp"].index_add_(0, tok, g_pre @ W1)
    return res


def per_expert_linear(inp_sorted, counts, weight, bias):
    """fmoe_cuda.linear_forward (cuda/parallel_linear.cuh:55-88): rows are already
    grouped by expert; segment e is ``counts[e]`` rows long."""
    outs = []
    ptr = 0
    for e, n in enumerate([int(c) for c in counts]):
        seg = inp_sorted[ptr:ptr + n] @ weight[e].t()
        if bias is not None:
            seg = seg + bias[e]
        outs.append(seg)
        ptr += n
    return torch.cat(outs, dim=0) if outs else inp_sorted.new_zeros(0, weight.shape[1])


def time_cpu_baseline(n_tokens, d_model, d_hidden, n_expert, top_k, activation="gelu",
                      seed=0, repeats=1, threads=None, warmup=0, return_median=False):
    """Wall-clock fwd+bwd of the brute-force oracle in fp32 on the host cores: ``warmup`` untimed
    iterations, then ``repeats`` timed ones.  Returns (tokens_per_second of the best iteration,
    cores_used, seconds of the best iteration[, seconds of the median iteration])."""
    import os
    threads = threads or os.cpu_count()
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n_tokens, d_model, generator=g)
    logits = torch.randn(n_tokens, n_expert, generator=g)
    val, idx = torch.topk(logits, top_k, dim=-1)
    score = torch.softmax(val, dim=-1)
    bound1, bound2 = (d_hidden * d_model) ** -0.5, (d_hidden * d_model) ** -0.5
    w1 = (torch.rand(n_expert, d_hidden, d_model, generator=g) * 2 - 1) * bound1
    w2 = (torch.rand(n_expert, d_model, d_hidden, generator=g) * 2 - 1) * bound2
    b1 = torch.zeros(n_expert, d_hidden)
    b2 = torch.zeros(n_expert, d_model)
    times = []
    for it in range(warmup + repeats):
        t0 = time.perf_counter()
        moe_mlp_forward_backward(x, idx, score, w1, b1, w2, b2, activation, top_k,
                                 dtype=torch.float32, loss="sum")
        if it >= warmup:
            times.append(time.perf_counter() - t0)
    times.sort()
    best, median = times[0], times[len(times) // 2]
    if return_median:
        return n_tokens / best, threads, best, median
    return n_tokens / best, threads, best
