"""GPU parity of the routing / capacity kernels: bit-exact against the CPU oracle
and the committed golden cases, through the operator module (which calls the C ABI)."""
import json
import os

import numpy as np
import pytest
import torch

from fastermoe_amd import fmoe_native
from fastermoe_amd.functions import count_by_gate, prepare_forward
from fastermoe_amd.gates.utils import limit_by_capacity
from oracle import routing as orouting
from helpers import TOL, rel_err

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "routing_cases.json")


def _cases():
    with open(GOLDEN) as f:
        return json.load(f)


def _dev(a, device, dtype):
    return torch.as_tensor(np.asarray(a), dtype=dtype).to(device)


@pytest.mark.parametrize("case", _cases(), ids=lambda c: c["name"])
def test_golden_cases(case, device):
    e = case["n_expert"]
    gate = _dev(case["gate"], device, torch.int64)
    cnt = torch.zeros(e, dtype=torch.int32, device=device)
    fmoe_native.expert_count(gate, cnt)
    assert cnt.cpu().tolist() == case["counts"]
    cum = torch.cumsum(cnt.long(), 0).int()
    pos = torch.full((sum(case["counts"]),), -7, dtype=torch.int64, device=device)
    fmoe_native.assign_pos(cum, gate, pos)
    assert pos.cpu().tolist() == case["pos"]
    if len(case["gate"]):
        assert cum.cpu().tolist() == case["cum_after"]
    cap = torch.full((e,), case["capacity"], dtype=torch.int32, device=device)
    lim = fmoe_native.limit_by_capacity(cnt.long(), cap, e, 1)
    assert lim.cpu().tolist() == case["limited"]
    ec = lim.int()
    pruned = fmoe_native.prune_gate_by_capacity(gate, ec, e, 1)
    assert pruned.cpu().tolist() == case["pruned"]
    if len(case["gate"]):
        assert ec.cpu().tolist() == case["cap_after"]
    # fused route
    c2, pos2, s2r = fmoe_native.route(gate, e)
    assert c2.cpu().tolist() == case["counts"]
    total = sum(case["counts"])
    assert pos2[:total].cpu().tolist() == case["pos"]
    inv = [-1] * len(case["gate"])
    for row, slot in enumerate(case["pos"]):
        inv[slot] = row
    assert s2r.cpu().tolist() == inv


SHAPES = [  # (n_tokens, top_k, n_expert, drop_fraction)
    (4096, 2, 8, 0.0),       # config 1
    (16384, 2, 16, 0.0),     # config 2
    (16384, 1, 64, 0.0),     # config 3 (Zipf below)
    (32768, 2, 8, 0.0),      # config 4
    (8192, 8, 256, 0.0),     # config 5
    (1000, 3, 7, 0.3),       # ragged sizes, dropped slots
    (2049, 1, 1, 0.0),       # one expert, one slot past a workgroup boundary
    (63, 2, 300, 0.1),       # more experts than slots
    (5000, 2, 8192, 0.0),    # largest supported expert count
]


@pytest.mark.parametrize("n,k,e,drop", SHAPES)
def test_route_bit_exact(n, k, e, drop, device):
    rng = np.random.default_rng(n + k + e)
    if e == 64:
        p = (np.arange(1, e + 1) ** -1.2)
        gate = rng.permutation(e)[rng.choice(e, size=(n, k), p=p / p.sum())]
    else:
        gate = rng.integers(0, e, size=(n, k))
    gate = gate.astype(np.int64)
    gate[rng.random((n, k)) < drop] = -1
    ref_pos, ref_cnt = orouting.count_by_gate(gate, e)
    g = torch.from_numpy(gate).to(device)
    if k == 1:
        g = g.view(-1)

    pos, lec, all_ec, gec, all_gec = count_by_gate(g, e, 1)
    assert lec.dtype == torch.int64 and pos.dtype == torch.int64
    assert np.array_equal(lec.cpu().numpy(), ref_cnt)
    assert np.array_equal(pos.cpu().numpy(), ref_pos)
    assert gec is lec and all_ec is lec

    # the separate entry points, as fmoe/functions.py:19-42 strings them together
    cnt32 = torch.zeros(e, dtype=torch.int32, device=device)
    fmoe_native.expert_count(g, cnt32)
    fmoe_native.expert_count(g, cnt32)          # accumulates
    assert np.array_equal(cnt32.cpu().numpy(), 2 * ref_cnt)
    cum = torch.cumsum(torch.from_numpy(ref_cnt), 0).int().to(device)
    pos2 = torch.empty(int(ref_cnt.sum()), dtype=torch.int64, device=device)
    fmoe_native.assign_pos(cum, g, pos2)
    assert np.array_equal(pos2.cpu().numpy(), ref_pos)
    assert np.array_equal(cum.cpu().numpy(), (np.cumsum(ref_cnt) - ref_cnt).astype(np.int32))

    out = prepare_forward(g, e, 1)
    assert len(out) == 6 and all(not t.is_cuda for t in out[1:])
    assert np.array_equal(out[5].numpy(), ref_cnt)

    # the whole position buffer: routed slots first, -1 for the entries dropped slots leave unused
    cnt, pos_buf, s2r = fmoe_native.route(g, e)
    total = int(ref_cnt.sum())
    assert pos_buf.numel() == n * k and np.array_equal(pos_buf[:total].cpu().numpy(), ref_pos)
    assert bool((pos_buf[total:] == -1).all())


@pytest.mark.parametrize("n,k,e,cap", [(16384, 2, 16, 2458), (16384, 1, 64, 300), (8192, 8, 256, 100),
                                       (777, 2, 5, 0), (4096, 2, 8, 10 ** 6)])
def test_limit_and_prune_bit_exact(n, k, e, cap, device):
    rng = np.random.default_rng(cap % 1000 + n)
    gate = rng.integers(0, e, size=(n, k)).astype(np.int64)
    ref_lec, ref_gec, ref_pruned = orouting.limit_and_prune(gate, e, cap)
    g = torch.from_numpy(gate).to(device)
    new_lec, new_gec, pruned = limit_by_capacity(g, e, 1, cap)
    assert np.array_equal(new_gec.cpu().numpy(), ref_gec)
    assert np.array_equal(new_lec.cpu().numpy(), ref_lec)
    assert pruned.shape == g.shape and pruned.dtype == torch.int64
    assert np.array_equal(pruned.cpu().numpy(), ref_pruned)
    kept = np.bincount(ref_pruned[ref_pruned >= 0], minlength=e)
    assert np.all(kept <= cap)                       # tests/test_gates.py:51-57
    assert np.array_equal(g.cpu().numpy(), gate)     # input untouched, new tensor returned


def test_limit_by_capacity_several_workers(device):
    rng = np.random.default_rng(11)
    e, w = 37, 5
    ec = rng.integers(0, 50, size=w * e).astype(np.int64)
    cap = rng.integers(0, 120, size=e).astype(np.int32)
    cap_ref = cap.copy()
    ref = orouting.limit_by_capacity(ec, cap_ref, e, w)
    cap_dev = torch.from_numpy(cap).to(device)
    got = fmoe_native.limit_by_capacity(torch.from_numpy(ec).to(device), cap_dev, e, w)
    assert np.array_equal(got.cpu().numpy(), ref)
    assert np.array_equal(cap_dev.cpu().numpy(), cap_ref)


def test_prune_with_existing_drops_and_state(device):
    rng = np.random.default_rng(5)
    e = 12
    gate = rng.integers(-1, e, size=5000).astype(np.int64)
    ec = rng.integers(0, 300, size=e).astype(np.int32)
    ec_ref = ec.copy()
    ref = orouting.prune_gate_by_capacity(gate, ec_ref)
    ec_dev = torch.from_numpy(ec).to(device)
    got = fmoe_native.prune_gate_by_capacity(torch.from_numpy(gate).to(device), ec_dev, e, 1)
    assert np.array_equal(got.cpu().numpy(), ref)
    assert np.array_equal(ec_dev.cpu().numpy(), ec_ref)


def test_full_size_invariants(device):
    """Size-independent properties at the largest configuration (65 536 slots, 256 experts)."""
    torch.manual_seed(0)
    logits = torch.randn(8192, 256) + 0.5 * torch.randn(256)
    gate = torch.topk(logits, 8, dim=-1).indices.to(device)
    cnt, pos_buf, s2r = fmoe_native.route(gate, 256)
    total = int(cnt.sum())
    pos = pos_buf[:total]
    flat = gate.view(-1)
    assert total == flat.numel()
    assert torch.equal(torch.sort(pos).values, torch.arange(total, device=device))
    experts_along_pos = flat[pos]
    assert bool((experts_along_pos[1:] >= experts_along_pos[:-1]).all())
    assert torch.equal(s2r[pos], torch.arange(total, device=device))
    assert torch.equal(cnt, torch.bincount(flat, minlength=256))
    # idempotence of pruning: pruning the pruned gate with the same caps changes nothing
    cap = torch.full((256,), 200, dtype=torch.int32, device=device)
    once = fmoe_native.prune_gate_by_capacity(gate, cap.clone(), 256, 1)
    twice = fmoe_native.prune_gate_by_capacity(once, cap.clone(), 256, 1)
    assert torch.equal(once, twice)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,e,k", [
    (32768, 8, 2),      # the Mixtral-like share
    (8192, 256, 8),     # the fine-grained layer
    (16384, 64, 1),     # top-1
    (16384, 16, 2),
    (1000, 5, 4),       # experts not a power of two, token count not a multiple of a workgroup's share
    (77, 1003, 8),      # rows that do not start on 16-byte boundaries
    (700, 300, 4),
    (3, 2, 2),          # every expert chosen
    (0, 4, 2),
])
def test_gate_topk_route(dtype, n, e, k, device):
    """fmoe_gate_topk_route against torch.topk (tie-free logits, choices by descending logit), the
    scores in both modes, and its expert counts / pos / slot_to_row against the CPU oracle run on
    the SAME index tensor; its backward against autograd through torch.topk and softmax."""
    from fastermoe_amd import fmoe_native
    gen = torch.Generator().manual_seed(n + e + k)
    # distinct values per token, exactly representable in every dtype: consecutive bfloat16 bit patterns
    # (0.0078 .. 2.6, alternating sign), in a random order per token
    table = (torch.arange(e, dtype=torch.int16) + 0x3C00).view(torch.bfloat16).float()
    table = table * (1 - 2 * (torch.arange(e) % 2)).float()
    base = table[torch.argsort(torch.rand(n, e, generator=gen), dim=1)] if n else torch.zeros(0, e)
    logits = base.to(dtype).to(device)
    assert torch.equal(logits.float().cpu(), base)
    for mode in (0, 1):
        idx, score, cnt, pos_buf, s2r = fmoe_native.gate_topk_route(logits, k, mode)
        want_val, want_idx = torch.topk(logits.float(), k, dim=-1, largest=True, sorted=True)
        assert torch.equal(idx, want_idx)
        want_score = torch.softmax(want_val, dim=-1) if mode == 1 else want_val
        if mode == 0:
            assert torch.equal(score.float(), want_score)
        else:
            assert torch.allclose(score.float(), want_score, rtol={torch.float32: 1e-5}.get(dtype, 1e-2), atol=1e-6)
        ref_pos, ref_cnt = orouting.count_by_gate(idx.cpu().numpy(), e)
        assert np.array_equal(cnt.cpu().numpy(), ref_cnt)
        total = int(ref_cnt.sum())
        assert total == n * k
        assert np.array_equal(pos_buf[:total].cpu().numpy(), ref_pos)
        inv = np.full(n * k, -1, dtype=np.int64)
        inv[ref_pos] = np.arange(total)
        assert np.array_equal(s2r.cpu().numpy(), inv)
        if n == 0:
            continue
        # backward: d(sum(score * g)) / d(logits)
        g = torch.randn(n, k, generator=gen).to(dtype).to(device)
        got = fmoe_native.gate_topk_backward(g, score, idx, e, mode)
        leaf = logits.float().clone().requires_grad_(True)
        val, _ = torch.topk(leaf, k, dim=-1, sorted=True)
        sc = torch.softmax(val, dim=-1) if mode == 1 else val
        (sc * g.float()).sum().backward()
        assert torch.allclose(got.float(), leaf.grad, rtol={torch.float32: 1e-5}.get(dtype, 2e-2), atol=1e-2 if dtype != torch.float32 else 1e-6)


def test_gate_topk_ties_go_to_the_lower_expert(device):
    from fastermoe_amd import fmoe_native
    logits = torch.zeros(9, 6, device=device)
    logits[:, 4] = 1.0
    idx, score, cnt, _, _ = fmoe_native.gate_topk_route(logits, 4, 0)
    assert idx.cpu().tolist() == [[4, 0, 1, 2]] * 9
    assert cnt.cpu().tolist() == [9, 9, 9, 0, 9, 0]
    with pytest.raises(ValueError):
        fmoe_native.gate_topk_route(logits, 3, 0)        # not a power of two: torch.topk + route instead


def test_naive_gate_hands_its_routing_to_the_layer(device):
    """NaiveGate's index tensor carries the routing computed with the top-k; the layer's routing step
    uses it only for that very tensor, unmodified, and recomputes otherwise."""
    from fastermoe_amd import functions
    from fastermoe_amd.gates import NaiveGate
    torch.manual_seed(8)
    gate = NaiveGate(32, 8, 1, top_k=2).to(device)
    x = torch.randn(500, 32, device=device)
    idx, val = gate(x)
    assert hasattr(idx, "_fmoe_route")
    pos_a, cnt_a, cnt_cpu_a, s2r_a = functions._route(idx, 8, 1)
    fresh = idx.clone()
    assert not hasattr(fresh, "_fmoe_route")
    pos_b, cnt_b, _, s2r_b = functions._route(fresh, 8, 1)
    assert torch.equal(pos_a, pos_b) and torch.equal(cnt_a, cnt_b) and torch.equal(s2r_a, s2r_b)
    idx[0, 0] = -1                                       # an in-place edit invalidates what rides on the tensor
    pos_c, cnt_c, _, _ = functions._route(idx, 8, 1)
    assert int(cnt_c.sum()) == 999
    # scores are differentiable: the gate's weight gets a gradient through the selected logits
    idx2, val2 = gate(x)
    val2.sum().backward()
    assert gate.gate.weight.grad is not None and torch.isfinite(gate.gate.weight.grad).all()
    logits = gate.gate(x)
    # (the gate's linear layer ran inside the top-k kernel: same logits up to the order of the fp32 sums)
    assert torch.allclose(val2, torch.gather(logits, 1, idx2), rtol=1e-5, atol=1e-5)


def test_gate_topk_with_masked_out_logits(device):
    """Logits of -inf (experts masked out by a caller) and NaN: a token with fewer than top_k finite
    logits still names top_k distinct experts -- the finite ones first, then the lowest-numbered of
    the rest -- instead of -1, which the gates would feed to bincount / index_add."""
    from fastermoe_amd import fmoe_native
    ninf = float("-inf")
    logits = torch.tensor([[ninf, 2.0, ninf, ninf, 1.0, ninf],
                           [ninf, ninf, ninf, ninf, ninf, ninf],
                           [0.5, ninf, 3.0, float("nan"), ninf, -1.0]], device=device)
    idx, score, cnt, pos_buf, s2r = fmoe_native.gate_topk_route(logits, 4, 0)
    assert idx.cpu().tolist() == [[1, 4, 0, 2], [0, 1, 2, 3], [2, 0, 5, 1]]
    assert score[0, :2].cpu().tolist() == [2.0, 1.0] and torch.isinf(score[0, 2:]).all()
    ref_pos, ref_cnt = orouting.count_by_gate(idx.cpu().numpy(), 6)
    assert np.array_equal(cnt.cpu().numpy(), ref_cnt) and int(ref_cnt.sum()) == 12
    assert np.array_equal(pos_buf.cpu().numpy(), ref_pos)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,d,e,k,bias", [
    (32768, 4096, 8, 2, True),     # the Mixtral-like share's gate
    (4096, 512, 8, 2, True),       # the tiny fp32 layer's gate
    (16384, 2048, 64, 1, True),    # top-1 over 64 experts
    (16384, 1024, 16, 2, False),
    (1000, 72, 5, 4, True),        # experts not a multiple of 16, tokens not a multiple of a workgroup's share,
                                   # contraction not a multiple of a wave's step
    (33, 8, 2, 2, True),
    (100, 264, 64, 8, True),
    (0, 64, 4, 2, True),
])
def test_gate_linear_topk_route(dtype, n, d, e, k, bias, device):
    """The gate's linear layer inside the top-k kernel (fmoe_gate_linear_topk_route) against
    nn.Linear + torch.topk: the logits, formed in float64 from the same operands and rounded to the
    element type, fix the selection for every token whose k+1 largest logits are further apart than
    the rounding of the two different summation orders can move them -- those tokens must match
    torch.topk exactly; the scores must be the (rounded) logits of whatever was selected; and the
    routing must be the oracle's on the same index tensor, bit for bit."""
    from fastermoe_amd import fmoe_native
    gen = torch.Generator().manual_seed(n + d + e)
    x = torch.randn(n, d, generator=gen).to(dtype)
    w = (torch.randn(e, d, generator=gen) * (3.0 / d ** 0.5)).to(dtype)
    b = torch.randn(e, generator=gen).to(dtype) if bias else None
    xd, wd, bd = x.to(device), w.to(device), (b.to(device) if bias else None)
    ref = x.double() @ w.double().t()
    if bias:
        ref = ref + b.double()
    for mode in (0, 1):
        idx, score, cnt, pos_buf, s2r = fmoe_native.gate_linear_topk_route(xd, wd, bd, k, mode)
        assert idx.shape == (n, k) and score.dtype == dtype
        ref_pos, ref_cnt = orouting.count_by_gate(idx.cpu().numpy(), e)
        assert np.array_equal(cnt.cpu().numpy(), ref_cnt) and int(ref_cnt.sum()) == n * k
        assert np.array_equal(pos_buf.cpu().numpy(), ref_pos)
        inv = np.full(n * k, -1, dtype=np.int64)
        inv[ref_pos] = np.arange(n * k)
        assert np.array_equal(s2r.cpu().numpy(), inv)
        if n == 0:
            continue
        got_idx = idx.cpu()
        assert (got_idx.sort(dim=1).values.diff(dim=1) > 0).all() if k > 1 else True   # distinct experts
        top_val, top_idx = torch.topk(ref, min(k + 1, e), dim=1, sorted=True)
        # (float32: the two fp32 summation orders differ by about sqrt(d) roundings of the partial sums)
        step = {torch.float32: 2.0 ** -22 * max(1.0, d ** 0.5), torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}[dtype]
        # choice j of a token is settled when its logit is clear of both neighbours in the sorted order
        gaps = top_val[:, :-1] - top_val[:, 1:]                                   # [n, k] (or [n, e-1])
        ok = gaps > 4 * step * top_val.abs().max(dim=1, keepdim=True).values.clamp(min=1.0)
        below = ok if ok.shape[1] == k else torch.cat([ok, torch.ones(n, 1, dtype=torch.bool)], dim=1)
        above = torch.cat([torch.ones(n, 1, dtype=torch.bool), ok[:, :k - 1]], dim=1)
        clear = above & below[:, :k]
        assert clear.float().mean() > 0.3
        assert torch.equal(got_idx[clear], top_idx[:, :k][clear])
        picked = torch.gather(ref, 1, got_idx)
        if mode == 0:
            want = picked
        else:
            want = torch.softmax(picked, dim=1)
        tol = {torch.float32: 1e-5, torch.bfloat16: 1.6e-2, torch.float16: 2e-3}[dtype]
        assert torch.allclose(score.double().cpu(), want, rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode", [0, 1])
def test_gate_linear_topk_autograd(dtype, mode, device):
    """GateLinearTopK's backward against autograd through nn.Linear, a gather at the SAME indices
    and the softmax: gradients of the input, the weight and the bias."""
    from fastermoe_amd.functions import GateLinearTopK
    torch.manual_seed(12)
    n, d, e, k = 600, 96, 12, 4
    lin = torch.nn.Linear(d, e).to(dtype).to(device)
    x = torch.randn(n, d, device=device).to(dtype).requires_grad_(True)
    g = torch.randn(n, k, device=device).to(dtype)
    idx, score = GateLinearTopK.apply(x, lin.weight, lin.bias, k, mode)
    assert hasattr(idx, "_fmoe_route")
    (score * g).sum().backward()
    got = [x.grad.clone(), lin.weight.grad.clone(), lin.bias.grad.clone()]
    x64 = x.detach().double().requires_grad_(True)
    w64, b64 = lin.weight.detach().double().requires_grad_(True), lin.bias.detach().double().requires_grad_(True)
    val = torch.gather(x64 @ w64.t() + b64, 1, idx)
    sc = torch.softmax(val, dim=1) if mode == 1 else val
    (sc * g.double()).sum().backward()
    tol = TOL[dtype] if dtype != torch.float32 else 1e-5
    for a, r in zip(got, [x64.grad, w64.grad, b64.grad]):
        assert rel_err(a, r) <= tol


def test_naive_gate_uses_the_fused_linear_and_matches_the_unfused_one(device, monkeypatch):
    from fastermoe_amd.gates import NaiveGate
    torch.manual_seed(4)
    gate = NaiveGate(256, 16, 1, top_k=2).to(device)
    x = torch.randn(3000, 256, device=device)
    results = []
    for flag in ("1", "0"):
        monkeypatch.setenv("FMOE_GATE_LINEAR_FUSED", flag)
        gate.zero_grad()
        idx, val = gate(x)
        val.square().sum().backward()
        results.append((idx, val, gate.gate.weight.grad.clone(), gate.gate.bias.grad.clone()))
    assert torch.equal(results[0][0], results[1][0])            # random fp32 logits: no near-ties
    for a, b in zip(results[0][1:], results[1][1:]):
        assert torch.allclose(a, b, rtol=1e-4, atol=1e-4)
    # with all logits asked for, the gate runs the linear layer by itself
    idx3, val3, logits = gate(x, return_all_scores=True)
    assert logits.shape == (3000, 16) and torch.equal(idx3, results[1][0])
