"""Pins the CPU oracle (oracle/) before anything is compared against it.

The checks are chosen so that a plausible slip in the oracle (an off-by-one in
the placement, ascending instead of descending order, a dropped bias, a
transposed weight, a missing gate score) fails at least one of them; none of
them re-types the oracle's own formula.
"""
import json
import os

import numpy as np
import pytest
import torch

from oracle import moe as omoe
from oracle import routing as orouting

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "routing_cases.json")


def _cases():
    with open(GOLDEN) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _cases(), ids=lambda c: c["name"])
def test_routing_oracle_matches_golden(case):
    gate = np.array(case["gate"], dtype=np.int64)
    e = case["n_expert"]
    cnt = orouting.expert_count(gate, e)
    assert cnt.tolist() == case["counts"]
    cum = np.cumsum(cnt).astype(np.int32)
    pos = orouting.assign_pos(cum, gate)
    assert pos.tolist() == case["pos"]
    assert cum.tolist() == case["cum_after"]
    cap = np.full(e, case["capacity"], dtype=np.int32)
    lim = orouting.limit_by_capacity(cnt.astype(np.int64), cap, e, 1)
    assert lim.tolist() == case["limited"]
    ec = lim.astype(np.int32)
    pruned = orouting.prune_gate_by_capacity(gate, ec)
    assert pruned.tolist() == case["pruned"]
    assert ec.tolist() == case["cap_after"]


def test_hand_worked_case_is_what_a_person_gets():
    # gate = [1,0,0,1,1,2,0,1]: expert 0 <- slots 1,2,6; expert 1 <- 0,3,4,7; expert 2 <- 5.
    # Sequential atomicSub hands the LAST position of a segment to the FIRST slot.
    pos, cnt = orouting.count_by_gate(np.array([1, 0, 0, 1, 1, 2, 0, 1]), 3)
    assert cnt.tolist() == [3, 4, 1]
    assert pos.tolist() == [6, 2, 1, 7, 4, 3, 0, 5]


@pytest.mark.parametrize("n,e,seed", [(1000, 7, 0), (4096, 64, 1), (65536, 256, 2), (33, 1, 3)])
def test_routing_oracle_closed_forms(n, e, seed):
    rng = np.random.default_rng(seed)
    gate = rng.integers(-1, e, size=n).astype(np.int64)
    valid = np.flatnonzero(gate >= 0)
    cnt = orouting.expert_count(gate, e)
    # closed form: bincount
    assert np.array_equal(cnt, np.bincount(gate[valid], minlength=e))
    cum = np.cumsum(cnt).astype(np.int32)
    cum_in = cum.copy()
    pos = orouting.assign_pos(cum, gate)
    # invariants that hold for ANY schedule of the reference kernel
    assert np.array_equal(np.sort(pos), valid)               # permutation of the valid slots
    assert np.all(np.diff(gate[pos]) >= 0)                   # grouped by expert, ascending
    assert np.array_equal(cum, cum_in - cnt)                 # cum_count consumed to exclusive
    # canonical (sequential) order: inside a segment, descending slot index;
    # closed form: stable sort by expert of the REVERSED valid slots
    rev = valid[::-1]
    expect = rev[np.argsort(gate[rev], kind="stable")]
    assert np.array_equal(pos, expect)
    # accumulate semantics of expert_count
    again = orouting.expert_count(gate, e, cnt.copy())
    assert np.array_equal(again, 2 * cnt)


@pytest.mark.parametrize("n,e,cap,seed", [(500, 8, 40, 0), (8192, 16, 300, 1), (999, 3, 0, 2), (64, 70, 1, 3)])
def test_prune_oracle_closed_form(n, e, cap, seed):
    rng = np.random.default_rng(seed)
    gate = rng.integers(0, e, size=(n // 2, 2)).astype(np.int64)
    new_lec, new_gec, pruned = orouting.limit_and_prune(gate, e, cap)
    cnt = np.bincount(gate.reshape(-1), minlength=e)
    assert np.array_equal(new_gec, np.minimum(cnt, cap))     # one worker: min(count, cap)
    flat = gate.reshape(-1)
    # closed form: rank among earlier slots of the same expert
    onehot = flat[:, None] == np.arange(e)[None, :]
    rank = (np.cumsum(onehot, axis=0) - onehot)[np.arange(flat.size), flat]
    expect = np.where(rank < cap, flat, -1).reshape(gate.shape)
    assert np.array_equal(pruned, expect)
    # the reference's own test criterion (tests/test_gates.py:51-57)
    kept = np.bincount(pruned[pruned >= 0], minlength=e)
    assert np.all(kept <= cap)
    assert pruned.shape == gate.shape


def test_limit_by_capacity_three_workers_by_hand():
    # expert 0: cap 5, proposals 3,4,2 -> grants 3, 2 (what is left), 0 (left went negative)
    # expert 1: cap 10, proposals 1,2,3 -> all granted
    ec = np.array([3, 1, 4, 2, 2, 3], dtype=np.int64)  # [w,e] row-major, W=3, E=2
    cap = np.array([5, 10], dtype=np.int32)
    eca = orouting.limit_by_capacity(ec, cap, 2, 3)
    assert eca.reshape(3, 2).tolist() == [[3, 1], [2, 2], [0, 3]]
    assert cap.tolist() == [5 - 9, 10 - 6]


def test_prune_keeps_existing_drops():
    ec = np.array([1, 1], dtype=np.int32)
    out = orouting.prune_gate_by_capacity(np.array([-1, 0, 0, -1, 1]), ec)
    assert out.tolist() == [-1, 0, -1, -1, 1]
    assert ec.tolist() == [-1, 0]


# ---- MLP oracle -------------------------------------------------------------------

def _dense_formulation(x, idx, score, w1, b1, w2, b2, act, k):
    """Every expert applied to every token (einsum), then the chosen ones selected
    with a one-hot mask: shares no code path with the masked per-expert loop."""
    h = torch.einsum("nd,ehd->neh", x, w1) + b1[None]
    y = torch.einsum("neh,edh->ned", act(h), w2) + b2[None]
    idx = idx.view(-1, k)
    out = torch.zeros_like(x)
    for j in range(k):
        sel = torch.nn.functional.one_hot(idx[:, j].clamp(min=0), w1.shape[0]).to(x.dtype)
        sel = sel * (idx[:, j] >= 0).to(x.dtype)[:, None]
        out = out + score[:, j, None] * torch.einsum("ne,ned->nd", sel, y)
    return out


@pytest.mark.parametrize("k,drops", [(1, False), (2, False), (3, True)])
def test_mlp_oracle_against_dense_formulation(k, drops):
    g = torch.Generator().manual_seed(7 + k)
    n, d, h, e = 24, 6, 10, 5
    x = torch.randn(n, d, generator=g, dtype=torch.float64)
    w1 = torch.randn(e, h, d, generator=g, dtype=torch.float64)
    w2 = torch.randn(e, d, h, generator=g, dtype=torch.float64)
    b1 = torch.randn(e, h, generator=g, dtype=torch.float64)
    b2 = torch.randn(e, d, generator=g, dtype=torch.float64)
    score = torch.randn(n, k, generator=g, dtype=torch.float64)
    idx = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(n)])
    if drops:
        idx[torch.rand(n, k, generator=g) < 0.3] = -1
    got = omoe.brute_force_moe_mlp(x, idx, score, w1, b1, w2, b2, "gelu", k)
    ref = _dense_formulation(x, idx, score, w1, b1, w2, b2, torch.nn.functional.gelu, k)
    assert torch.allclose(got, ref, rtol=1e-12, atol=1e-12)


def test_mlp_oracle_single_expert_is_a_plain_mlp():
    torch.manual_seed(0)
    mlp = torch.nn.Sequential(torch.nn.Linear(5, 9), torch.nn.ReLU(), torch.nn.Linear(9, 5)).double()
    x = torch.randn(11, 5, dtype=torch.float64)
    idx = torch.zeros(11, 1, dtype=torch.int64)
    score = torch.full((11, 1), 0.5, dtype=torch.float64)
    got = omoe.brute_force_moe_mlp(x, idx, score, mlp[0].weight[None], mlp[0].bias[None],
                                   mlp[2].weight[None], mlp[2].bias[None], "relu", 1)
    assert torch.allclose(got, 0.5 * mlp(x), rtol=1e-12, atol=1e-12)


def test_mlp_oracle_hand_worked():
    # two tokens, two experts, d=1, h=1, ReLU, top-2 with scores (2, 3):
    # expert e: y = w2*relu(w1*x + b1) + b2 with (w1,b1,w2,b2) = (1,0,2,1) and (-1,1,1,0)
    x = torch.tensor([[1.0], [-2.0]], dtype=torch.float64)
    w1 = torch.tensor([[[1.0]], [[-1.0]]], dtype=torch.float64)
    b1 = torch.tensor([[0.0], [1.0]], dtype=torch.float64)
    w2 = torch.tensor([[[2.0]], [[1.0]]], dtype=torch.float64)
    b2 = torch.tensor([[1.0], [0.0]], dtype=torch.float64)
    idx = torch.tensor([[0, 1], [1, 0]])
    score = torch.tensor([[2.0, 3.0], [2.0, 3.0]], dtype=torch.float64)
    out = omoe.brute_force_moe_mlp(x, idx, score, w1, b1, w2, b2, "relu", 2)
    # token 0: e0 -> 2*1+1 = 3, e1 -> relu(-1+1)=0 -> 0 ; 2*3 + 3*0 = 6
    # token 1: e1 -> relu(2+1)=3 -> 3, e0 -> relu(-2)=0 -> 1 ; 2*3 + 3*1 = 9
    assert out.view(-1).tolist() == [6.0, 9.0]


def test_mlp_oracle_gradients_against_finite_differences():
    g = torch.Generator().manual_seed(3)
    n, d, h, e, k = 6, 3, 4, 3, 2
    x = torch.randn(n, d, generator=g, dtype=torch.float64)
    w1 = torch.randn(e, h, d, generator=g, dtype=torch.float64)
    w2 = torch.randn(e, d, h, generator=g, dtype=torch.float64)
    b1 = torch.randn(e, h, generator=g, dtype=torch.float64)
    b2 = torch.randn(e, d, generator=g, dtype=torch.float64)
    score = torch.rand(n, k, generator=g, dtype=torch.float64)
    idx = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(n)])
    res = omoe.moe_mlp_forward_backward(x, idx, score, w1, b1, w2, b2, "gelu", k)
    f = lambda W1: omoe.brute_force_moe_mlp(x, idx, score, W1, b1, w2, b2, "gelu", k).mean()
    eps = 1e-6
    for pos in [(0, 0, 0), (2, 3, 1), (1, 2, 2)]:
        wp, wm = w1.clone(), w1.clone()
        wp[pos] += eps
        wm[pos] -= eps
        fd = (f(wp) - f(wm)) / (2 * eps)
        assert abs(fd.item() - res["grad_w1"][pos].item()) < 1e-7


def test_per_expert_linear_matches_masked_loop():
    g = torch.Generator().manual_seed(5)
    counts = torch.tensor([3, 0, 5, 1])
    x = torch.randn(9, 4, generator=g, dtype=torch.float64)
    w = torch.randn(4, 6, 4, generator=g, dtype=torch.float64)
    b = torch.randn(4, 6, generator=g, dtype=torch.float64)
    y = omoe.per_expert_linear(x, counts, w, b)
    owner = torch.repeat_interleave(torch.arange(4), counts)
    for r in range(9):
        assert torch.allclose(y[r], w[owner[r]] @ x[r] + b[owner[r]], rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("act", ["gelu", "relu"])
@pytest.mark.parametrize("bias", [True, False])
def test_per_expert_backward_matches_autograd(act, bias):
    """The written-out backward (one expert at a time) against autograd on the masked-loop
    forward: drops, an expert without tokens, top-3."""
    g = torch.Generator().manual_seed(17)
    n, d, h, e, k = 37, 12, 20, 5, 3
    x = torch.randn(n, d, generator=g)
    idx = torch.randint(-1, e - 1, (n, k), generator=g)     # expert e-1 gets nothing, some slots dropped
    score = torch.rand(n, k, generator=g)
    w1, w2 = torch.randn(e, h, d, generator=g), torch.randn(e, d, h, generator=g)
    b1 = torch.randn(e, h, generator=g) if bias else None
    b2 = torch.randn(e, d, generator=g) if bias else None
    ref = omoe.moe_mlp_forward_backward(x, idx, score, w1, b1, w2, b2, act, k)
    got = omoe.moe_mlp_forward_backward_per_expert(x, idx, score, w1, b1, w2, b2, act, k)
    for name in ref:
        if ref[name] is None:
            assert got[name] is None
        else:
            assert torch.allclose(got[name], ref[name], rtol=1e-11, atol=1e-13), name
    # an explicit output gradient instead of the mean
    go = torch.randn(n, d, generator=g)
    got = omoe.moe_mlp_forward_backward_per_expert(x, idx, score, w1, b1, w2, b2, act, k, grad_out=go)
    xx = x.double().requires_grad_(True)
    W1 = w1.double().requires_grad_(True)
    out = omoe.brute_force_moe_mlp(xx, idx, score.double(), W1, None if b1 is None else b1.double(), w2.double(),
                                   None if b2 is None else b2.double(), act, k)
    out.backward(go.double())
    assert torch.allclose(got["grad_inp"], xx.grad, rtol=1e-11, atol=1e-13)
    assert torch.allclose(got["grad_w1"], W1.grad, rtol=1e-11, atol=1e-13)


@pytest.mark.parametrize("counts,cap", [([3, 0, 700, 256, 1, 0], 960), ([0, 0, 0], 10), ([5000], 5000),
                                        ([300, 300, 300], 700), ([-4, 10, 2 ** 40, 7], 100)])
def test_segment_table_oracle_closed_forms(counts, cap):
    """Pins oracle.routing.segment_table by what the arithmetic fixes: the segments are the clipped
    running sums of the (clamped) counts, every expert has ceil(rows / block) tiles, the tiles of an
    expert tile its segment exactly and in order, and only an expert's last tile may be short."""
    t = orouting.segment_table(np.array(counts, dtype=np.int64), cap)
    clamped = np.clip(np.array(counts, dtype=object), 0, None)
    run = np.minimum(np.concatenate([[0], np.cumsum(clamped)]), cap).astype(np.int64)
    assert t["seg"].tolist() == run.tolist()
    rows = np.diff(run)
    for block, key in ((256, "tiles256"), (128, "tiles128")):
        tiles = t[key]
        assert np.array_equal(np.bincount(tiles[:, 0], minlength=len(counts)) if len(tiles) else np.zeros(len(counts), int),
                              -(-rows // block))
        assert np.all(np.diff(tiles[:, 0]) >= 0)
        covered = np.zeros(max(int(run[-1]), 1), dtype=int)
        for e, first, n in tiles.tolist():
            assert run[e] <= first and first + n <= run[e + 1] and 1 <= n <= block
            assert (first - run[e]) % block == 0
            assert n == block or first + n == run[e + 1]
            covered[first:first + n] += 1
        assert np.all(covered[:int(run[-1])] == 1)


def test_segment_table_oracle_hand_case():
    # 3 experts with 300, 0 and 130 rows: expert 0 has a whole 256-row tile and 44 rows more
    t = orouting.segment_table([300, 0, 130], 1000)
    assert t["seg"].tolist() == [0, 300, 300, 430]
    assert t["tiles256"].tolist() == [[0, 0, 256], [0, 256, 44], [2, 300, 130]]
    assert t["tiles128"].tolist() == [[0, 0, 128], [0, 128, 128], [0, 256, 44], [2, 300, 128], [2, 428, 2]]
