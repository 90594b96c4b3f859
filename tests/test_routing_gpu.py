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
