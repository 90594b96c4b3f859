"""GPU parity of the MoE modules against the brute-force oracle: the cases of the
reference's tests/test_numerical.py (test_fmoe_linear, test_fmoe), tests/test_fused.py,
tests/test_gates.py and tests/test_zero.py, plus the five benchmark configurations at
reduced token counts."""
import math

import numpy as np
import pytest
import torch
import torch.nn as nn

import fastermoe_amd as fmoe
from fastermoe_amd.gates import GShardGate, NaiveGate, SwitchGate, ZeroGate, NoisyGate
from fastermoe_amd.layers import FMoE
from fastermoe_amd.transformer import _Expert
from oracle import moe as omoe
from oracle import routing as orouting
from helpers import TOL, assert_close, close_stats, rel_err, zipf_experts

pytestmark = pytest.mark.gpu


def _oracle(moe, x, idx, score, act, top_k):
    e = moe.experts
    return omoe.moe_mlp_forward_backward(
        x, idx, score, e.htoh4.weight, e.htoh4.bias, e.h4toh.weight, e.h4toh.bias, act, top_k)


def _compare(moe, x, act, top_k, dtype, grads_of_score=False):
    x = x.clone().requires_grad_(True)
    with torch.no_grad():
        idx, score = moe.gate(x)
    # fix the routing so that the layer and the oracle see the same gate output
    moe.gate.forward = lambda inp: (idx, score)
    moe.zero_grad()
    out = moe(x)
    out.mean().backward()
    ref = _oracle(moe, x, idx, score, act, top_k)
    tol = TOL[dtype]
    e = moe.experts
    got = {"out": out, "grad_inp": x.grad, "grad_w1": e.htoh4.weight.grad, "grad_w2": e.h4toh.weight.grad,
           "grad_b1": e.htoh4.bias.grad if e.htoh4.bias is not None else None,
           "grad_b2": e.h4toh.bias.grad if e.h4toh.bias is not None else None}
    for name, val in got.items():
        if val is None:
            assert ref[name] is None
            continue
        assert rel_err(val, ref[name]) <= tol, (name, rel_err(val, ref[name]))
        if dtype == torch.float32:
            # float32 is held to the element-by-element and root-mean-square bounds as well
            assert_close(val, ref[name], tol, name)
    return got


def _compare_per_expert(moe, x, idx, score, act, top_k, tol):
    """Layer against the one-expert-at-a-time float64 oracle (for layers whose float64 autograd graph
    would not fit in memory): max|d| <= tol max|ref|, |d| <= tol |ref| + 3 tol rms(ref) element by
    element, and rms(d) <= tol / 2 rms(ref); the weight gradients expert by expert, against the
    expert's own root mean square.  The floor of three: a weight gradient is a sum over the expert's
    rows of products that went through four roundings to the element type on the way (pre-activation,
    activation, both gradient buffers); over the 10^7 elements of such a tensor the tail of that
    rounding noise reaches a few percent of the root mean square.  A wrong or missing term shows in the
    rms bound, where the noise averages out."""
    floor = 3.0
    x = x.clone().requires_grad_(True)
    moe.gate.forward = lambda inp: (idx, score)
    moe.zero_grad()
    out = moe(x)
    out.mean().backward()
    e = moe.experts
    ref = omoe.moe_mlp_forward_backward_per_expert(x, idx, score, e.htoh4.weight, e.htoh4.bias, e.h4toh.weight,
                                                   e.h4toh.bias, act, top_k, grad_dtype=torch.float32)
    assert_close(out, ref["out"], tol, "out", floor)
    assert_close(x.grad, ref["grad_inp"], tol, "grad_inp", floor)
    counts = torch.bincount(idx[idx >= 0].view(-1).cpu(), minlength=e.htoh4.weight.shape[0])
    for name, got in (("grad_w1", e.htoh4.weight.grad), ("grad_w2", e.h4toh.weight.grad),
                      ("grad_b1", e.htoh4.bias.grad), ("grad_b2", e.h4toh.bias.grad)):
        scale = ref[name].abs().max().item()
        for ex in range(got.shape[0]):
            if counts[ex] == 0:
                assert torch.count_nonzero(got[ex]) == 0, (name, ex)
                continue
            _, elem, rms = close_stats(got[ex], ref[name][ex], floor)
            big = (got[ex].double().cpu() - ref[name][ex].double()).abs().max().item() / scale
            assert big <= tol and elem <= tol and rms <= tol / 2, (name, ex, int(counts[ex]), big, elem, rms)


class MyMoE(FMoE):
    """The reference tests' module (tests/test_numerical.py:65-81): FMoE with a fused
    _Expert whose weights are N(0,1) from numpy's default_rng(1234)."""

    def __init__(self, num_expert, d_model, d_hidden, top_k, activation, enable_fuse=False):
        super().__init__(num_expert=num_expert, d_model=d_model, gate=NaiveGate, world_size=1, top_k=top_k,
                         enable_fuse=enable_fuse)
        self.experts = _Expert(num_expert, d_model, d_hidden, activation)
        rng = np.random.default_rng(1234)
        for lin in (self.experts.htoh4, self.experts.h4toh):
            lin.weight.data = torch.from_numpy(rng.normal(0.0, 1.0, size=tuple(lin.weight.shape))).float()
            lin.bias.data.zero_()


@pytest.mark.parametrize("num_expert", [4, 8])
@pytest.mark.parametrize("top_k", [2, 3])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.float16, torch.bfloat16])
def test_fmoe_linear_reference_grid(num_expert, top_k, dtype, device):
    """tests/test_numerical.py:84-207: batch 4, d_model 16, d_hidden 32, GELU, seed 42."""
    torch.manual_seed(42)
    moe = MyMoE(num_expert, 16, 32, top_k, torch.nn.functional.gelu).to(dtype).to(device)
    x = torch.rand(4, 16).to(dtype).to(device)
    got = _compare(moe, x, "gelu", top_k, dtype)
    # the reference's own criterion: max abs error 1e-3 (5e-1 for half)
    ref = _oracle(moe, x, *moe.gate(x), "gelu", top_k)
    bound = 5e-1 if dtype in (torch.float16, torch.bfloat16) else 1e-3
    assert (got["out"].double().cpu() - ref["out"]).abs().max() <= bound


@pytest.mark.parametrize("fuse", [False, True])
@pytest.mark.parametrize("dtype,n,d,h,e,k,act", [
    (torch.float32, 512, 512, 1024, 8, 2, "gelu"),      # config 1 shape
    (torch.float32, 4096, 512, 1024, 8, 2, "gelu"),     # config 1 at its full size (the oracle runs it whole)
    (torch.bfloat16, 512, 1024, 4096, 16, 2, "gelu"),   # config 2 shape
    (torch.bfloat16, 768, 1024, 2048, 64, 1, "gelu"),   # config 3 routing (64 experts, Zipf top-1), half width
    (torch.bfloat16, 384, 4096, 3584, 8, 2, "gelu"),    # config 4 shape (quarter hidden)
    (torch.bfloat16, 256, 512, 256, 256, 8, "gelu"),    # config 5 routing (256 experts, top-8), quarter width
    (torch.float32, 200, 24, 40, 3, 2, "relu"),
])
def test_transformer_mlp_configs(fuse, dtype, n, d, h, e, k, act, device):
    torch.manual_seed(42 + e)
    activation = nn.GELU() if act == "gelu" else nn.ReLU()
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=activation)
    moe.enable_fuse = fuse
    # biases away from zero so that they matter
    with torch.no_grad():
        moe.experts.htoh4.bias.normal_(0, 0.02)
        moe.experts.h4toh.bias.normal_(0, 0.02)
    moe = moe.to(dtype).to(device)
    x = torch.randn(n, d).to(dtype).to(device)
    if e == 64:  # Zipf-skewed top-1 routing with empty experts and unit scores
        p = torch.arange(1, e + 1, dtype=torch.float64) ** -1.2
        idx = torch.multinomial(p / p.sum(), n, replacement=True).view(n, 1).to(device)
        moe.gate.forward = lambda inp: (idx, torch.ones(n, 1, dtype=dtype, device=device))
    _compare(moe, x, act, k, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
@pytest.mark.parametrize("act", ["gelu", "relu", "none", "tanh"])
def test_expert_epilogue_node_matches_the_three_modules(dtype, act, device, monkeypatch):
    """_Expert runs Linear -> activation -> Linear as one autograd node with the activation in the
    GEMM epilogues when the activation is the exact GELU, ReLU or none; FMOE_EXPERT_EPILOGUE=0 (and
    any other activation, here tanh) runs the reference's three modules (fmoe/transformer.py:22-30).
    Both against each other and, for GELU / ReLU, against the float64 oracle."""
    torch.manual_seed(31)
    n, d, h, e, k = 333, 96, 160, 5, 2
    module = {"gelu": nn.GELU(), "relu": nn.ReLU(), "none": nn.Identity(), "tanh": nn.Tanh()}[act]
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=module)
    with torch.no_grad():
        moe.experts.htoh4.weight.mul_((d * h) ** 0.5 * d ** -0.5)
        moe.experts.h4toh.weight.mul_((d * h) ** 0.5 * h ** -0.5)
        moe.experts.htoh4.bias.normal_(0, 0.3)
        moe.experts.h4toh.bias.normal_(0, 0.3)
    moe = moe.to(dtype).to(device)
    assert (moe.experts._epilogue_activation() is None) == (act == "tanh")
    x = torch.randn(n, d).to(dtype).to(device)
    idx = torch.randint(-1, e - 1, (n, k), device=device)     # drops, and expert e-1 without rows
    score = torch.rand(n, k, device=device).to(dtype)
    moe.gate.forward = lambda inp: (idx, score)
    results = []
    for flag in ("1", "0"):
        monkeypatch.setenv("FMOE_EXPERT_EPILOGUE", flag)
        moe.zero_grad()
        xi = x.clone().requires_grad_(True)
        out = moe(xi)
        out.float().mean().backward()
        results.append([out, xi.grad] + [p.grad.clone() for p in moe.experts.parameters()])
    tol = TOL[dtype]
    for a, b in zip(*results):
        assert rel_err(a, b) <= (2 * tol if dtype == torch.bfloat16 else 10 * tol)
    if act in ("gelu", "relu"):
        monkeypatch.setenv("FMOE_EXPERT_EPILOGUE", "1")
        _compare(moe, x, act, k, dtype)


@pytest.mark.parametrize("fuse", [False, True])
@pytest.mark.parametrize("n,d,h,e,k,routing", [
    (1024, 2048, 8192, 64, 1, "zipf"),     # the skewed Switch-style layer at full width: Zipf(1.2) top-1, empty experts
    (512, 2048, 1024, 256, 8, "biased"),   # the fine-grained layer at full width: 256 experts, top-8
])
def test_full_width_bf16_layers(fuse, n, d, h, e, k, routing, device):
    """The many-expert configurations at their real feature sizes (only the token count is reduced),
    bf16, forward and all gradients against the float64 oracle, normwise and element by element."""
    torch.manual_seed(e)
    gen = torch.Generator().manual_seed(e + 1)
    with torch.device(device):  # 2 x 1 G weights: initialised on the GPU
        moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.GELU())
    moe.enable_fuse = fuse
    with torch.no_grad():
        moe.experts.htoh4.weight.mul_((d * h) ** 0.5 * d ** -0.5)   # unit-variance activations instead of ~1e-3
        moe.experts.h4toh.weight.mul_((d * h) ** 0.5 * h ** -0.5)
        moe.experts.htoh4.bias.normal_(0, 0.1)
        moe.experts.h4toh.bias.normal_(0, 0.1)
    moe = moe.to(torch.bfloat16).to(device)
    x = torch.randn(n, d, generator=gen).bfloat16().to(device)
    if routing == "zipf":
        idx = zipf_experts(n, e, 1.2, gen).view(n, 1).to(device)
        score = torch.ones(n, 1, dtype=torch.bfloat16, device=device)
        assert int(torch.bincount(idx.view(-1).cpu(), minlength=e).max()) > n // 10
        assert int((torch.bincount(idx.view(-1).cpu(), minlength=e) == 0).sum()) > 0
    else:
        logits = torch.randn(n, e, generator=gen) + 0.5 * torch.randn(e, generator=gen)
        val, idx = torch.topk(logits, k, dim=-1)
        idx, score = idx.to(device), torch.softmax(val, dim=-1).bfloat16().to(device)
    _compare_per_expert(moe, x, idx, score, "gelu", k, 2e-2)


@pytest.mark.parametrize("fuse", [False, True])
def test_gshard_shaped_bf16_layer_with_capacity_drops(fuse, device):
    """The GShard-style top-2 layer (d 1024, h 4096, 16 experts, bf16) with a per-expert capacity of
    ceil(1.2 N k / E) applied by the capacity kernels, so that overflow slots are dropped: the gate
    output after limit_by_capacity goes to the layer and to the float64 oracle alike."""
    from fastermoe_amd.gates.utils import limit_by_capacity
    torch.manual_seed(2)
    n, d, h, e, k = 2048, 1024, 4096, 16, 2
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.GELU())
    moe.enable_fuse = fuse
    with torch.no_grad():
        moe.experts.htoh4.weight.mul_((d * h) ** 0.5 * d ** -0.5)
        moe.experts.h4toh.weight.mul_((d * h) ** 0.5 * h ** -0.5)
        moe.experts.htoh4.bias.normal_(0, 0.1)
        moe.experts.h4toh.bias.normal_(0, 0.1)
    moe = moe.to(torch.bfloat16).to(device)
    x = torch.randn(n, d).bfloat16().to(device)
    logits = torch.randn(n, e) + torch.linspace(-0.6, 0.6, e)      # mild imbalance: some experts overflow
    val, top = torch.topk(logits, k, dim=-1)
    cap = math.ceil(1.2 * n * k / e)
    _, _, idx = limit_by_capacity(top.to(device), e, 1, cap)
    dropped = int((idx < 0).sum())
    assert 0 < dropped < n * k // 2
    assert int(torch.bincount(idx[idx >= 0].view(-1), minlength=e).max()) == cap
    _, _, want = orouting.limit_and_prune(top.numpy(), e, cap)
    assert np.array_equal(idx.cpu().numpy(), want)
    score = torch.softmax(val, dim=-1).bfloat16().to(device)
    _compare_per_expert(moe, x, idx, score, "gelu", k, 2e-2)


def test_fused_bf16_expert_split_across_chunks(device, monkeypatch):
    """Four chunks over three experts: the chunk bounds (read back from the planner) cut at least one
    expert's rows, so its forward and data-grad rows come from two launches; output and all gradients
    against the float64 oracle.  The weight gradients are produced by one launch over all rows."""
    import ctypes
    from fastermoe_amd import _lib
    monkeypatch.setenv("FMOE_FUSE_GRAN", "4")
    torch.manual_seed(9)
    n, d, h, e, k = 1500, 512, 1024, 3, 2
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.GELU())
    moe.enable_fuse = True
    with torch.no_grad():
        moe.experts.htoh4.weight.mul_((d * h) ** 0.5 * d ** -0.5)
        moe.experts.h4toh.weight.mul_((d * h) ** 0.5 * h ** -0.5)
        moe.experts.htoh4.bias.normal_(0, 0.1)
    moe = moe.to(torch.bfloat16).to(device)
    x = torch.randn(n, d).bfloat16().to(device)
    idx = torch.randint(0, e, (n, k), device=device)
    score = torch.rand(n, k, device=device).bfloat16()
    counts = torch.bincount(idx.view(-1).cpu(), minlength=e)
    c = (ctypes.c_int64 * e)(*counts.tolist())
    b = (ctypes.c_int64 * 5)()
    _lib.check(_lib.load().fmoe_fused_chunk_bounds(ctypes.cast(c, ctypes.c_void_p), e, 4, d, h, 0,
                                                   ctypes.cast(b, ctypes.c_void_p)))
    edges = set(torch.cumsum(counts, 0).tolist()) | {0}
    assert any(x not in edges for x in list(b)[1:4]), "no chunk bound cuts an expert"
    _compare_per_expert(moe, x, idx, score, "gelu", k, 2e-2)


@pytest.mark.parametrize("fuse", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_folded_combine_equals_gather_then_combine(fuse, dtype, device, monkeypatch):
    """The layer folds MOEGather and the bmm with the gate scores into one pass; with
    FMOE_FOLD_COMBINE=0 it runs them apart as fmoe/layers.py:139-149,321-322 does.  Output, input
    gradient, expert and gate gradients agree (dropped slots, an expert without tokens)."""
    torch.manual_seed(5)
    n, d, h, e, k = 257, 128, 192, 5, 2
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.GELU())
    moe.enable_fuse = fuse
    moe = moe.to(dtype).to(device)
    x = torch.randn(n, d).to(dtype).to(device)
    idx = torch.randint(0, e - 1, (n, k), device=device)
    idx[torch.rand(n, k, device=device) < 0.2] = -1
    gate_linear = moe.gate.gate

    def gate_forward(inp):  # scores that depend on the input, so that their gradient is exercised
        return idx, torch.softmax(gate_linear(inp)[:, :k].float(), dim=-1).to(dtype)

    moe.gate.forward = gate_forward
    results = []
    for fold in ("0", "1"):
        monkeypatch.setenv("FMOE_FOLD_COMBINE", fold)
        moe.zero_grad()
        xi = x.clone().requires_grad_(True)
        out = moe(xi)
        out.float().mean().backward()
        results.append([out, xi.grad, gate_linear.weight.grad.clone()] + [p.grad.clone() for p in moe.experts.parameters()])
    tol = TOL[dtype]
    for a, b in zip(*results):
        assert rel_err(a, b) <= tol


@pytest.mark.parametrize("dtype,n,d,h,e,k", [
    # 512+ tiles in the second data-grad: 256-row tiles, ragged row and column tails (bfloat16 only: the
    # mean() loss of a batch this large puts float16 gradients into the subnormal range)
    (torch.bfloat16, 4100, 256, 4104, 2, 2),
    (torch.bfloat16, 300, 128, 520, 3, 2),     # contraction of exactly two slabs, 128-row tiles
    (torch.float16, 300, 128, 520, 3, 2),
    (torch.bfloat16, 300, 64, 264, 3, 2),      # one slab: no tail slabs to carry the pre-activation tile
    (torch.float16, 300, 64, 264, 3, 2),
    (torch.bfloat16, 700, 200, 776, 2, 1),     # three slabs and a ragged contraction tail
    (torch.float16, 700, 200, 776, 2, 1),
])
def test_fused_backward_tail_slabs(dtype, n, d, h, e, k, device, monkeypatch):
    """The second data-grad of the fused 16-bit path loads its pre-activation tile in the
    load slots of the last two contraction slabs: shapes with one, two, three and many
    slabs, both tile heights, ragged tails, against the float64 oracle."""
    monkeypatch.setenv("FMOE_FUSE_GRAN", "1")
    torch.manual_seed(n + d)
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.GELU())
    moe.enable_fuse = True
    with torch.no_grad():
        moe.experts.htoh4.weight.normal_(0, d ** -0.5)
        moe.experts.h4toh.weight.normal_(0, h ** -0.5)
        moe.experts.htoh4.bias.normal_(0, 0.5)
        moe.experts.h4toh.bias.normal_(0, 0.1)
    moe = moe.to(dtype).to(device)
    x = torch.randn(n, d).to(dtype).to(device)
    _compare(moe, x, "gelu", k, dtype)


@pytest.mark.parametrize("chunks", ["1", "3", "7"])
def test_fused_equals_unfused(chunks, device, monkeypatch):
    """tests/test_fused.py:9-34 (forward, input grad, both weight grads within 1e-3),
    for several chunk counts, with dropped slots and an expert left without tokens."""
    monkeypatch.setenv("FMOE_FUSE_GRAN", chunks)
    torch.manual_seed(0)
    n, d, h, e, k = 300, 64, 96, 6, 2
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.GELU()).to(device)
    with torch.no_grad():
        moe.experts.htoh4.bias.normal_()
        moe.experts.h4toh.bias.normal_()
    x = torch.randn(n, d, device=device)
    idx = torch.randint(0, e - 1, (n, k), device=device)      # expert e-1 gets nothing
    idx[torch.rand(n, k, device=device) < 0.2] = -1
    score = torch.rand(n, k, device=device)
    moe.gate.forward = lambda inp: (idx, score)
    results = []
    for fuse in (False, True):
        moe.enable_fuse = fuse
        moe.zero_grad()
        xi = x.clone().requires_grad_(True)
        out = moe(xi)
        out.mean().backward()
        results.append([out, xi.grad] + [p.grad.clone() for p in moe.experts.parameters()])
    for a, b in zip(*results):
        assert (a - b).abs().max() <= 1e-3
        assert rel_err(a, b) <= 1e-5
    assert torch.count_nonzero(moe.experts.htoh4.weight.grad[e - 1]) == 0


def test_reference_fused_entry_points(device):
    """fmoe_native.fused_forward / fused_backward with the reference's argument lists
    (fmoe/fused_functions.py:25-29,49-55): ReLU, no bias, one expert, d=4, h=8, 6 rows
    (tests/test_fused.py:41-46)."""
    from fastermoe_amd import fmoe_native
    torch.manual_seed(1)
    w1 = torch.randn(1, 8, 4, device=device, requires_grad=True)
    w2 = torch.randn(1, 4, 8, device=device, requires_grad=True)
    x = torch.randn(6, 4, device=device)
    cnt = torch.tensor([6])
    stored = torch.zeros(1, dtype=torch.bool)
    out, gib, gmb, gob = fmoe_native.fused_forward(x, [[(w1, w2)]], cnt, cnt, stored, 6, 1, False)
    ref = torch.relu(x @ w1[0].t()) @ w2[0].t()
    assert torch.allclose(out, ref, rtol=1e-5, atol=1e-6)
    assert torch.equal(gib, x) and torch.allclose(gmb, torch.relu(x @ w1[0].t()), rtol=1e-5, atol=1e-6)
    go = torch.randn(6, 4, device=device)
    (grad_in,) = fmoe_native.fused_backward(gib, [[(w1, w2)]], gmb, gob, go, cnt, cnt, x, stored, 6, 6, 1, False)
    xr = x.clone().requires_grad_(True)
    w1r, w2r = w1.detach().clone().requires_grad_(True), w2.detach().clone().requires_grad_(True)
    (torch.relu(xr @ w1r[0].t()) @ w2r[0].t()).backward(go)
    assert torch.allclose(grad_in, xr.grad, rtol=1e-5, atol=1e-6)
    assert torch.allclose(w1.grad, w1r.grad, rtol=1e-5, atol=1e-6)
    assert torch.allclose(w2.grad, w2r.grad, rtol=1e-5, atol=1e-6)


class _LinearExpert(nn.Module):
    def __init__(self, d_model):
        super().__init__()
        self.model = nn.Sequential(nn.Linear(d_model, d_model * 2), nn.ReLU(), nn.Linear(d_model * 2, d_model))

    def forward(self, x):
        return self.model(x)


@pytest.mark.parametrize("as_list", [False, True])
def test_fmoe_generic_experts(as_list, device):
    """tests/test_numerical.py:210-308,387-485: FMoE(expert=cls or list) against calling the
    expert module of each slot one row at a time (tests/moe.py:52-75)."""
    torch.manual_seed(42)
    n, d, e, k = 12, 16, 4, 2
    moe = FMoE(num_expert=e, d_model=d, top_k=k, gate=NaiveGate,
               expert=[_LinearExpert] * e if as_list else _LinearExpert).to(device)
    x = torch.rand(n, d, device=device, requires_grad=True)
    idx, score = moe.gate(x)
    out = moe(x)
    out.mean().backward()
    got = [x.grad.clone()] + [p.grad.clone() for p in moe.experts.parameters()]
    x.grad = None
    moe.zero_grad()
    rows = x.repeat_interleave(k, dim=0)
    per_slot = torch.stack([moe.experts[int(g)](rows[i]) for i, g in enumerate(idx.view(-1))])
    ref = torch.bmm(score.detach().view(n, 1, k), per_slot.view(n, k, d)).reshape(n, d)
    assert torch.allclose(out, ref, rtol=1e-4, atol=1e-5)
    # gradients through the experts (the gate's own path is cut on both sides: idx and score are data here)
    ref.mean().backward()
    want = [x.grad] + [p.grad for p in moe.experts.parameters()]
    gate_part = torch.autograd.grad(moe(x).mean(), moe.gate.gate.weight, allow_unused=True)[0]
    assert gate_part is not None                      # the layer does feed the gate's linear
    for g, w in zip(got[1:], want[1:]):
        assert torch.allclose(g, w, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("cap", [0.1, 1.1])
@pytest.mark.parametrize("n,e", [(4096, 4), (1000, 16)])
def test_gshard_gate(cap, n, e, device):
    """tests/test_gates.py:25-64."""
    torch.manual_seed(3)
    gate = GShardGate(64, e, 1, capacity=(cap, cap)).to(device)
    x = torch.rand(n, 64, device=device)
    idx, val = gate(x)
    assert idx.shape == (n, 2) and val.shape == (n, 2)
    limit = math.ceil(cap * n)
    counts = torch.bincount(idx[idx >= 0].view(-1), minlength=e)
    assert int(counts.max()) <= limit
    logits = gate.gate(x).detach()
    kept = idx >= 0
    assert torch.equal(torch.gather(logits, 1, idx.clamp(min=0))[kept], val[kept])
    # the balance loss of fmoe/gates/gshard_gate.py:23-34 in closed form: both choices of every token counted
    top_val, top_idx = torch.topk(logits, 2, dim=-1, sorted=True)   # the gate lists a token's choices by logit
    c_e = torch.bincount(top_idx.reshape(-1), minlength=e).double() / n
    m_e = torch.softmax(logits.double(), dim=1).mean(0)
    want_loss = float((c_e * m_e).sum() / e * e * e)
    assert abs(float(gate.get_loss().detach()) - want_loss) <= 1e-5 * want_loss
    assert abs(float(c_e.sum()) - 2.0) < 1e-9
    # first-come-first-kept: what survives the capacity step is the oracle's pruning
    _, _, pruned = orouting.limit_and_prune(top_idx.cpu().numpy(), e, limit)
    survivors = torch.from_numpy(pruned).to(device)
    assert bool(((idx == survivors) | (idx == -1)).all())
    assert torch.equal(idx[:, 0], survivors[:, 0])      # random routing only touches column 1


@pytest.mark.parametrize("cap", [0.1, 0.8])
def test_switch_gate(cap, device):
    """tests/test_gates.py:67-115."""
    torch.manual_seed(4)
    n, e = 2048, 8
    gate = SwitchGate(32, e, 1, capacity=(cap, cap)).to(device)
    gate.eval()
    x = torch.rand(n, 32, device=device)
    idx, score = gate(x)
    assert idx.shape == (n, 1)
    counts = torch.bincount(idx[idx >= 0].view(-1), minlength=e)
    assert int(counts.max()) <= math.ceil(cap * n)
    prob = torch.softmax(gate.gate(x).float(), dim=-1)
    kept = (idx >= 0).view(-1)
    assert torch.allclose(torch.gather(prob, 1, idx.clamp(min=0)).view(-1)[kept], score.view(-1)[kept])
    assert torch.isfinite(gate.get_loss())


def test_capacity_gate_in_layer(device):
    """A GShard-gated layer end to end: dropped slots contribute zero rows."""
    torch.manual_seed(5)
    n, d, h, e = 512, 64, 128, 4
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=2,
                                  gate=lambda *a: GShardGate(*a, capacity=(0.3, 0.3))).to(device)
    x = torch.randn(n, d, device=device)
    _compare(moe, x, "gelu", 2, torch.float32)


def test_zero_and_noisy_gate_and_mask(device):
    """tests/test_zero.py (runs without crashing, everything to expert 0) and the mask path."""
    torch.manual_seed(6)
    moe = fmoe.FMoETransformerMLP(num_expert=2, d_model=16, d_hidden=32, top_k=1, gate=ZeroGate).to(device)
    x = torch.rand(10, 16, device=device)
    y = moe(x)
    e = moe.experts
    ref = nn.functional.gelu(x @ e.htoh4.weight[0].t() + e.htoh4.bias[0]) @ e.h4toh.weight[0].t() + e.h4toh.bias[0]
    assert torch.allclose(y, ref, rtol=1e-5, atol=1e-6)
    # NoisyGate hands back flattened indices and [N,1,k] scores (fmoe/gates/noisy_gate.py:139-142)
    noisy = NoisyGate(16, 4, 1, top_k=2).to(device)
    nidx, nscore = noisy(torch.rand(10, 16, device=device))
    assert nidx.shape == (20,) and nscore.shape == (10, 1, 2)
    assert torch.allclose(nscore.sum(-1), torch.ones(10, 1, device=device)) and torch.isfinite(noisy.get_loss())
    mask = torch.tensor([0, 1, 0, 0, 1, 0, 0, 0, 0, 0], device=device)
    fill = torch.full((1, 16), 7.0, device=device)
    masked = fmoe.FMoETransformerMLP(num_expert=2, d_model=16, d_hidden=32, top_k=1, mask=mask,
                                     mask_dict={1: fill}).to(device)
    ym = masked(x)
    score = masked.gate(x)[1]
    assert torch.allclose(ym[mask == 1], 7.0 * score[mask == 1].expand(-1, 16))


@pytest.mark.parametrize("fuse", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_masked_tokens_index_kernels_match_boolean_indexing(fuse, dtype, device, monkeypatch):
    """mask / mask_dict (fmoe/layers.py:288-319): the index-kernel path (select kept tokens, experts,
    folded combine, one restore pass) against the reference's boolean-index formulation
    (FMOE_MASK_KERNELS=0): output, input gradient, expert gradients and the gate's gradient, which
    also flows through the masked tokens' scores.  Mask values: 0 keep, 1 and 2 replaced by their
    mask_dict rows, 5 without an entry (zero rows); a CPU mask as in tests/test_zero.py."""
    torch.manual_seed(21)
    n, d, h, e, k = 301, 64, 96, 4, 2
    mask = torch.zeros(n, dtype=torch.long)
    mask[torch.randperm(n)[:120]] = torch.tensor([1, 2, 5]).repeat(40)
    fills = {1: torch.randn(d).to(dtype).to(device), 2: torch.randn(1, d).to(dtype).to(device)}
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, mask=mask, mask_dict=fills)
    moe.enable_fuse = fuse
    moe = moe.to(dtype).to(device)
    x = torch.randn(n, d).to(dtype).to(device)
    results = []
    for flag in ("1", "0"):
        monkeypatch.setenv("FMOE_MASK_KERNELS", flag)
        moe.zero_grad()
        xi = x.clone().requires_grad_(True)
        out = moe(xi)
        (out.float() * torch.linspace(-1, 1, d, device=device)).mean().backward()
        results.append([out, xi.grad, moe.gate.gate.weight.grad.clone()] + [p.grad.clone() for p in moe.experts.parameters()])
    tol = TOL[dtype] * (1 if dtype == torch.bfloat16 else 10)
    for a, b in zip(*results):
        assert rel_err(a, b) <= tol, rel_err(a, b)
    out = results[0][0]
    assert torch.count_nonzero(out[(mask == 5).to(device)]) == 0
    with torch.no_grad():
        score = moe.gate(x)[1]
    want = score.float().sum(-1, keepdim=True)[(mask == 1).to(device)] * fills[1].float()
    assert torch.allclose(out[(mask == 1).to(device)].float(), want, rtol=2e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-5)


def test_gate_hook_and_state_dict(device):
    seen = {}
    moe = fmoe.FMoETransformerMLP(num_expert=2, d_model=8, d_hidden=16, top_k=2,
                                  gate_hook=lambda i, s, _: seen.update(idx=i, score=s)).to(device)
    moe(torch.rand(5, 8, device=device))
    assert seen["idx"].shape == (5, 2)
    clone = fmoe.FMoETransformerMLP(num_expert=2, d_model=8, d_hidden=16, top_k=2).to(device)
    clone.load_state_dict(moe.state_dict())
    x = torch.rand(5, 8, device=device)
    assert torch.equal(moe(x), clone(x))


@pytest.mark.parametrize("fuse", [False, True])
def test_no_tokens(fuse, device):
    """An empty batch goes through every kernel wrapper without a launch failing and gives
    zero weight gradients."""
    moe = fmoe.FMoETransformerMLP(num_expert=4, d_model=32, d_hidden=64, top_k=2).to(device)
    moe.enable_fuse = fuse
    x = torch.zeros(0, 32, device=device, requires_grad=True)
    out = moe(x)
    assert out.shape == (0, 32)
    out.sum().backward()
    assert x.grad.shape == (0, 32)
    for p in moe.experts.parameters():
        assert p.grad is not None and torch.count_nonzero(p.grad) == 0


@pytest.mark.parametrize("chunks", ["2", "32"])
def test_fused_many_experts_few_rows(chunks, device, monkeypatch):
    """More experts than one launch's segment table holds (256) and more chunks than some
    experts have rows: fused and unfused still agree, experts without rows get zero grads."""
    monkeypatch.setenv("FMOE_FUSE_GRAN", chunks)
    torch.manual_seed(11)
    n, d, h, e, k = 200, 32, 48, 300, 2
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.ReLU()).to(device)
    x = torch.randn(n, d, device=device)
    idx = torch.randint(0, e, (n, k), device=device)
    score = torch.rand(n, k, device=device)
    moe.gate.forward = lambda inp: (idx, score)
    results = []
    for fuse in (False, True):
        moe.enable_fuse = fuse
        moe.zero_grad()
        xi = x.clone().requires_grad_(True)
        out = moe(xi)
        out.mean().backward()
        results.append([out, xi.grad] + [p.grad.clone() for p in moe.experts.parameters()])
    for a, b in zip(*results):
        assert rel_err(a, b) <= 1e-5
    used = torch.zeros(e, dtype=torch.bool, device=device)
    used[idx.view(-1)] = True
    assert torch.count_nonzero(moe.experts.htoh4.weight.grad[~used]) == 0
    ref = _oracle(moe, x, idx, score, "relu", k)
    assert rel_err(results[1][0], ref["out"]) <= 1e-5
    assert rel_err(results[1][2], ref["grad_w1"]) <= 1e-5


@pytest.mark.parametrize("erf", ["0", "1"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_fused_gelu_epilogue_accuracy(dtype, erf, device, monkeypatch):
    """The activation computed in the GEMM epilogue against torch's exact (erf) GELU of the
    saved pre-activation, over pre-activations from -9 to 9: within one rounding step of the
    element type (relative), plus 1e-4 absolute for the far negative tail where GELU -> 0;
    and the derivative used by the backward against autograd's.  Both forms of the 16-bit
    epilogues: the polynomials, and the erf formula that FMOE_GELU_ERF=1 selects."""
    from fastermoe_amd import _lib, fmoe_native
    monkeypatch.setenv("FMOE_GELU_ERF", erf)
    n, d, h = 512, 64, 256
    x = torch.randn(n, d, device=device).to(dtype)
    w1 = (torch.randn(1, h, d, device=device) * 0.4).to(dtype)      # pre-activations ~ N(0, 3.2^2)
    b1 = torch.linspace(-6, 6, h, device=device).view(1, h).to(dtype)
    w2 = torch.eye(h, device=device).view(1, h, h)[:, :d, :].contiguous().to(dtype)  # picks the first d hidden units
    pos = torch.arange(n, device=device)
    cnt = torch.tensor([n])
    out, buf_in, buf_pre, buf_mid = fmoe_native.fused_mlp_forward(x, pos, pos.clone(), cnt, w1, b1, w2, None, 1,
                                                                  _lib.ACT_GELU, 1)
    pre = buf_pre.float()
    assert pre.min() < -6 and pre.max() > 6
    want = torch.nn.functional.gelu(pre)
    step = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -20}[dtype]
    # buf_pre is the rounded pre-activation, the kernel activates the unrounded one: allow that rounding too
    slack = step * pre.abs() * 1.13  # |GELU'| <= 1.13
    assert ((buf_mid.float() - want).abs() <= 2 * step * want.abs() + slack + 1e-4).all()
    # derivative: grad of sum(mid) w.r.t. pre through the library's backward = GELU'(pre)
    pre_leaf = pre.clone().requires_grad_(True)
    torch.nn.functional.gelu(pre_leaf).sum().backward()
    grad_inp, gw1, gb1, gw2, gb2 = fmoe_native.fused_mlp_backward(
        torch.ones(n, d, device=device, dtype=dtype), pos, pos.clone(), cnt, w1, b1, w2, None, buf_in, buf_pre,
        buf_mid, n, 1, _lib.ACT_GELU, 1, inp=x)
    # gb1[j] = sum_rows g_mid[:, j] with g_mid = (ones . W2)[:, j] * GELU'(pre[:, j]); W2 picks the first d units
    want_gb1 = (pre_leaf.grad[:, :d]).sum(0)
    got_gb1 = gb1.float().view(-1)[:d]
    assert ((got_gb1 - want_gb1).abs() <= 4 * step * want_gb1.abs() + 0.05 * step * n).all()
    assert torch.count_nonzero(gb1.float().view(-1)[d:]) == 0


def test_noisy_gate_against_the_published_definitions(device):
    """NoisyGate (Shazeer et al. 2017): evaluation mode against top-k + softmax + hard counts; training
    mode with the noise replayed from the seed, the smooth load against kth_excluding computed by
    brute force (sort the noisy logits without component i) for every (token, expert)."""
    torch.manual_seed(13)
    n, d, e, k = 40, 16, 6, 2
    gate = NoisyGate(d, e, 1, top_k=k).to(device)
    x = torch.randn(n, d, device=device)

    def cv2(v):
        return v.var() / (v.mean() ** 2 + 1e-10)

    gate.eval()
    idx, score = gate(x)
    clean = x @ gate.w_gate
    want_val, want_idx = torch.topk(clean, k, dim=1, sorted=True)
    assert torch.equal(idx.view(n, k), want_idx)
    assert torch.allclose(score.view(n, k), torch.softmax(want_val, dim=1), rtol=1e-5, atol=1e-6)
    imp = torch.zeros(e, device=device).index_add(0, want_idx.reshape(-1), torch.softmax(want_val, dim=1).reshape(-1))
    load = torch.bincount(want_idx.reshape(-1), minlength=e).float()
    assert torch.allclose(gate.get_loss(), cv2(imp) + cv2(load), rtol=1e-4)
    assert hasattr(idx, "_fmoe_route")

    gate.train()
    torch.manual_seed(99)
    idx, score = gate(x)
    torch.manual_seed(99)
    noise = torch.randn_like(clean)
    std = torch.nn.functional.softplus(x @ gate.w_noise) + 1e-2
    noisy = clean + noise * std
    want_val, want_idx = torch.topk(noisy, k, dim=1, sorted=True)
    assert torch.equal(idx.view(n, k), want_idx)
    assert torch.allclose(score.view(n, k), torch.softmax(want_val, dim=1), rtol=1e-5, atol=1e-6)
    prob = torch.zeros(n, e, dtype=torch.float64)
    nz, cl, sd = noisy.detach().double().cpu(), clean.detach().double().cpu(), std.detach().double().cpu()
    for t in range(n):
        for i in range(e):
            others = torch.cat([nz[t, :i], nz[t, i + 1:]]).sort(descending=True).values
            z = (cl[t, i] - others[k - 1]) / sd[t, i]
            prob[t, i] = 0.5 * (1 + math.erf(float(z) / math.sqrt(2)))
    imp = torch.zeros(e, device=device).index_add(0, want_idx.reshape(-1), torch.softmax(want_val, dim=1).reshape(-1))
    want_loss = cv2(imp.detach().double().cpu()) + cv2(prob.sum(0))
    loss = gate.get_loss()
    assert abs(float(loss.detach()) - float(want_loss)) <= 1e-4 * float(want_loss)
    loss.backward()
    assert gate.w_noise.grad is not None and torch.isfinite(gate.w_noise.grad).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_scatter_in_the_gemm_loader_equals_the_scattered_copy(dtype, device, monkeypatch):
    """The fused pipeline's first GEMM reads the token rows through pos in its loader
    (FMOE_FOLD_SCATTER=0: from a scattered copy made by the permute stage, as
    fmoe/fused_functions.py:22 does).  Same bits out of the forward -- the products and their order
    are identical -- and the same gradients; drops, an empty expert, ragged tiles, several chunks."""
    from fastermoe_amd import fmoe_native
    monkeypatch.setenv("FMOE_FUSE_GRAN", "3")
    torch.manual_seed(77)
    n, d, h, e, k = 700, 128, 320, 5, 2
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.GELU())
    moe.enable_fuse = True
    moe = moe.to(dtype).to(device)
    x = torch.randn(n, d).to(dtype).to(device)
    idx = torch.randint(-1, e - 1, (n, k), device=device)
    score = torch.rand(n, k, device=device).to(dtype)
    moe.gate.forward = lambda inp: (idx, score)
    results = []
    for flag in ("1", "0"):
        monkeypatch.setenv("FMOE_FOLD_SCATTER", flag)
        moe.zero_grad()
        xi = x.clone().requires_grad_(True)
        out = moe(xi)
        out.float().mean().backward()
        results.append([out, xi.grad] + [p.grad.clone() for p in moe.experts.parameters()])
    for a, b in zip(*results):
        assert torch.equal(a, b)
    # and the low-level call really runs without a scattered copy
    cnt, pos_buf, s2r = fmoe_native.route(idx, e)
    pos = pos_buf[: int(cnt.sum())]
    ex = moe.experts
    monkeypatch.setenv("FMOE_FOLD_SCATTER", "1")
    _, buf_in, _, _ = fmoe_native.fused_mlp_forward(x, pos, s2r, cnt.cpu(), ex.htoh4.weight, ex.htoh4.bias,
                                                    ex.h4toh.weight, ex.h4toh.bias, k, 2, 3)
    assert buf_in is None


FULL_SIZE = [  # name, tokens, d_model, d_hidden, experts, top_k, fused, routing
    ("gshard-style top-2 with capacity drops", 16384, 1024, 4096, 16, 2, False, "capacity"),
    ("skewed switch-style top-1", 16384, 2048, 8192, 64, 1, False, "zipf"),
    ("mixtral-like share, fused pipeline with 4 chunks", 32768, 4096, 14336, 8, 2, True, "topk"),
    ("fine-grained top-8", 8192, 2048, 1024, 256, 8, False, "biased"),
]


@pytest.mark.parametrize("name,n,d,h,e,k,fuse,routing", FULL_SIZE, ids=[c[0].split(",")[0].replace(" ", "-") for c in FULL_SIZE])
def test_bf16_configurations_at_full_size_sampled_against_the_oracle(name, n, d, h, e, k, fuse, routing, device, monkeypatch):
    """The four bf16 benchmark configurations at their FULL size: one forward + backward on the GPU, then
      * output and input gradient of 48 sampled tokens against the float64 oracle run on those tokens
        (a token's output and input gradient depend on no other token);
      * for the expert with the most rows and 8 of its hidden units, the matching rows of grad_w1 / grad_b1
        and columns of grad_w2, plus all of grad_b2, computed in float64 on the CPU over ALL of that expert's
        rows from the textbook formulas
            gy = score * grad_out[token],  pre_J = x W1[J]^T + b1[J],  mid_J = gelu(pre_J),
            grad_w2[:, J] = gy^T mid_J,  g_pre_J = (gy W2[:, J]) * gelu'(pre_J),
            grad_w1[J] = g_pre_J^T x,  grad_b1[J] = sum g_pre_J,  grad_b2 = sum gy;
      * an expert without rows (the skewed routing leaves some) has zero gradients.
    In the fused case the contraction of the weight gradients runs over the whole expert although the
    pipeline's chunks cut it, and the last chunk ends in a split tail."""
    from fastermoe_amd.gates.utils import limit_by_capacity
    monkeypatch.setenv("FMOE_FUSE_GRAN", "4")
    monkeypatch.delenv("FMOE_GEMM_TILE", raising=False)
    torch.manual_seed(e)
    with torch.device(device):
        moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.GELU())
        with torch.no_grad():
            moe.experts.htoh4.weight.mul_((d * h) ** 0.5 * d ** -0.5)   # unit-variance activations
            moe.experts.h4toh.weight.mul_((d * h) ** 0.5 * h ** -0.5)
            moe.experts.htoh4.bias.normal_(0, 0.1)
            moe.experts.h4toh.bias.normal_(0, 0.1)
        moe = moe.to(torch.bfloat16)
        x = torch.randn(n, d).bfloat16().requires_grad_(True)
        grad = torch.randn(n, d).bfloat16()
        logits = torch.randn(n, e)
        if routing == "biased":
            logits = logits + 0.5 * torch.randn(e)
        if routing == "capacity":
            logits = logits + torch.linspace(-0.6, 0.6, e)   # mild imbalance, so that some experts overflow
    moe.enable_fuse = fuse
    if routing == "zipf":
        idx = zipf_experts(n, e, 1.2, torch.Generator().manual_seed(7)).view(n, 1).to(device)
        score = torch.ones(n, 1, dtype=torch.bfloat16, device=device)
    else:
        val, idx = torch.topk(logits, k, dim=-1)
        score = torch.softmax(val, dim=-1).bfloat16()
        if routing == "capacity":
            idx = limit_by_capacity(idx, e, 1, math.ceil(1.2 * n * k / e))[2]
            assert 0 < int((idx < 0).sum()) < n * k // 2
    moe.gate.forward = lambda inp: (idx, score)
    out = moe(x)
    out.backward(grad)
    ex = moe.experts
    w1, b1, w2, b2 = ex.htoh4.weight, ex.htoh4.bias, ex.h4toh.weight, ex.h4toh.bias

    # -- sampled tokens: output and input gradient
    sample = torch.randperm(n, generator=torch.Generator().manual_seed(5))[:48].to(device)
    ref = omoe.moe_mlp_forward_backward_per_expert(x[sample], idx[sample], score[sample], w1, b1, w2, b2, "gelu", k,
                                                   grad_out=grad[sample], grad_dtype=torch.float32)
    # (two roundings to bfloat16 on the way to these: floor 1; the weight gradients below, four and a long sum: 3)
    assert_close(out[sample], ref["out"], 2e-2, f"{name}: output of the sampled tokens", floor=1.0)
    assert_close(x.grad[sample], ref["grad_inp"], 2e-2, f"{name}: input gradient of the sampled tokens", floor=1.0)
    del ref

    # -- the largest expert, 8 hidden units: weight and bias gradients over all of the expert's rows
    f64 = torch.float64
    counts = torch.bincount(idx[idx >= 0].reshape(-1), minlength=e)
    e0 = int(counts.argmax())
    units = torch.tensor([0, 1, 255, 256, h // 2, h // 2 + 1, h - 2, h - 1], device=device)
    slots = torch.nonzero(idx.reshape(-1) == e0).reshape(-1)
    tok = slots // k
    xe = x.detach()[tok].to("cpu", f64)
    gy = score.reshape(-1)[slots].to("cpu", f64).unsqueeze(1) * grad[tok].to("cpu", f64)
    w1_j = w1[e0][units].detach().to("cpu", f64)           # [8, d]
    w2_j = w2[e0][:, units].detach().to("cpu", f64)        # [d, 8]
    pre = xe @ w1_j.t() + b1[e0][units].detach().to("cpu", f64)
    cdf = 0.5 * (1.0 + torch.erf(pre / 2.0 ** 0.5))
    mid = pre * cdf
    dact = cdf + pre * torch.exp(-0.5 * pre * pre) / (2.0 * math.pi) ** 0.5
    g_pre = (gy @ w2_j) * dact
    assert_close(w2.grad[e0][:, units], gy.t() @ mid, 2e-2, f"{name}: grad_w2 columns", floor=3.0)
    assert_close(w1.grad[e0][units], g_pre.t() @ xe, 2e-2, f"{name}: grad_w1 rows", floor=3.0)
    assert_close(b1.grad[e0][units], g_pre.sum(0), 2e-2, f"{name}: grad_b1 entries", floor=3.0)
    assert_close(b2.grad[e0], gy.sum(0), 2e-2, f"{name}: grad_b2", floor=3.0)
    for empty in torch.nonzero(counts == 0).reshape(-1).tolist()[:2]:
        assert torch.count_nonzero(w1.grad[empty]) == 0 and torch.count_nonzero(w2.grad[empty]) == 0
        assert torch.count_nonzero(b1.grad[empty]) == 0 and torch.count_nonzero(b2.grad[empty]) == 0


class _CountReadingExperts(nn.Module):
    """A user's fused expert module: reads the counts on the host, as the reference allows."""

    def __init__(self, num_expert, d_model):
        super().__init__()
        self.scale = nn.Parameter(torch.arange(1.0, num_expert + 1))
        self.seen = None

    def forward(self, inp, fwd_expert_count):
        sizes = fwd_expert_count.tolist()
        assert sum(sizes) == inp.shape[0], "a fused expert module gets exactly the routed rows"
        self.seen = sizes
        return inp * torch.repeat_interleave(self.scale, torch.tensor(sizes, device=inp.device)).unsqueeze(1)


def test_user_fused_experts_get_the_routed_rows_and_readable_counts(device):
    """The layer defers the read-back of the expert counts only for its own expert module; a user's
    fused module sees exactly the routed rows (dropped slots are gone) and counts it can read."""
    torch.manual_seed(3)
    n, d, e, k = 200, 32, 4, 2

    class Layer(FMoE):
        def __init__(self):
            super().__init__(num_expert=e, d_model=d, top_k=k, gate=NaiveGate)
            self.experts = _CountReadingExperts(e, d)

    moe = Layer().to(device)
    x = torch.randn(n, d, device=device, requires_grad=True)
    idx = torch.randint(-1, e, (n, k), device=device)          # -1: dropped slots
    score = torch.rand(n, k, device=device)
    moe.gate.forward = lambda inp: (idx, score)
    out = moe(x)
    assert moe.experts.seen == torch.bincount(idx[idx >= 0].view(-1).cpu(), minlength=e).tolist()
    scale = torch.where(idx >= 0, moe.experts.scale.detach()[idx.clamp(min=0)], torch.zeros((), device=device))
    ref = x.detach() * (score * scale).sum(dim=1, keepdim=True)
    assert torch.allclose(out, ref, rtol=1e-5, atol=1e-6)
    out.sum().backward()
    assert torch.allclose(x.grad, (score * scale).sum(dim=1, keepdim=True).expand(n, d), rtol=1e-5, atol=1e-6)


def test_replaced_expert_fn_reads_ready_counts(device):
    """Only FMoE.expert_fn itself is bypassed by the layer's own path over device tables.  An
    overriding sub-class, or a function assigned on the instance as the reference's tests do
    (``model.expert_fn = ...``), is called with exactly the routed rows and CPU counts that are
    there to read, and its result is what the layer returns."""
    torch.manual_seed(5)
    n, d, h, e, k = 300, 32, 64, 4, 2
    seen = []

    class Sub(fmoe.FMoETransformerMLP):
        def expert_fn(self, inp, models, fwd_expert_count, num_expert):
            seen.append((inp.shape[0], fwd_expert_count.view(-1).tolist()))
            return super().expert_fn(inp, models, fwd_expert_count, num_expert)

    idx = torch.randint(-1, e, (n, k), device=device)
    score = torch.rand(n, k, device=device)
    want = torch.bincount(idx[idx >= 0].view(-1).cpu(), minlength=e).tolist()
    x = torch.randn(n, d, device=device)
    plain = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k).to(device)
    sub = Sub(num_expert=e, d_model=d, d_hidden=h, top_k=k).to(device)
    sub.load_state_dict(plain.state_dict())
    assigned = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k).to(device)
    assigned.load_state_dict(plain.state_dict())
    original = assigned.expert_fn

    def replacement(inp, models, fwd_expert_count, num_expert):
        seen.append((inp.shape[0], [int(c) for c in fwd_expert_count.view(-1, num_expert).sum(0)]))
        return original(inp, models, fwd_expert_count, num_expert)

    assigned.expert_fn = replacement
    outs = []
    for moe in (plain, sub, assigned):
        moe.gate.forward = lambda inp: (idx, score)
        xi = x.clone().requires_grad_(True)
        out = moe(xi)
        out.sum().backward()
        outs.append((out, xi.grad, moe.experts.htoh4.weight.grad))
    assert seen == [(sum(want), want), (sum(want), want)]
    for other in outs[1:]:
        for a, b in zip(outs[0], other):
            assert rel_err(a, b) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("fold", ["1", "0"])
def test_unfused_layer_over_device_tables_equals_the_host_count_path(dtype, fold, device, monkeypatch):
    """The unfused layer's own path (row segments from a device table, token rows read through pos in
    the first GEMM's loader, no scattered copy, nothing read back) against FMOE_DEVICE_TABLES=0
    (MOEScatter, host counts, as fmoe/layers.py:117-148): the same products in the same order, so
    the same bits out of the forward and the same gradients.  Drops, an empty expert, ragged tiles."""
    torch.manual_seed(78)
    monkeypatch.setenv("FMOE_FOLD_COMBINE", fold)
    monkeypatch.setenv("FMOE_GEMM_TILE", "128x128")   # (the two paths pick the tile from different estimates)
    n, d, h, e, k = 700, 128, 320, 5, 2
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.GELU())
    moe = moe.to(dtype).to(device)
    x = torch.randn(n, d).to(dtype).to(device)
    idx = torch.randint(-1, e - 1, (n, k), device=device)
    score = torch.rand(n, k, device=device).to(dtype)
    moe.gate.forward = lambda inp: (idx, score)
    results = []
    for flag in ("1", "0"):
        monkeypatch.setenv("FMOE_DEVICE_TABLES", flag)
        moe.zero_grad()
        xi = x.clone().requires_grad_(True)
        out = moe(xi)
        out.float().mean().backward()
        results.append([out, xi.grad] + [p.grad.clone() for p in moe.experts.parameters()])
    for a, b in zip(*results):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layer_forward_in_a_hip_graph_with_new_routing_per_replay(dtype, device):
    """Nothing in the unfused layer's forward waits for the host (the row segments stay on the device),
    so gate, routing, both grouped GEMMs and the combine can be captured in one HIP graph.  The graph
    is replayed on inputs that route differently each time (other expert counts, other tile counts),
    with eager work and synchronisations between the replays; every replay must equal the eager
    forward on the same input, bit for bit."""
    torch.manual_seed(9)
    n, d, h, e, k = 1500, 128, 256, 6, 2
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.GELU())
    moe = moe.to(dtype).to(device).eval()
    with torch.no_grad():
        moe.gate.gate.weight.mul_(30.0)   # well separated logits
    inputs = [torch.randn(n, d).to(dtype).to(device) for _ in range(4)]
    # skew the routing differently per input: push the tokens towards one expert's gate row
    for i, xin in enumerate(inputs):
        xin[: n // 2] += 0.5 * moe.gate.gate.weight[i % e].detach().to(dtype) / 30.0
    static_x = inputs[0].clone()
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                moe(static_x)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_out = moe(static_x)
        counts_seen = set()
        for rep in range(6):
            xin = inputs[rep % len(inputs)]
            static_x.copy_(xin)
            graph.replay()
            torch.cuda.synchronize()
            got = static_out.clone()
            want = moe(xin)                     # eager work between the replays
            idx, _ = moe.gate(xin)
            counts_seen.add(tuple(torch.bincount(idx.view(-1), minlength=e).tolist()))
            torch.cuda.synchronize()
            assert torch.equal(got, want), f"replay {rep}"
    assert len(counts_seen) >= 3   # the replays really routed differently


@pytest.mark.parametrize("dtype", [torch.float32])
@pytest.mark.parametrize("n,d,e,k", [(40, 16, 6, 2), (3000, 64, 64, 4), (1111, 32, 300, 8), (700, 48, 9, 1)])
def test_noisy_gate_kernel_against_the_torch_formulation(dtype, n, d, e, k, device, monkeypatch):
    """NoisyGate in training mode: the one-pass kernel (noise, softplus, top-(k+1), softmax, smooth load,
    routing) and its backward against the same gate written out in torch operators
    (FMOE_NOISY_GATE_KERNEL=0) with the same noise draw: indices, gates, loss, and the gradients of
    both weight matrices and of the input through loss + gates; the routing against the oracle."""
    torch.manual_seed(n + e)
    gate = NoisyGate(d, e, 1, top_k=k).to(device)
    with torch.no_grad():
        gate.w_gate.normal_(0, 1.0 / d ** 0.5)
        gate.w_noise.normal_(0, 1.0 / d ** 0.5)
    gate = gate.to(dtype)
    gate.train()
    x = torch.randn(n, d, device=device).to(dtype)
    g = torch.randn(n, 1, k, device=device).to(dtype)
    results = []
    for flag in ("1", "0"):
        monkeypatch.setenv("FMOE_NOISY_GATE_KERNEL", flag)
        gate.zero_grad()
        xi = x.clone().requires_grad_(True)
        torch.manual_seed(5)
        idx, score = gate(xi)
        loss = gate.get_loss()
        (loss + (score * g).float().sum()).backward()
        results.append((idx, score, loss.detach(), xi.grad, gate.w_gate.grad.clone(), gate.w_noise.grad.clone()))
        if flag == "1":
            assert hasattr(idx, "_fmoe_route")
            cnt, pos_buf, s2r = idx._fmoe_route[2:]
            ref_pos, ref_cnt = orouting.count_by_gate(idx.cpu().numpy(), e)
            assert np.array_equal(cnt.cpu().numpy(), ref_cnt) and np.array_equal(pos_buf.cpu().numpy(), ref_pos)
    (idx_a, sc_a, loss_a, gx_a, gwg_a, gwn_a), (idx_b, sc_b, loss_b, gx_b, gwg_b, gwn_b) = results
    assert torch.equal(idx_a, idx_b)
    assert torch.allclose(sc_a, sc_b, rtol=1e-5, atol=1e-6)
    assert abs(float(loss_a) - float(loss_b)) <= 1e-4 * abs(float(loss_b))
    for a, b in ((gx_a, gx_b), (gwg_a, gwg_b), (gwn_a, gwn_b)):
        assert rel_err(a, b) <= 1e-4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,e,k", [(3000, 64, 4), (500, 12, 2)])
def test_noisy_top_k_16_bit_against_float64(dtype, n, e, k, device):
    """NoisyTopK on 16-bit logits (the kernel computes in float32 and rounds its outputs once) against
    the same formulas in float64 on the same 16-bit inputs: indices equal, gates / load / gradients
    within 2e-2."""
    from fastermoe_amd.functions import NoisyTopK
    torch.manual_seed(e)
    clean = torch.randn(n, e, device=device).to(dtype).requires_grad_(True)
    raw = torch.randn(n, e, device=device).to(dtype).requires_grad_(True)
    noise = torch.randn(n, e, device=device).to(dtype)
    gg = torch.randn(n, k, device=device).to(dtype)
    gl = torch.randn(e, device=device)
    idx, gates, load = NoisyTopK.apply(clean, raw, noise, k, 1e-2)
    ((gates * gg).float().sum() + (load * gl).sum()).backward()
    c64, r64 = clean.detach().double().requires_grad_(True), raw.detach().double().requires_grad_(True)
    std = torch.nn.functional.softplus(r64) + 1e-2
    noisy = c64 + noise.double() * std
    top_vals, top_idx = noisy.topk(k + 1, dim=1)
    assert torch.equal(idx, top_idx[:, :k])
    ref_gates = torch.softmax(top_vals[:, :k], dim=1)
    inside = noisy > top_vals[:, k:k + 1]
    thr = torch.where(inside, top_vals[:, k:k + 1], top_vals[:, k - 1:k])
    ref_load = torch.special.ndtr((c64 - thr) / std).sum(dim=0)
    ((ref_gates * gg.double()).sum() + (ref_load * gl.double()).sum()).backward()
    tol = TOL[dtype]
    assert rel_err(gates, ref_gates) <= tol and rel_err(load, ref_load) <= 1e-4
    assert_close(clean.grad, c64.grad, tol, "grad_clean")
    assert_close(raw.grad, r64.grad, tol, "grad_raw")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ["one_token", "one_expert_takes_all", "all_dropped", "single_expert_layer",
                                  "one_slot_survives", "more_experts_than_rows"])
def test_device_table_path_at_extreme_routings(case, dtype, device):
    """The layer's own unfused path (segment table built on the device, launches sized for an upper
    bound of tiles) at the routings that stress that bound: a single token, every slot on one expert,
    no surviving slot at all, a one-expert layer, a single surviving slot, and more experts than
    rows.  Against the brute-force oracle (tests/moe.py:30-49 semantics: a dropped slot contributes a
    zero row); experts without rows must come out with zero gradients."""
    torch.manual_seed(91)
    n, d, h, e, k = 37, 64, 96, 6, 2
    if case == "one_token":
        n = 1
    if case == "single_expert_layer":
        e, k = 1, 1
    if case == "more_experts_than_rows":
        n, e = 3, 40
    moe = fmoe.FMoETransformerMLP(num_expert=e, d_model=d, d_hidden=h, top_k=k, activation=nn.GELU())
    moe = moe.to(dtype).to(device)
    x = torch.randn(n, d).to(dtype).to(device)
    idx = torch.randint(0, e, (n, k), device=device)
    if case == "one_expert_takes_all":
        idx.fill_(e - 2)
    elif case == "all_dropped":
        idx.fill_(-1)
    elif case == "one_slot_survives":
        idx.fill_(-1)
        idx[n // 2, 1] = 3
    score = torch.rand(n, k, device=device).to(dtype)
    x = x.clone().requires_grad_(True)
    moe.gate.forward = lambda inp: (idx, score)
    out = moe(x)
    out.float().sum().backward()
    ex = moe.experts
    ref = omoe.moe_mlp_forward_backward(x, idx, score, ex.htoh4.weight, ex.htoh4.bias, ex.h4toh.weight, ex.h4toh.bias,
                                        nn.GELU(), k, loss="sum")
    tol = TOL[dtype]
    got = {"out": out, "grad_inp": x.grad, "grad_w1": ex.htoh4.weight.grad, "grad_w2": ex.h4toh.weight.grad,
           "grad_b1": ex.htoh4.bias.grad, "grad_b2": ex.h4toh.bias.grad}
    counts = torch.bincount(idx[idx >= 0].view(-1).cpu(), minlength=e)
    for name, val in got.items():
        assert val is not None and torch.isfinite(val.float()).all(), name
        want = ref[name] if ref[name] is not None else torch.zeros(val.shape, dtype=torch.float64)   # (no slot used it)
        scale = max(want.abs().max().item(), 1.0)
        assert (val.double().cpu() - want.double().cpu()).abs().max().item() <= tol * scale, name
    for name in ("grad_w1", "grad_w2", "grad_b1", "grad_b2"):
        for expert in range(e):
            if counts[expert] == 0:
                assert torch.count_nonzero(got[name][expert]) == 0, (name, expert)
