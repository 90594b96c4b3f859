"""GPU parity of the local scatter / gather kernels against the torch index ops that
define them in the reference (fmoe/functions.py:72-84); copies are bit-exact, sums are
compared with a float32 sequential sum in the kernel's documented order."""
import numpy as np
import pytest
import torch

from fastermoe_amd import fmoe_native
from fastermoe_amd.functions import MOEGather, MOEScatter, _local_gather, _local_scatter

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16, torch.float64]


def _route(n, k, e, drop, seed, device):
    g = torch.Generator().manual_seed(seed)
    gate = torch.randint(0, e, (n, k), generator=g)
    gate[torch.rand(n, k, generator=g) < drop] = -1
    cnt, pos_buf, s2r = fmoe_native.route(gate.to(device), e)
    pos = pos_buf[: int(cnt.sum())]
    return gate, pos, s2r


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,k,d,drop", [(512, 2, 1024, 0.0), (300, 3, 72, 0.25), (64, 1, 5, 0.1), (1, 2, 8, 0.0)])
def test_scatter_and_gather_copy(dtype, n, k, d, drop, device):
    gate, pos, s2r = _route(n, k, 6, drop, n + d, device)
    x = torch.randn(n, d).to(dtype)
    xd = x.to(device)
    pos_c = pos.cpu()
    # scatter = index_select
    buf = _local_scatter(xd, pos // k)
    assert torch.equal(buf.cpu(), torch.index_select(x, 0, pos_c // k))
    # the same scatter straight from the slot positions (index // k inside the kernel), over the whole position
    # buffer: its -1 tail gives zero rows
    cnt, pos_buf, _ = fmoe_native.route(gate.to(device), 6)
    full = fmoe_native.gather_rows(xd, pos_buf, index_div=k)
    assert full.shape[0] == n * k and torch.equal(full[: pos.numel()], buf)
    assert torch.count_nonzero(full[pos.numel():]) == 0
    # gather (copy) = zeros + index_copy_
    y = torch.randn(pos.numel(), d).to(dtype)
    ref = torch.zeros(n * k, d, dtype=dtype).index_copy_(0, pos_c, y)
    got = _local_gather(y.to(device), pos, n * k, maybe_overlap=False)
    assert torch.equal(got.cpu(), ref)
    got2 = fmoe_native.gather_rows(y.to(device), s2r, n * k)
    assert torch.equal(got2.cpu(), ref)


def _sequential_index_add(y, index, n_out, acc_dtype):
    out = torch.zeros(n_out, y.shape[1], dtype=acc_dtype)
    for i in range(y.shape[0]):        # ascending source row = the kernel's order
        out[index[i]] += y[i].to(acc_dtype)
    return out.to(y.dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,k,d,drop", [(256, 2, 512, 0.0), (100, 8, 40, 0.2), (50, 3, 7, 0.0), (40, 20, 16, 0.1)])
def test_gather_add(dtype, n, k, d, drop, device):
    gate, pos, s2r = _route(n, k, 5, drop, 3 * n + d, device)
    pos_c = pos.cpu()
    y = torch.randn(pos.numel(), d).to(dtype)
    acc = torch.float64 if dtype == torch.float64 else torch.float32
    # the per-token reduction adds a token's rows in ascending slot order
    order_ref = torch.zeros(n, d, dtype=acc)
    s2r_c = s2r.cpu().view(n, k)
    for j in range(k):
        live = s2r_c[:, j] >= 0
        order_ref[live] += y[s2r_c[live, j]].to(acc)
    got = fmoe_native.reduce_slots(y.to(device), s2r, n, k)
    assert torch.equal(got.cpu(), order_ref.to(dtype))
    # the general index-add adds in ascending source row
    ref = _sequential_index_add(y, pos_c // k, n, acc)
    got2 = _local_gather(y.to(device), pos // k, n, maybe_overlap=True)
    assert torch.equal(got2.cpu(), ref)
    # and agrees with torch's index_add_ up to summation order
    lib = torch.zeros(n, d, dtype=torch.float64).index_add_(0, pos_c // k, y.double())
    tol = {torch.float32: 1e-5, torch.float64: 1e-12}.get(dtype, 2e-2)
    assert (got2.cpu().double() - lib).abs().max() <= tol * max(1.0, lib.abs().max().item())


def test_index_add_long_chains(device):
    """More sources per row than the reducer sorts at once (several passes)."""
    g = torch.Generator().manual_seed(9)
    idx = torch.randint(0, 3, (70,), generator=g)
    y = torch.randn(70, 24, generator=g)
    ref = _sequential_index_add(y, idx, 4, torch.float32)
    got = fmoe_native.index_add_rows(y.to(device), idx.to(device), 4)
    assert torch.equal(got.cpu(), ref)
    assert torch.count_nonzero(got[3]) == 0


def test_autograd_functions_match_torch_index_ops(device):
    n, k, d = 128, 2, 64
    gate, pos, s2r = _route(n, k, 4, 0.2, 77, device)
    x = torch.randn(n, d, device=device, requires_grad=True)
    xr = x.detach().clone().requires_grad_(True)
    w = torch.randn(pos.numel(), d, device=device)
    for extras in ((), (s2r, k)):
        x.grad = None
        buf = MOEScatter.apply(x, pos // k, None, None, None, pos.numel(), 1, *extras)
        (buf * w).sum().backward()
        xr.grad = None
        (torch.index_select(xr, 0, pos // k) * w).sum().backward()
        assert torch.equal(buf, torch.index_select(xr, 0, pos // k))
        assert torch.allclose(x.grad, xr.grad, rtol=1e-6, atol=1e-6)
    y = torch.randn(pos.numel(), d, device=device, requires_grad=True)
    w2 = torch.randn(n * k, d, device=device)
    out = MOEGather.apply(y, pos, None, None, None, n * k, 1)
    (out * w2).sum().backward()
    assert torch.equal(y.grad, w2[pos])
    assert torch.equal(out, torch.zeros(n * k, d, device=device).index_copy_(0, pos, y.detach()))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,k,d", [(300, 2, 1024), (64, 8, 40), (17, 3, 7), (5, 1, 16)])
def test_combine_matches_bmm(dtype, n, k, d, device):
    """The score-weighted top-k combination and its backward against torch.bmm in float64."""
    from fastermoe_amd.functions import MOECombine
    g = torch.Generator().manual_seed(n * k + d)
    x = torch.randn(n * k, d, generator=g).to(dtype)
    score = torch.randn(n, 1, k, generator=g).to(dtype)
    go = torch.randn(n, d, generator=g).to(dtype)
    x64 = x.detach().clone().double().requires_grad_(True)
    s64 = score.detach().clone().double().requires_grad_(True)
    ref = torch.bmm(s64, x64.view(n, k, d)).reshape(n, d)
    ref.backward(go.double())
    xd = x.detach().to(device).requires_grad_(True)
    sd = score.detach().to(device).requires_grad_(True)
    out = MOECombine.apply(xd, sd, n, k)
    out.backward(go.to(device))
    tol = {torch.float32: 1e-5, torch.float64: 1e-12}.get(dtype, 2e-2)
    for got, want in ((out, ref), (xd.grad, x64.grad), (sd.grad, s64.grad)):
        assert got.shape == want.shape
        assert (got.double().cpu() - want).abs().max() <= tol * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,k,d,e,drop", [(300, 2, 1024, 8, 0.2), (64, 8, 40, 16, 0.5), (17, 3, 7, 4, 0.0),
                                          (5, 1, 16, 3, 1.0)])
def test_gather_combine_matches_gather_then_bmm(dtype, n, k, d, e, drop, device):
    """The folded gather + combine and its backward against _local_gather (zero rows for
    dropped slots, fmoe/functions.py:77-84) followed by torch.bmm (fmoe/layers.py:321-322),
    both in float64 on the CPU."""
    from fastermoe_amd.functions import MOEGatherCombine
    gate, pos, s2r = _route(n, k, e, drop, n * 31 + d, device)
    n_rows = pos.numel()
    g = torch.Generator().manual_seed(n * k + d)
    rows = torch.randn(n_rows, d, generator=g).to(dtype)
    score = torch.randn(n, k, generator=g).to(dtype)
    go = torch.randn(n, d, generator=g).to(dtype)
    r64 = rows.detach().clone().double().requires_grad_(True)
    s64 = score.detach().clone().double().requires_grad_(True)
    slots = torch.zeros(n * k, d, dtype=torch.float64).index_copy(0, pos.cpu(), r64)
    ref = torch.bmm(s64.view(n, 1, k), slots.view(n, k, d)).reshape(n, d)
    ref.backward(go.double())
    rd = rows.detach().to(device).requires_grad_(True)
    sd = score.detach().to(device).requires_grad_(True)
    out = MOEGatherCombine.apply(rd, s2r, sd, n, k)
    out.backward(go.to(device))
    tol = {torch.float32: 1e-5, torch.float64: 1e-12}.get(dtype, 2e-2)
    for got, want in ((out, ref), (rd.grad, r64.grad), (sd.grad, s64.grad)):
        assert got.shape == want.shape
        if want.numel():
            assert (got.double().cpu() - want).abs().max() <= tol * max(1.0, want.abs().max().item())
    # dropped slots get a zero score gradient
    assert torch.count_nonzero(sd.grad.view(-1)[s2r < 0]) == 0


def test_full_size_round_trip(device):
    """config-4 sized rows: scatter then gather restores every kept slot, dropped slots are zero;
    linearity of the reduction."""
    n, k, d = 32768, 2, 4096
    gate, pos, s2r = _route(n, k, 8, 0.05, 4, device)
    x = torch.randn(n, d, device=device, dtype=torch.bfloat16)
    buf = _local_scatter(x, pos // k)
    back = fmoe_native.gather_rows(buf, s2r, n * k).view(n, k, d)
    kept = (s2r >= 0).view(n, k)
    assert torch.equal(back[kept], x[:, None, :].expand(n, k, d)[kept])
    assert torch.count_nonzero(back[~kept]) == 0
    red = fmoe_native.reduce_slots(buf, s2r, n, k)
    expect = (x.float() * kept.sum(1, keepdim=True)).to(torch.bfloat16)   # x + x or x or 0: exact in bf16
    assert torch.equal(red, expect)
