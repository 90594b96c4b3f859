"""GPU parity of the per-expert linear (grouped GEMM) against the float64 oracle.

Tolerances (relative to the largest reference magnitude): 1e-5 for float32,
2e-2 for bfloat16 / float16, 1e-10 for float64."""
import pytest
import torch

from fastermoe_amd import fmoe_native
from fastermoe_amd.functions import MOELinear
from oracle import moe as omoe
from helpers import TOL, assert_close, ragged_counts, rel_err

pytestmark = pytest.mark.gpu


def _reference(x, counts, w, b, gy):
    x64 = x.double().requires_grad_(True)
    w64 = w.double().requires_grad_(True)
    b64 = b.double().requires_grad_(True) if b is not None else None
    y = omoe.per_expert_linear(x64, counts, w64, b64)
    y.backward(gy.double())
    return y.detach(), x64.grad, w64.grad, (b64.grad if b is not None else None)


CASES = [  # rows, experts, in, out, bias, empties
    (1000, 4, 64, 128, True, 1),     # ragged segments, one empty expert
    (777, 8, 256, 72, True, 2),      # out not a multiple of the tile, rows odd
    (2048, 2, 512, 512, False, 0),   # full tiles
    (300, 16, 40, 24, True, 5),      # many empty experts, tiny segments
    (5, 3, 8, 8, True, 1),           # fewer rows than a tile
    (0, 3, 16, 16, True, 3),         # no rows at all
    (64, 2, 12, 20, True, 0),        # feature sizes off the vector grid -> any-shape kernel
    (33, 1, 4, 8, False, 0),         # the shape of the reference's fused test (d=4, h=8)
]


# The MFMA kernel is built for three tile shapes (256 x 256 and 128 x 256 with eight waves, 128 x 128
# with four); the library picks one from the launch's tile count.  FMOE_GEMM_TILE forces one, so
# that every shape runs every case.
TILES = [None, "256x256", "128x256", "128x128"]


@pytest.fixture(params=TILES, ids=lambda t: t or "auto")
def tile(request, monkeypatch):
    if request.param is None:
        monkeypatch.delenv("FMOE_GEMM_TILE", raising=False)
    else:
        monkeypatch.setenv("FMOE_GEMM_TILE", request.param)
    return request.param


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.float64])
@pytest.mark.parametrize("rows,e,fin,fout,bias,empties", CASES)
def test_linear_forward_backward(dtype, rows, e, fin, fout, bias, empties, device, tile):
    g = torch.Generator().manual_seed(rows + e + fin)
    counts = ragged_counts(rows, e, g, empties) if rows else torch.zeros(e, dtype=torch.int64)
    x = (torch.randn(rows, fin, generator=g)).to(dtype)
    w = (torch.randn(e, fout, fin, generator=g) / fin ** 0.5).to(dtype)
    b = torch.randn(e, fout, generator=g).to(dtype) if bias else None
    gy = torch.randn(rows, fout, generator=g).to(dtype)
    ref_y, ref_gx, ref_gw, ref_gb = _reference(x, counts, w, b, gy)

    xd, wd, gyd = x.to(device), w.to(device), gy.to(device)
    bd = b.to(device) if bias else None
    y = fmoe_native.linear_forward(xd, counts, wd, bd)
    tol = TOL[dtype]
    assert y.shape == (rows, fout) and y.dtype == dtype
    assert rel_err(y, ref_y) <= tol
    gx, gw, gb = fmoe_native.linear_backward(gyd, xd, counts, wd, bd)
    assert rel_err(gx, ref_gx) <= tol
    assert rel_err(gw, ref_gw) <= tol
    for ex in range(e):
        if counts[ex] == 0:
            assert torch.count_nonzero(gw[ex]) == 0      # cuda/parallel_linear.cuh:113-118
    if bias:
        assert rel_err(gb, ref_gb) <= tol
    else:
        assert gb is None


# The grouped GEMM keeps three slabs of 128 contraction bytes in flight (64 bf16 / 32 fp32
# elements each): contraction lengths of one to five slabs, with and without a ragged tail,
# for the forward/data-grad (contraction = features) and the weight-grad (contraction = the
# expert's rows), several row and column tiles per expert, and both tile heights (launches
# of 512 tiles and more use 256-row tiles, smaller ones 128) -- and every tile shape forced.
DEPTH_CASES = [  # rows, experts, in, out
    (300, 2, 64, 264),      # one slab (bf16), column tail
    (520, 2, 128, 256),     # two slabs
    (600, 3, 192, 520),     # three slabs: every P buffer used once
    (700, 2, 200, 300),     # three slabs and a tail of 8
    (1100, 2, 328, 272),    # five slabs and a tail, experts of 4-5 row tiles
    (63, 1, 64, 256),       # weight-grad contraction shorter than a slab
    (129, 2, 72, 8200),     # 33 column tiles
    (9000, 2, 256, 4100),   # 36 x 17 tiles of 256 rows: the 256-row kernel with ragged tails
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,e,fin,fout", DEPTH_CASES)
def test_linear_pipeline_depths(dtype, rows, e, fin, fout, device, tile):
    g = torch.Generator().manual_seed(rows * 7 + fin)
    counts = ragged_counts(rows, e, g, 0)
    x = torch.randn(rows, fin, generator=g).to(dtype)
    w = (torch.randn(e, fout, fin, generator=g) / fin ** 0.5).to(dtype)
    b = torch.randn(e, fout, generator=g).to(dtype)
    gy = torch.randn(rows, fout, generator=g).to(dtype)
    ref_y, ref_gx, ref_gw, ref_gb = _reference(x, counts, w, b, gy)
    xd, wd, bd, gyd = x.to(device), w.to(device), b.to(device), gy.to(device)
    tol = TOL[dtype]
    assert rel_err(fmoe_native.linear_forward(xd, counts, wd, bd), ref_y) <= tol
    gx, gw, gb = fmoe_native.linear_backward(gyd, xd, counts, wd, bd)
    assert rel_err(gx, ref_gx) <= tol
    assert rel_err(gw, ref_gw) <= tol
    assert rel_err(gb, ref_gb) <= tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_moelinear_autograd(dtype, device):
    g = torch.Generator().manual_seed(1)
    counts = torch.tensor([100, 0, 156, 44])
    x = torch.randn(300, 96, generator=g).to(dtype)
    w = (torch.randn(4, 160, 96, generator=g) / 10).to(dtype)
    b = torch.randn(4, 160, generator=g).to(dtype)
    gy = torch.randn(300, 160, generator=g).to(dtype)
    ref_y, ref_gx, ref_gw, ref_gb = _reference(x, counts, w, b, gy)
    xd = x.to(device).requires_grad_(True)
    wd = w.to(device).requires_grad_(True)
    bd = b.to(device).requires_grad_(True)
    y = MOELinear.apply(xd, counts, wd, bd)
    y.backward(gy.to(device))
    tol = TOL[dtype]
    assert rel_err(y, ref_y) <= tol and rel_err(xd.grad, ref_gx) <= tol
    assert rel_err(wd.grad, ref_gw) <= tol and rel_err(bd.grad, ref_gb) <= tol


def test_many_experts_split_into_several_launches(device):
    """More experts than one launch's segment table holds (256)."""
    g = torch.Generator().manual_seed(2)
    e, fin, fout = 600, 32, 48
    counts = torch.randint(0, 9, (e,), generator=g)
    rows = int(counts.sum())
    x = torch.randn(rows, fin, generator=g).bfloat16()
    w = (torch.randn(e, fout, fin, generator=g) / 6).bfloat16()
    gy = torch.randn(rows, fout, generator=g).bfloat16()
    ref_y, ref_gx, ref_gw, _ = _reference(x, counts, w, None, gy)
    y = fmoe_native.linear_forward(x.to(device), counts, w.to(device), None)
    gx, gw, gb = fmoe_native.linear_backward(gy.to(device), x.to(device), counts, w.to(device), None)
    assert rel_err(y, ref_y) <= 2e-2 and rel_err(gx, ref_gx) <= 2e-2 and rel_err(gw, ref_gw) <= 2e-2


def test_linearity_at_full_width(device):
    """config-4 feature sizes on a slice of its rows: f(a*x) = a*f(x) for a power of two
    (exact in bf16), and zero input rows give exactly the bias."""
    g = torch.Generator().manual_seed(3)
    e, d, h = 2, 4096, 14336
    counts = torch.tensor([700, 324])
    x = torch.randn(1024, d, generator=g).bfloat16().to(device)
    w = ((torch.rand(e, h, d, generator=g) * 2 - 1) * (d * h) ** -0.5).bfloat16().to(device)
    b = torch.randn(e, h, generator=g).bfloat16().to(device)
    y1 = fmoe_native.linear_forward(x, counts, w, None)
    y4 = fmoe_native.linear_forward(x * 4, counts, w, None)
    assert torch.equal(y4, y1 * 4)
    yb = fmoe_native.linear_forward(torch.zeros_like(x), counts, w, b)
    assert torch.equal(yb[:700], b[0].expand(700, h)) and torch.equal(yb[700:], b[1].expand(324, h))
    ref = (x[:700].double().cpu() @ w[0].double().cpu().t())
    assert rel_err(y1[:700], ref) <= 2e-2


@pytest.mark.parametrize("forced_tile", ["128x256", "256x256", "128x128"])
@pytest.mark.parametrize("fin,fout", [(14336, 4096), (4096, 14336)])
def test_full_depth_bf16_forward_backward(fin, fout, forced_tile, device, monkeypatch):
    """The Mixtral-like share's feature sizes at full contraction depth, both linears: bf16 forward,
    data-grad (contraction 4096 / 14336), weight-grad and bias-grad against the float64 oracle, on
    ragged segments that leave partial row tiles; normwise AND element by element (|d| <= tol |ref| +
    tol rms(ref)).  With 128 x 256 tiles both the forward and the data-grad launch fill less than half
    a round of the chip after their whole rounds, so they also run the contraction-split tail with its
    fp32 partial sums."""
    import ctypes
    from fastermoe_amd import _lib
    monkeypatch.setenv("FMOE_GEMM_TILE", forced_tile)
    g = torch.Generator().manual_seed(fin // 7)
    counts = torch.tensor([350, 0, 250])
    rows, e = 600, 3
    x = torch.randn(rows, fin, generator=g).bfloat16()
    w = (torch.randn(e, fout, fin, generator=g) / fin ** 0.5).bfloat16()
    b = torch.randn(e, fout, generator=g).bfloat16()
    gy = torch.randn(rows, fout, generator=g).bfloat16()
    # 128-row tiles: 3 + 2 row tiles; both products are split
    plan = (ctypes.c_int64 * 3)()
    for width, depth in ((fout, fin), (fin, fout)) if forced_tile == "128x256" else ():
        _lib.check(_lib.load().fmoe_gemm_tail_plan(5 * ((width + 255) // 256), (depth + 63) // 64, 256,
                                                  ctypes.cast(plan, ctypes.c_void_p)))
        assert plan[1] > 1
    ref_y, ref_gx, ref_gw, ref_gb = _reference(x, counts, w, b, gy)
    xd, wd, bd, gyd = x.to(device), w.to(device), b.to(device), gy.to(device)
    assert_close(fmoe_native.linear_forward(xd, counts, wd, bd), ref_y, 2e-2, "forward")
    gx, gw, gb = fmoe_native.linear_backward(gyd, xd, counts, wd, bd)
    assert_close(gx, ref_gx, 2e-2, "data-grad")
    assert_close(gw, ref_gw, 2e-2, "weight-grad")
    assert_close(gb, ref_gb, 2e-2, "bias-grad")
    assert torch.count_nonzero(gw[1]) == 0 and torch.count_nonzero(gb[1]) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_contraction_split_tail_matches_oracle(dtype, device, monkeypatch):
    """A launch of (2 + 1) x 20 row/column tiles (128 x 256) whose contraction (80 slabs of bf16, 160
    of fp32) is split into parts: forward with bias and data-grad, with a ragged contraction tail."""
    monkeypatch.setenv("FMOE_GEMM_TILE", "128x256")
    g = torch.Generator().manual_seed(23)
    counts = torch.tensor([200, 100])
    fin, fout = 5120 - 8, 5120 - 24
    x = torch.randn(300, fin, generator=g).to(dtype)
    w = (torch.randn(2, fout, fin, generator=g) / fin ** 0.5).to(dtype)
    b = torch.randn(2, fout, generator=g).to(dtype)
    gy = torch.randn(300, fout, generator=g).to(dtype)
    ref_y, ref_gx, ref_gw, ref_gb = _reference(x, counts, w, b, gy)
    xd, wd, bd, gyd = x.to(device), w.to(device), b.to(device), gy.to(device)
    tol = TOL[dtype]
    assert_close(fmoe_native.linear_forward(xd, counts, wd, bd), ref_y, tol, "forward")
    gx, gw, gb = fmoe_native.linear_backward(gyd, xd, counts, wd, bd)
    assert_close(gx, ref_gx, tol, "data-grad")
    assert_close(gw, ref_gw, tol, "weight-grad")
    # twice the same call: the partial sums are added in a fixed order, so the result is reproducible
    assert torch.equal(fmoe_native.linear_forward(xd, counts, wd, bd), fmoe_native.linear_forward(xd, counts, wd, bd))


def test_validation_errors(device):
    x = torch.zeros(4, 8, device=device)
    w = torch.zeros(2, 8, 8, device=device)
    with pytest.raises(ValueError, match="CPU"):
        fmoe_native.linear_forward(x, torch.tensor([2, 2], device=device), w, None)
    with pytest.raises(ValueError, match="sums to"):
        fmoe_native.linear_forward(x, torch.tensor([2, 3]), w, None)
    with pytest.raises(TypeError):
        fmoe_native.linear_forward(x, torch.tensor([2, 2]), w.half(), None)
    with pytest.raises(ValueError, match="features"):
        fmoe_native.linear_forward(torch.zeros(4, 6, device=device), torch.tensor([2, 2]), w, None)


@pytest.mark.parametrize("d,h,count_list,forced_tile", [
    (128, 256, [100, 0, 333, 79], None),          # small tiles, no split
    (5120, 5120, [200, 100], "128x256"),          # every forward / data-grad launch ends in a split tail
])
def test_expert_mlp_launches_replay_from_a_hip_graph(d, h, count_list, forced_tile, device, monkeypatch):
    """The GEMM entry points neither synchronise nor allocate nor clear memory with a memset once their split
    workspace exists, so a launch-bound sequence (the six products of a small expert MLP) can be captured
    into a HIP graph: three replays with new inputs, eager work and synchronisations between them, each
    compared with the eager result of the same inputs."""
    from fastermoe_amd import _lib as lib
    if forced_tile:
        monkeypatch.setenv("FMOE_GEMM_TILE", forced_tile)
    g = torch.Generator().manual_seed(11)
    counts = torch.tensor(count_list)
    e, rows = len(count_list), int(counts.sum())
    w1 = (torch.randn(e, h, d, generator=g) / d ** 0.5).bfloat16().to(device)
    b1 = torch.randn(e, h, generator=g).bfloat16().to(device)
    w2 = (torch.randn(e, d, h, generator=g) / h ** 0.5).bfloat16().to(device)
    x = torch.randn(rows, d, generator=g).bfloat16().to(device)
    gy = torch.randn(rows, d, generator=g).bfloat16().to(device)

    def sequence(x, gy):
        mid, pre = fmoe_native.linear_act_forward(x, counts, w1, b1, lib.ACT_GELU, True)
        y = fmoe_native.linear_forward(mid, counts, w2, None)
        g_pre = fmoe_native.linear_dact_backward(gy, counts, w2, pre, lib.ACT_GELU)
        gw2, _ = fmoe_native.linear_weight_backward(gy, mid, counts, w2, None)
        gx, gw1, gb1 = fmoe_native.linear_backward(g_pre, x, counts, w1, b1)
        return y, gx, gw1, gb1, gw2

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):           # warm-up on the capture stream (its split workspace gets allocated)
        sequence(x, gy)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    xs, gys = x.clone(), gy.clone()
    with torch.cuda.graph(graph, stream=side):
        captured = sequence(xs, gys)
    for step in range(3):
        xn = torch.randn(rows, d, generator=g).bfloat16().to(device)
        gn = torch.randn(rows, d, generator=g).bfloat16().to(device)
        want = sequence(xn, gn)              # eager, between the replays
        torch.cuda.synchronize()
        xs.copy_(xn)
        gys.copy_(gn)
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip(captured, want):
            assert torch.equal(got, ref), f"replay {step} differs from the eager result"


def test_rows_past_the_counted_ones_are_left_alone(device):
    """A buffer with one row per slot of which only the first sum(counts) are routed (the layer's sorted
    buffers when slots were dropped): the linears read and write the counted rows only."""
    g = torch.Generator().manual_seed(5)
    counts = torch.tensor([70, 0, 130])
    rows, pad, fin, fout = 200, 57, 64, 96
    x = torch.randn(rows + pad, fin, generator=g).bfloat16()
    x[rows:] = float("nan")                       # must never be read
    w = (torch.randn(3, fout, fin, generator=g) / 8).bfloat16()
    b = torch.randn(3, fout, generator=g).bfloat16()
    gy = torch.randn(rows + pad, fout, generator=g).bfloat16()
    gy[rows:] = float("nan")
    ref_y, ref_gx, ref_gw, ref_gb = _reference(x[:rows], counts, w, b, gy[:rows])
    xd, wd, bd, gyd = x.to(device), w.to(device), b.to(device), gy.to(device)
    y = fmoe_native.linear_forward(xd, counts, wd, bd)
    assert y.shape[0] == rows + pad and rel_err(y[:rows], ref_y) <= 2e-2
    gx, gw, gb = fmoe_native.linear_backward(gyd, xd, counts, wd, bd)
    assert rel_err(gx[:rows], ref_gx) <= 2e-2 and rel_err(gw, ref_gw) <= 2e-2 and rel_err(gb, ref_gb) <= 2e-2
    assert torch.isfinite(gw).all() and torch.isfinite(gb).all()
