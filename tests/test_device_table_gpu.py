"""GPU parity of the segment table built on the device and of the grouped GEMMs launched over it
(no expert counts on the host).

The table is integer work: bit-exact against oracle.routing.segment_table.  The products over the
table run the same kernels as the host-count entry points, so with the tile shape forced they must
equal them bit for bit; beside that they are held to the float64 oracle like every other product
(1e-5 for float32, 2e-2 for bfloat16 / float16, relative to the largest reference magnitude)."""
import numpy as np
import pytest
import torch

from fastermoe_amd import _lib, fmoe_native
from oracle import moe as omoe
from oracle import routing as orouting
from helpers import TOL, ragged_counts, rel_err, zipf_experts

pytestmark = pytest.mark.gpu

HEADER = 8


def _unpack(table, n_expert):
    """The parts of the device table that the kernels read, as numpy arrays."""
    t = table.cpu().numpy()
    seg = t[HEADER:HEADER + n_expert + 1]
    n256, n128, off256, off128 = int(t[2]), int(t[3]), int(t[4]), int(t[5])
    assert off256 % 4 == 0 and off128 % 4 == 0
    return {"n_expert": int(t[0]), "rows": int(t[1]), "seg": seg,
            "tiles256": t[off256:off256 + 4 * n256].reshape(-1, 4),
            "tiles128": t[off128:off128 + 4 * n128].reshape(-1, 4)}


def _check_table(counts, rows_cap, device):
    counts = torch.as_tensor(counts, dtype=torch.int64)
    got = _unpack(fmoe_native.segment_table(counts.to(device), rows_cap), counts.numel())
    ref = orouting.segment_table(counts.numpy(), rows_cap)
    assert got["n_expert"] == counts.numel()
    assert got["rows"] == int(ref["seg"][-1])
    assert np.array_equal(got["seg"], ref["seg"])
    for key in ("tiles256", "tiles128"):
        assert np.array_equal(got[key][:, :3], ref[key]), key
        assert not got[key][:, 3].any()


CONFIG_COUNTS = {
    "config1": lambda g: torch.bincount(torch.randint(0, 8, (8192,), generator=g), minlength=8),
    "config2": lambda g: torch.bincount(torch.randint(0, 16, (32768,), generator=g), minlength=16).clamp(max=2458),
    "config3": lambda g: torch.bincount(zipf_experts(16384, 64, 1.2, g), minlength=64),
    "config4": lambda g: torch.bincount(torch.randint(0, 8, (65536,), generator=g), minlength=8),
    "config5": lambda g: torch.bincount(torch.randint(0, 256, (65536,), generator=g), minlength=256),
}
CONFIG_SLOTS = {"config1": 8192, "config2": 32768, "config3": 16384, "config4": 65536, "config5": 65536}


@pytest.mark.parametrize("name", sorted(CONFIG_COUNTS))
def test_segment_table_at_the_configurations(name, device):
    g = torch.Generator().manual_seed(11)
    _check_table(CONFIG_COUNTS[name](g), CONFIG_SLOTS[name], device)


@pytest.mark.parametrize("counts,cap", [
    ([0, 0, 0, 0], 64),                 # nothing routed at all
    ([0, 0, 0, 0], 0),                  # no slots at all
    ([5000], 5000),                     # a single expert owns every row
    ([0, 1, 0, 255, 256, 257, 0], 769), # tile edges
    ([128] * 7, 896),                   # every expert exactly one 128-row tile
    ([300, 300, 300], 700),             # counts beyond rows_cap are clamped in order
    ([-4, 10, 2 ** 40, 7], 100),        # garbage counts never overrun the tile maps
])
def test_segment_table_edge_cases(counts, cap, device):
    _check_table(counts, cap, device)


@pytest.mark.parametrize("n_expert", [1023, 1024, 1025, 4100, 8192])
def test_segment_table_many_experts(n_expert, device):
    """More experts than the kernel's 1024 threads: several passes with carried sums."""
    g = torch.Generator().manual_seed(n_expert)
    counts = torch.randint(0, 40, (n_expert,), generator=g)
    counts[torch.randperm(n_expert, generator=g)[: n_expert // 3]] = 0
    counts[n_expert // 2] = 700
    _check_table(counts, int(counts.sum()) + 17, device)


def test_segment_table_argument_checks(device):
    cnt = torch.zeros(4, dtype=torch.int64, device=device)
    small = torch.empty(4, dtype=torch.int32, device=device)
    lib = _lib.load()
    rc = lib.fmoe_segment_table_build(cnt.data_ptr(), 4, 1000, small.data_ptr(), small.numel() * 4, None)
    assert rc == -4 and b"needs" in lib.fmoe_last_error()
    assert lib.fmoe_segment_table_build(None, 4, 1000, small.data_ptr(), 1 << 20, None) == -1
    assert lib.fmoe_segment_table_bytes(-1, 4) == 0 and lib.fmoe_segment_table_bytes(10, 0) == 0
    assert lib.fmoe_linear_dev_supported(64, 128, _lib.BF16) == 1
    assert lib.fmoe_linear_dev_supported(12, 20, _lib.BF16) == 0     # rows that are not whole 16-byte chunks
    assert lib.fmoe_linear_dev_supported(64, 128, _lib.F64) == 0


TILES = ["256x256", "128x256", "128x128"]
DEV_CASES = [  # rows, slots (rows_cap), experts, in, out, empties
    (1000, 1000, 4, 64, 128, 1),
    (777, 900, 8, 256, 72, 2),        # fewer rows than slots (dropped slots): rows past the routed ones untouched
    (2048, 2048, 2, 512, 512, 0),
    (300, 300, 16, 40, 24, 5),
    (5, 64, 3, 8, 8, 1),
    (0, 32, 3, 16, 16, 3),            # no rows at all
    (1100, 1100, 2, 328, 272, 0),
    (3000, 3000, 300, 64, 96, 40),    # more experts than a host-count launch carries in its arguments
]


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,slots,e,fin,fout,empties", DEV_CASES)
def test_products_over_the_device_table(dtype, rows, slots, e, fin, fout, empties, tile, device, monkeypatch):
    monkeypatch.setenv("FMOE_GEMM_TILE", tile)
    g = torch.Generator().manual_seed(rows + e + fin)
    counts = ragged_counts(rows, e, g, empties) if rows else torch.zeros(e, dtype=torch.int64)
    x = torch.randn(slots, fin, generator=g).to(dtype)
    w = (torch.randn(e, fout, fin, generator=g) / fin ** 0.5).to(dtype)
    b = torch.randn(e, fout, generator=g).to(dtype)
    gy = torch.randn(slots, fout, generator=g).to(dtype)
    xd, wd, bd, gyd = x.to(device), w.to(device), b.to(device), gy.to(device)
    table = fmoe_native.segment_table(counts.to(device), slots)

    # against the host-count entry points (same kernels, same tile shape): bit for bit on the routed rows
    y, pre = fmoe_native.linear_forward_dev(xd, wd, bd, table, slots)
    assert pre is None and y.shape == (slots, fout)
    y_host = fmoe_native.linear_forward(xd, counts, wd, bd)
    assert torch.equal(y[:rows], y_host[:rows])
    gx = fmoe_native.linear_dgrad_dev(gyd, wd, table, slots)
    gw, gb = fmoe_native.linear_wgrad_dev(gyd, xd, wd, table, slots, True)
    gx_host, gw_host, gb_host = fmoe_native.linear_backward(gyd, xd, counts, wd, bd)
    assert torch.equal(gx[:rows], gx_host[:rows])
    assert torch.equal(gw, gw_host) and torch.equal(gb, gb_host)

    # against the float64 oracle
    x64, w64, b64 = x[:rows].double().requires_grad_(True), w.double().requires_grad_(True), b.double().requires_grad_(True)
    ref = omoe.per_expert_linear(x64, counts, w64, b64)
    ref.backward(gy[:rows].double())
    tol = TOL[dtype]
    assert rel_err(y[:rows], ref) <= tol
    assert rel_err(gx[:rows], x64.grad) <= tol
    assert rel_err(gw, w64.grad) <= tol and rel_err(gb, b64.grad) <= tol
    for ex in range(e):
        if counts[ex] == 0:
            assert torch.count_nonzero(gw[ex]) == 0 and torch.count_nonzero(gb[ex]) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("act", ["gelu", "relu", "none"])
def test_activation_epilogues_over_the_device_table(dtype, act, device):
    """bias + activation in the forward epilogue (with the pre-activation kept) and x act' in the data
    gradient's, rows gathered through an index in the loader: equal to the host-count entry points
    on the scattered copy, bit for bit."""
    code = {"gelu": _lib.ACT_GELU, "relu": _lib.ACT_RELU, "none": _lib.ACT_NONE}[act]
    g = torch.Generator().manual_seed(5)
    n_tokens, k, e, d, h = 700, 2, 6, 64, 192
    gate = torch.randint(-1, e, (n_tokens, k), generator=g).to(device)
    counts, pos_buf, s2r = fmoe_native.route(gate, e)
    slots = n_tokens * k
    rows = int(counts.sum())
    table = fmoe_native.segment_table(counts, slots)
    inp = torch.randn(n_tokens, d, generator=g).to(dtype).to(device)
    w = (torch.randn(e, h, d, generator=g) / d ** 0.5).to(dtype).to(device)
    b = torch.randn(e, h, generator=g).to(dtype).to(device)
    y, pre = fmoe_native.linear_forward_dev(inp, w, b, table, slots, code, True, row_index=pos_buf, index_div=k)
    scattered = fmoe_native.gather_rows(inp, pos_buf[:rows], index_div=k)
    y_host, pre_host = fmoe_native.linear_act_forward(scattered, counts.cpu(), w, b, code, True)
    assert torch.equal(y[:rows], y_host) and torch.equal(pre[:rows], pre_host)
    # data gradient of a following linear [e, d, h] with the derivative in the epilogue
    w2 = (torch.randn(e, d, h, generator=g) / h ** 0.5).to(dtype).to(device)
    gy = torch.randn(slots, d, generator=g).to(dtype).to(device)
    gx = fmoe_native.linear_dgrad_dev(gy, w2, table, slots, pre, code)
    gx_host = fmoe_native.linear_dact_backward(gy[:rows].contiguous(), counts.cpu(), w2, pre_host, code)
    assert torch.equal(gx[:rows], gx_host)


def test_unsupported_shapes_are_refused(device):
    counts = torch.tensor([3, 5], dtype=torch.int64, device=device)
    table = fmoe_native.segment_table(counts, 8)
    x = torch.randn(8, 10, device=device)        # rows of 40 bytes: not whole 16-byte chunks
    w = torch.randn(2, 20, 10, device=device)
    with pytest.raises(_lib.FmoeHipError):
        fmoe_native.linear_forward_dev(x, w, None, table, 8)
    with pytest.raises(ValueError):
        fmoe_native.linear_forward_dev(x[:4].contiguous(), w, None, table, 8)   # fewer rows than rows_cap
    with pytest.raises(ValueError):
        fmoe_native.linear_forward_dev(x, w, None, table[:10].contiguous(), 8)  # table too short


@pytest.mark.parametrize("tile", ["256x256", "128x256"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,slots,e,fin,fout", [
    (600, 700, 2, 4096, 520),     # forward: a short last round of deep tiles -> split along the contraction
    (600, 600, 3, 520, 4096),     # data gradient: the same
    (70000, 70000, 4, 3584, 264), # more than one round of tiles before the split tail
])
def test_split_tail_over_the_device_table(dtype, rows, slots, e, fin, fout, tile, device, monkeypatch):
    """A last, partial round of tiles is split along the contraction by the workgroups themselves when the
    segments come from a device table (the host does not know the tile count): same plan, same order of
    the partial sums and so the same bits as the host-count launch, with and without the caller's workspace
    (FMOE_DEV_SPLIT=0: no workspace, no split -- another order of the sums, equal within the tolerance)."""
    monkeypatch.setenv("FMOE_GEMM_TILE", tile)
    g = torch.Generator().manual_seed(rows + fin)
    counts = ragged_counts(rows, e, g, 0)
    x = torch.randn(slots, fin, generator=g).to(dtype).to(device)
    w = (torch.randn(e, fout, fin, generator=g) / fin ** 0.5).to(dtype).to(device)
    b = torch.randn(e, fout, generator=g).to(dtype).to(device)
    gy = torch.randn(slots, fout, generator=g).to(dtype).to(device)
    table = fmoe_native.segment_table(counts.to(device), slots)
    y_host = fmoe_native.linear_forward(x, counts, w, b)
    gx_host = fmoe_native.linear_backward(gy, x, counts, w, b)[0]
    for flag in ("1", "0"):
        monkeypatch.setenv("FMOE_DEV_SPLIT", flag)
        y, _ = fmoe_native.linear_forward_dev(x, w, b, table, slots)
        gx = fmoe_native.linear_dgrad_dev(gy, w, table, slots)
        if flag == "1":
            assert torch.equal(y[:rows], y_host[:rows]) and torch.equal(gx[:rows], gx_host[:rows])
        else:
            assert rel_err(y[:rows], y_host[:rows]) <= TOL[dtype] and rel_err(gx[:rows], gx_host[:rows]) <= TOL[dtype]
