"""``fmoe_route_static`` -- the routing entry point that allocates nothing (its scratch is a
fixed array inside the library) -- against ``fmoe_route`` with a caller's workspace: counts,
positions and the slot -> row map must be bit-identical, on two calls in a row that share the
array, the second on a smaller input, and sizes beyond the array must be refused."""
import ctypes

import pytest
import torch

from fastermoe_amd import _lib

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 1 << 20  # FMOE_ROUTE_STATIC_SCRATCH_BYTES of include/fmoe_hip.h


def _vp(t):
    return ctypes.c_void_p(t.data_ptr())


def _route_both(gate, n_expert):
    lib = _lib.load()
    dev = gate.device
    n = gate.numel()
    st = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    outs = []
    for static in (False, True):
        cnt = torch.full((n_expert,), -7, dtype=torch.int64, device=dev)
        pos = torch.full((n,), -7, dtype=torch.int64, device=dev)
        s2r = torch.full((n,), -7, dtype=torch.int64, device=dev)
        if static:
            _lib.check(lib.fmoe_route_static(_vp(gate), n, n_expert, _vp(cnt), _vp(pos), _vp(s2r), st))
        else:
            ws = torch.empty(lib.fmoe_routing_workspace_bytes(n, n_expert), dtype=torch.uint8, device=dev)
            _lib.check(lib.fmoe_route(_vp(gate), n, n_expert, _vp(cnt), _vp(pos), _vp(s2r), _vp(ws), ws.numel(), st))
        torch.cuda.synchronize()
        outs.append((cnt.cpu(), pos.cpu(), s2r.cpu()))
    return outs


def test_route_static_matches_route_on_consecutive_calls(device):
    gen = torch.Generator().manual_seed(11)
    # the first call fills more of the shared array than the second one uses
    for n, k, e in ((8192, 8, 256), (1500, 2, 16), (37, 1, 3)):
        gate = torch.randint(-1, e, (n, k), generator=gen).to(device)
        (cnt_a, pos_a, s2r_a), (cnt_b, pos_b, s2r_b) = _route_both(gate, e)
        total = int(cnt_a.sum())
        assert total == int((gate >= 0).sum())
        assert torch.equal(cnt_a, cnt_b), (n, k, e)
        assert torch.equal(pos_a, pos_b), (n, k, e)
        assert torch.equal(pos_b[total:], torch.full_like(pos_b[total:], -1)), "entries past the routed slots must be -1"
        assert torch.equal(s2r_a, s2r_b), (n, k, e)


def test_route_static_empty_input(device):
    lib = _lib.load()
    cnt = torch.full((5,), 3, dtype=torch.int64, device=device)
    st = ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    _lib.check(lib.fmoe_route_static(None, 0, 5, _vp(cnt), None, None, st))
    assert cnt.cpu().tolist() == [0] * 5


def test_route_static_rejects_sizes_beyond_its_array(device):
    lib = _lib.load()
    n, e = 1 << 21, 4096
    assert lib.fmoe_routing_workspace_bytes(n, e) > SCRATCH_BYTES
    cnt = torch.zeros(e, dtype=torch.int64, device=device)
    dummy = torch.zeros(8, dtype=torch.int64, device=device)  # never dereferenced: the size check comes first
    rc = lib.fmoe_route_static(_vp(dummy), n, e, _vp(cnt), _vp(dummy), None, None)
    assert rc == -2  # FMOE_ELIMIT
    assert b"fmoe_route_static" in lib.fmoe_last_error()


def test_route_static_allocates_no_device_memory(device):
    """Free device memory, as the driver reports it, is the same before and after calls of
    fmoe_route_static on buffers that exist already -- and the call can be captured into a HIP graph,
    which an allocating call could not be."""
    lib = _lib.load()
    gen = torch.Generator().manual_seed(3)
    n, k, e = 4096, 2, 32
    gate = torch.randint(-1, e, (n, k), generator=gen).to(device)
    cnt = torch.empty(e, dtype=torch.int64, device=device)
    pos = torch.empty(n * k, dtype=torch.int64, device=device)
    s2r = torch.empty(n * k, dtype=torch.int64, device=device)
    st = ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    _lib.check(lib.fmoe_route_static(_vp(gate), n * k, e, _vp(cnt), _vp(pos), _vp(s2r), st))   # first call: symbol lookup
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(device)
    for _ in range(5):
        _lib.check(lib.fmoe_route_static(_vp(gate), n * k, e, _vp(cnt), _vp(pos), _vp(s2r), st))
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(device)
    assert free_after == free_before
    want = (cnt.clone(), pos.clone(), s2r.clone())
    # under capture (no allocation is allowed there), replayed on another gate tensor's contents
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cap = ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
        _lib.check(lib.fmoe_route_static(_vp(gate), n * k, e, _vp(cnt), _vp(pos), _vp(s2r), cap))
    for rep in range(3):
        cnt.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(cnt, want[0]) and torch.equal(pos, want[1]) and torch.equal(s2r, want[2]), rep
