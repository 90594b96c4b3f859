"""Routing / capacity oracle: ctypes front-end of ``routing_oracle.c``.

TEST INFRASTRUCTURE ONLY (see the package docstring).  Each function mirrors one
entry point of the reference's extension module (cuda/fmoe_cuda.cpp:105-130) and
follows the sequential execution of the kernel it names.  The ``*_py`` variants
are the same loops in pure Python, meant for tiny inputs where the loop can be
followed by hand.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librouting_oracle.so")
_lib = None

_i64p = ctypes.POINTER(ctypes.c_int64)
_i32p = ctypes.POINTER(ctypes.c_int32)


def build(force=False):
    """Compile ``routing_oracle.c`` with gcc (a second or so)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "librouting_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_LIB_PATH)
        lib.oracle_expert_count.argtypes = [_i64p, _i32p, ctypes.c_int64, ctypes.c_int64]
        lib.oracle_assign_pos.argtypes = [_i32p, _i64p, _i64p, ctypes.c_int64]
        lib.oracle_limit_by_capacity.argtypes = [_i64p, _i32p, _i64p, ctypes.c_int64, ctypes.c_int64]
        lib.oracle_prune_gate_by_capacity.argtypes = [_i64p, _i64p, _i32p, ctypes.c_int64]
        for f in (lib.oracle_expert_count, lib.oracle_assign_pos,
                  lib.oracle_limit_by_capacity, lib.oracle_prune_gate_by_capacity):
            f.restype = None
        _lib = lib
    return _lib


def _p64(a):
    return a.ctypes.data_as(_i64p)


def _p32(a):
    return a.ctypes.data_as(_i32p)


def expert_count(gate_idx, n_expert, expert_count=None):
    """fmoe_cuda.expert_count (cuda/local_exchange.cu:22-32): adds the histogram
    of ``gate_idx`` (any shape, -1 skipped) into an int32 ``[n_expert]`` array."""
    g = np.ascontiguousarray(np.asarray(gate_idx, dtype=np.int64).reshape(-1))
    if expert_count is None:
        expert_count = np.zeros(n_expert, dtype=np.int32)
    assert expert_count.dtype == np.int32 and expert_count.flags.c_contiguous
    _load().oracle_expert_count(_p64(g), _p32(expert_count), g.size, n_expert)
    return expert_count


def assign_pos(cum_count, gate):
    """fmoe_cuda.assign_pos (cuda/local_exchange.cu:5-20).  ``cum_count`` is the
    int32 inclusive cumsum of the counts and is consumed (left as the exclusive
    cumsum).  Returns ``pos`` int64 ``[cum_count[-1]]``."""
    g = np.ascontiguousarray(np.asarray(gate, dtype=np.int64).reshape(-1))
    assert cum_count.dtype == np.int32 and cum_count.flags.c_contiguous
    total = int(cum_count[-1]) if cum_count.size else 0
    pos = np.full(total, -1, dtype=np.int64)
    _load().oracle_assign_pos(_p32(cum_count), _p64(g), _p64(pos), g.size)
    return pos


def count_by_gate(gate, n_expert):
    """fmoe/functions.py:19-42 at world_size 1: (pos, local_expert_count)."""
    cnt = expert_count(gate, n_expert).astype(np.int64)
    cum = np.cumsum(cnt).astype(np.int32)
    return assign_pos(cum, gate), cnt


def limit_by_capacity(expert_count_, capacity, n_expert, n_worker):
    """fmoe_cuda.limit_by_capacity (cuda/balancing.cu:7-20): int64 ``[W*E]``
    counts, int32 ``[E]`` capacity (consumed) -> granted int64 ``[W*E]``."""
    ec = np.ascontiguousarray(np.asarray(expert_count_, dtype=np.int64).reshape(-1))
    assert ec.size == n_expert * n_worker
    assert capacity.dtype == np.int32 and capacity.flags.c_contiguous
    eca = np.zeros_like(ec)
    _load().oracle_limit_by_capacity(_p64(ec), _p32(capacity), _p64(eca), n_expert, n_worker)
    return eca


def prune_gate_by_capacity(gate_idx, expert_count_):
    """fmoe_cuda.prune_gate_by_capacity (cuda/balancing.cu:22-37): returns a new
    index array of the same shape; ``expert_count_`` int32 is consumed."""
    g = np.ascontiguousarray(np.asarray(gate_idx, dtype=np.int64))
    assert expert_count_.dtype == np.int32 and expert_count_.flags.c_contiguous
    out = np.empty_like(g)
    _load().oracle_prune_gate_by_capacity(_p64(g.reshape(-1)), _p64(out.reshape(-1)),
                                          _p32(expert_count_), g.size)
    return out


def limit_and_prune(topk_idx, n_expert, capacity):
    """fmoe/gates/utils.py:9-26 at world_size 1: (new_lec, new_gec, pruned_idx).
    ``capacity`` is the per-expert cap (a scalar, broadcast to all experts)."""
    cap = np.full(n_expert, capacity, dtype=np.int32)
    gec = expert_count(topk_idx, n_expert).astype(np.int64)
    new_gec = limit_by_capacity(gec, cap, n_expert, 1)
    new_lec = new_gec
    pruned = prune_gate_by_capacity(topk_idx, new_lec.astype(np.int32))
    return new_lec, new_gec, pruned


def segment_table(counts, rows_cap):
    """The row segments the per-expert GEMMs walk, restated from the host loops of
    cuda/parallel_linear.cuh:69-88 and :113-155 (``ptr += expert_count[i]`` per expert): expert ``e``
    owns the expert-sorted rows ``[seg[e], seg[e+1])``.  Beside them, for row tiles of 256 and of
    128 rows counted from each expert's own first row, the list of ``(expert, first row, rows)``
    per tile in expert order.  Counts are taken in order and clamped so that they never add up
    to more than ``rows_cap`` (a negative count reads as 0).  One plain sequential walk."""
    seg = [0]
    tiles = {256: [], 128: []}
    for e, c in enumerate(np.asarray(counts).reshape(-1).tolist()):
        c = min(max(int(c), 0), rows_cap - seg[-1])
        first = seg[-1]
        for block in (256, 128):
            r = 0
            while r < c:
                tiles[block].append((e, first + r, min(block, c - r)))
                r += block
        seg.append(first + c)
    return {"seg": np.array(seg, dtype=np.int32),
            "tiles256": np.array(tiles[256], dtype=np.int32).reshape(-1, 3),
            "tiles128": np.array(tiles[128], dtype=np.int32).reshape(-1, 3)}


# ---- pure-Python loops, tiny inputs only -----------------------------------

def assign_pos_py(counts, gate):
    """Same sequential loop as ``oracle_assign_pos`` on Python lists."""
    cum = []
    s = 0
    for c in counts:
        s += int(c)
        cum.append(s)
    pos = [-1] * s
    for idx, g in enumerate(list(gate)):
        if g > -1:
            p = cum[g]
            cum[g] = p - 1
            pos[p - 1] = idx
    return pos, cum


def prune_py(gate, cap):
    cap = [int(c) for c in cap]
    out = []
    for g in list(gate):
        if g < 0:
            out.append(-1)
            continue
        old = cap[g]
        cap[g] = old - 1
        out.append(-1 if old <= 0 else g)
    return out, cap
