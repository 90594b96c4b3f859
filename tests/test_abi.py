"""CPU-side checks of the drop-in boundary: the shared library loads and exports
every symbol include/fmoe_hip.h declares, the Python API has the reference's
names and signatures, and bad arguments raise instead of reaching a kernel."""
import inspect
import os
import re

import pytest
import torch

import fastermoe_amd
from fastermoe_amd import _lib, fmoe_native, functions, fused_functions, gates, layers, transformer

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "fmoe_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fmoe_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 15
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in fmoe_hip.h but not exported"
    assert set(declared) == set(_lib.SIGNATURES), "ctypes table and header disagree"
    assert lib.fmoe_abi_version() == 3


def test_ctypes_signatures_match_the_header():
    """Every prototype in include/fmoe_hip.h against the ctypes table: same number of parameters,
    pointers where the header has pointers, 64-bit integers where it has int64_t, int where it has
    int -- a mismatch would silently corrupt the arguments of a call."""
    import ctypes
    text = open(os.path.join(ROOT, "include", "fmoe_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    protos = re.findall(r"\b([a-z0-9_ ]+?[ \*])(fmoe_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text)
    assert len(protos) == len(_lib.SIGNATURES)
    for ret, name, params in protos:
        restype, argtypes = _lib.SIGNATURES[name]
        params = [q.strip() for q in params.split(",") if q.strip() and q.strip() != "void"]
        assert len(params) == len(argtypes), f"{name}: header has {len(params)} parameters, ctypes table {len(argtypes)}"
        for q, a in zip(params, argtypes):
            if "*" in q:
                assert a is ctypes.c_void_p or issubclass(a, ctypes._Pointer), f"{name}: `{q}` is a pointer"
            elif q.startswith("int64_t"):
                assert a is ctypes.c_int64, f"{name}: `{q}` is int64_t"
            elif q.startswith("double"):
                assert a is ctypes.c_double, f"{name}: `{q}` is double"
            else:
                assert q.startswith("int ") and a is ctypes.c_int, f"{name}: `{q}`"
        if "*" in ret:
            assert restype in (ctypes.c_char_p, ctypes.c_void_p)
        elif "int64_t" in ret:
            assert restype is ctypes.c_int64
        else:
            assert restype is ctypes.c_int


def test_workspace_queries_run_without_a_gpu():
    lib = _lib.load()
    assert lib.fmoe_routing_workspace_bytes(65536, 256) >= (32 * 256 + 512) * 4
    assert lib.fmoe_index_add_workspace_bytes(100, 50) >= 600
    assert lib.fmoe_routing_workspace_bytes(-1, 4) == 0


def test_python_api_names_and_signatures():
    assert {"FMoE", "FMoELinear", "FMoETransformerMLP", "DistributedGroupedDataParallel"} <= set(dir(fastermoe_amd))
    for name in ("count_by_gate", "prepare_forward", "MOEScatter", "MOELinear", "MOEGather", "MOECache",
                 "ensure_comm", "AllGather", "Slice", "_local_scatter", "_local_gather"):
        assert hasattr(functions, name)
    assert hasattr(fused_functions, "MOEForward")
    for name in ("NaiveGate", "GShardGate", "SwitchGate", "ZeroGate", "NoisyGate"):
        assert hasattr(gates, name)
    for name in ("expert_count", "assign_pos", "linear_forward", "linear_backward", "limit_by_capacity",
                 "prune_gate_by_capacity", "fused_forward", "fused_backward"):
        assert hasattr(fmoe_native, name)
    # constructor signatures of fmoe/layers.py:169-184 and fmoe/transformer.py:96-112
    p = inspect.signature(layers.FMoE.__init__).parameters
    assert list(p)[1:] == ["num_expert", "d_model", "world_size", "mp_group", "moe_group", "top_k", "gate",
                           "expert", "gate_hook", "policy_fn", "mask", "mask_dict", "enable_fuse"]
    assert p["num_expert"].default == 32 and p["top_k"].default == 2 and p["d_model"].default == 1024
    p = inspect.signature(transformer.FMoETransformerMLP.__init__).parameters
    assert list(p)[1:] == ["num_expert", "d_model", "d_hidden", "world_size", "mp_group", "moe_group",
                           "activation", "gate", "top_k", "expert_dp_comm", "gate_hook", "bias", "mask",
                           "mask_dict"]
    assert p["d_hidden"].default == 4096 and p["bias"].default is True
    p = inspect.signature(functions.count_by_gate).parameters
    assert list(p) == ["gate", "num_expert", "world_size", "require_pos"]


def test_module_structure_and_parameter_names():
    m = fastermoe_amd.FMoETransformerMLP(num_expert=4, d_model=16, d_hidden=32, top_k=2)
    names = set(dict(m.named_parameters()))
    assert names == {"gate.gate.weight", "gate.gate.bias", "experts.htoh4.weight", "experts.htoh4.bias",
                     "experts.h4toh.weight", "experts.h4toh.bias"}
    assert tuple(m.experts.htoh4.weight.shape) == (4, 32, 16)
    assert tuple(m.experts.h4toh.weight.shape) == (4, 16, 32)
    assert torch.count_nonzero(m.experts.htoh4.bias) == 0
    # Kaiming-uniform over the 3-D tensor: bound 1/sqrt(out*in) (torch's fan_in for 3-D)
    bound = (32 * 16) ** -0.5
    assert m.experts.htoh4.weight.abs().max() <= bound
    assert getattr(m.experts.htoh4.weight, "dp_comm") == "none"
    assert getattr(m.gate.gate.weight, "dp_comm") == "moe"
    nobias = fastermoe_amd.FMoETransformerMLP(num_expert=2, d_model=8, d_hidden=8, bias=False)
    assert nobias.experts.htoh4.bias is None


def test_multi_worker_is_refused():
    with pytest.raises(NotImplementedError):
        fastermoe_amd.FMoE(num_expert=2, d_model=8, world_size=2)
    with pytest.raises(NotImplementedError):
        functions.count_by_gate(torch.zeros(4, dtype=torch.int64), 2, 2)
    with pytest.raises(NotImplementedError):
        fastermoe_amd.DistributedGroupedDataParallel(torch.nn.Linear(2, 2))


def test_cpu_tensors_are_rejected_not_computed():
    g = torch.zeros(8, dtype=torch.int64)
    with pytest.raises(ValueError, match="CUDA"):
        fmoe_native.expert_count(g, torch.zeros(2, dtype=torch.int32))
    with pytest.raises(ValueError, match="CUDA"):
        fmoe_native.linear_forward(torch.zeros(4, 8), torch.tensor([4]), torch.zeros(1, 8, 8), None)
    with pytest.raises(ValueError, match="CUDA"):
        fmoe_native.gather_rows(torch.zeros(4, 8), g)
    with pytest.raises((ValueError, TypeError)):
        fastermoe_amd.FMoETransformerMLP(num_expert=2, d_model=8, d_hidden=8)(torch.zeros(4, 8))


def test_c_abi_rejects_bad_arguments_before_any_launch():
    lib = _lib.load()
    import ctypes
    cnt = (ctypes.c_int64 * 2)(3, -1)
    rc = lib.fmoe_linear_forward(None, None, None, None, ctypes.cast(cnt, ctypes.c_void_p), 2, 8, 8, _lib.BF16, None)
    assert rc == -1 and b"negative" in lib.fmoe_last_error()
    rc = lib.fmoe_linear_forward(None, None, None, None, ctypes.cast(cnt, ctypes.c_void_p), 2, 8, 8, 99, None)
    assert rc == -1 and b"dtype" in lib.fmoe_last_error()
    rc = lib.fmoe_expert_count(None, None, 10, 1 << 20, None)
    assert rc == -2  # FMOE_ELIMIT
    rc = lib.fmoe_assign_pos(None, None, None, 0, 10, 4, None, 0, None)
    assert rc == -1
    with pytest.raises(_lib.FmoeHipError):
        _lib.check(rc)


def test_activation_codes():
    from fastermoe_amd.fused_functions import _activation_code
    assert _activation_code(torch.nn.GELU()) == _lib.ACT_GELU
    assert _activation_code(torch.nn.functional.gelu) == _lib.ACT_GELU
    assert _activation_code(torch.nn.ReLU()) == _lib.ACT_RELU
    assert _activation_code(torch.nn.Identity()) == _lib.ACT_NONE
    with pytest.raises(NotImplementedError):
        _activation_code(torch.nn.GELU(approximate="tanh"))
    with pytest.raises(NotImplementedError):
        _activation_code(torch.nn.Tanh())


def test_fused_chunk_bounds_host_logic():
    """Chunk planning of the fused pipeline (host only): monotone, covers all rows, every bound on a
    row-tile edge, and -- when the chunks are long enough -- whole rounds of workgroups for both
    output widths in every chunk but the last."""
    import ctypes
    lib = _lib.load()

    def bounds(counts, n_chunks, d=4096, h=14336, cus=256):
        c = (ctypes.c_int64 * len(counts))(*counts)
        b = (ctypes.c_int64 * (n_chunks + 1))()
        _lib.check(lib.fmoe_fused_chunk_bounds(ctypes.cast(c, ctypes.c_void_p), len(counts), n_chunks, d, h, cus,
                                               ctypes.cast(b, ctypes.c_void_p)))
        return list(b)

    def tiles_between(counts, lo, hi):
        """Row tiles of 256 of the rows [lo, hi), every expert tiled from its own first row."""
        t, start = 0, 0
        for n in counts:
            a, b = max(lo, start), min(hi, start + n)
            if b > a:
                t += -(-(b - a) // 256)
            start += n
        return t

    def tile_edges(counts):
        edges, start = {0}, 0
        for n in counts:
            edges |= {start + r for r in range(256, n, 256)} | {start + n}
            start += n
        return edges

    # the Mixtral-like share: 8 nearly equal experts, 4 chunks -> 64 row tiles (4 and 14 whole rounds
    # of 256 workgroups for widths 4096 and 14336) in the first three chunks, the rest in the last
    counts = [8100, 8300, 8192, 8000, 8400, 8192, 8150, 8202]
    b = bounds(counts, 4)
    assert b[0] == 0 and b[-1] == sum(counts) and all(x <= y for x, y in zip(b, b[1:]))
    assert all(x in tile_edges(counts) for x in b)
    per_chunk = [tiles_between(counts, lo, hi) for lo, hi in zip(b, b[1:])]
    assert per_chunk[:3] == [64, 64, 64] and sum(per_chunk) == sum(-(-n // 256) for n in counts)
    for t in per_chunk[:3]:
        assert t * 16 % 256 == 0 and t * 56 % 256 == 0
    # chunks too short for whole rounds: an even split of the row tiles, still on tile edges
    assert bounds([1000], 4) == [0, 256, 512, 768, 1000]
    assert bounds([100, 900], 2) == [0, 356, 1000]      # 1 + 4 tiles: bound after the second tile
    assert bounds([512, 512], 2, d=256, h=256, cus=2) == [0, 512, 1024]
    # more chunks than rows, empty experts: still monotone and complete
    b = bounds([0, 3, 0, 0, 2], 8)
    assert b[0] == 0 and b[-1] == 5 and all(x <= y for x, y in zip(b, b[1:]))
    assert bounds([0, 0], 3) == [0, 0, 0, 0]
    rc = lib.fmoe_fused_chunk_bounds(None, 2, 3, 64, 64, 0, None)
    assert rc == -1

    # n_chunks = 0, the library's own choice: up to 4 chunks, each with at least four rounds of tiles in
    # its narrower product (5 entries come back, those past the chosen count repeat the end)
    def auto(counts, d, h, cus=256):
        c = (ctypes.c_int64 * len(counts))(*counts)
        b = (ctypes.c_int64 * 5)()
        _lib.check(lib.fmoe_fused_chunk_bounds(ctypes.cast(c, ctypes.c_void_p), len(counts), 0, d, h, cus,
                                               ctypes.cast(b, ctypes.c_void_p)))
        return list(b)

    assert auto(counts, 4096, 14336) == bounds(counts, 4)           # 256 row tiles x 16: 4 rounds per chunk
    total = 16 * 2048
    assert auto([2048] * 16, 1024, 4096) == [0] + [total] * 4       # 128 row tiles x 4 = 2 rounds: one chunk
    two = auto([256] * 256, 2048, 1024)                             # 256 row tiles x 4 = 4 rounds: one chunk
    assert two == [0] + [65536] * 4
    assert auto([4096] * 32, 2048, 1024)[:3] == bounds([4096] * 32, 2, 2048, 1024)   # 512 row tiles: two chunks
    assert auto([0, 0], 64, 64) == [0, 0, 0, 0, 0]


def test_gemm_tail_plan_host_logic():
    """Which tiles of a launch are split along the contraction (host only)."""
    import ctypes
    lib = _lib.load()

    def plan(tiles, slabs, cus=256):
        out = (ctypes.c_int64 * 3)()
        _lib.check(lib.fmoe_gemm_tail_plan(tiles, slabs, cus, ctypes.cast(out, ctypes.c_void_p)))
        return list(out)

    assert plan(1024, 224)[:2] == [1024, 1]            # whole rounds: nothing to split
    assert plan(1040, 224) == [1024, 8, 28]            # 16 tail tiles x 8 parts of 28 slabs
    assert plan(1104, 224) == [1024, 3, 75]            # 80 tail tiles: 3 parts fit the idle units
    assert plan(3640, 64) == [3584, 4, 16]             # parts keep at least 16 slabs
    assert plan(3720, 64)[:2] == [3720, 1]             # the last round fills more than half the chip
    assert plan(80, 8)[:2] == [80, 1]                  # contraction too short to split
    assert plan(5, 33)[:2] == [5, 1]                   # two parts would save 16 slabs: less than the reduction costs
    m, f, per = plan(5, 100)
    assert (m, f) == (0, 6) and per * f >= 100 and per * (f - 1) < 100   # no empty part
    for tiles in range(1, 600, 7):
        for slabs in (1, 15, 16, 31, 32, 100, 224):
            m, f, per = plan(tiles, slabs)
            assert 0 <= m <= tiles and 1 <= f <= 8 and (tiles - m) * f <= 256 or f == 1
            if f > 1:
                assert per >= 16 and per * f >= slabs and per * (f - 1) < slabs and m % 256 == 0 and slabs - per >= 40


def test_reference_import_paths_resolve():
    """``import fmoe`` / ``import fmoe_cuda`` and the module paths the reference's users import from."""
    import importlib
    import fmoe
    import fmoe_cuda
    import fmoe_cuda as fmoe_native_alias
    assert fmoe_cuda is fmoe_native and fmoe_native_alias is fmoe_native
    for name in ("expert_count", "assign_pos", "linear_forward", "linear_backward", "limit_by_capacity",
                 "prune_gate_by_capacity", "fused_forward", "fused_backward"):
        assert callable(getattr(fmoe_cuda, name))
    assert fmoe.FMoE is fastermoe_amd.FMoE and fmoe.FMoETransformerMLP is fastermoe_amd.FMoETransformerMLP
    assert fmoe.FMoELinear is fastermoe_amd.FMoELinear
    assert fmoe.DistributedGroupedDataParallel is fastermoe_amd.DistributedGroupedDataParallel
    from fmoe.functions import (MOECache, MOEGather, MOELinear, MOEScatter, count_by_gate, ensure_comm,  # noqa: F401
                                prepare_forward)
    from fmoe.fused_functions import MOEForward  # noqa: F401
    from fmoe.gates import GShardGate, NaiveGate, NoisyGate, SwitchGate, ZeroGate  # noqa: F401
    from fmoe.gates.utils import limit_by_capacity  # noqa: F401
    from fmoe.layers import FMoE as LayersFMoE
    from fmoe.transformer import FMoETransformerMLP as TransformerMLP
    assert LayersFMoE is fastermoe_amd.FMoE and TransformerMLP is fastermoe_amd.FMoETransformerMLP
    assert importlib.import_module("fmoe.gates.naive_gate").NaiveGate is gates.NaiveGate
    assert importlib.import_module("fmoe.layers") is layers


def test_header_is_plain_c_and_a_c_program_links(tmp_path):
    """The boundary is a C ABI: include/fmoe_hip.h compiles as C99 (no C++ or torch types), and a C
    program that calls host-only entry points links against the library and runs without a GPU."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    lib_path = _lib.LIB_PATH
    src = tmp_path / "client.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include "fmoe_hip.h"
int main(void) {
    int64_t counts[3] = {300, 0, 724};
    int64_t bounds[3] = {-1, -1, -1};
    if (fmoe_abi_version() < 1) return 1;
    if (fmoe_fused_chunk_bounds(counts, 3, 2, 64, 64, 2, bounds) != FMOE_OK) return 2;
    if (bounds[0] != 0 || bounds[2] != 1024 || bounds[1] < 0 || bounds[1] > 1024) return 3;
    if (fmoe_fused_chunk_bounds(0, 3, 2, 64, 64, 2, bounds) != FMOE_EINVAL) return 4;
    if (strlen(fmoe_last_error()) == 0) return 5;
    printf("%lld %lld %lld\n", (long long)bounds[0], (long long)bounds[1], (long long)bounds[2]);
    return 0;
}
''')
    exe = tmp_path / "client"
    include = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    build = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", include, str(src), "-o", str(exe),
                            lib_path, f"-Wl,-rpath,{os.path.dirname(lib_path)}", "-Wl,-rpath,/opt/rocm/lib"],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0, (run.returncode, run.stdout, run.stderr)
    assert run.stdout.split()[0] == "0" and run.stdout.split()[2] == "1024"
