"""ctypes binding of ``libfmoe_hip.so`` (the C ABI of ``include/fmoe_hip.h``).

There is no fallback: if the library has not been built, importing this module
raises, and every operator of the package fails with it.  Build it with
``python -m fastermoe_amd.build``.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# FMOE_HIP_LIB points at another build of the same library (e.g. an experiment)
LIB_PATH = os.environ.get("FMOE_HIP_LIB") or os.path.join(_HERE, "lib", "libfmoe_hip.so")

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int


class MlpParams(ctypes.Structure):
    """``struct fmoe_mlp_params``."""
    _fields_ = [("w1", _vp), ("b1", _vp), ("w2", _vp), ("b2", _vp),
                ("n_expert", _i64), ("d_model", _i64), ("d_hidden", _i64),
                ("dtype", _int), ("activation", _int)]


# name -> (restype, argtypes); the authoritative list of exported symbols
SIGNATURES = {
    "fmoe_last_error": (ctypes.c_char_p, []),
    "fmoe_abi_version": (_int, []),
    "fmoe_expert_count": (_int, [_vp, _vp, _i64, _i64, _vp]),
    "fmoe_routing_workspace_bytes": (_i64, [_i64, _i64]),
    "fmoe_assign_pos": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp]),
    "fmoe_route": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _vp]),
    "fmoe_route_static": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _vp]),
    "fmoe_gate_topk_route": (_int, [_vp, _i64, _i64, _i64, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "fmoe_gate_linear_supported": (_int, [_i64, _i64, _i64, _int]),
    "fmoe_gate_linear_topk_route": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp,
                                           _i64, _vp]),
    "fmoe_gate_topk_backward": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _vp]),
    "fmoe_noisy_gate_forward": (_int, [_vp, _vp, _vp, ctypes.c_double, _i64, _i64, _i64, _int, _vp, _vp, _vp, _vp, _vp,
                                       _vp, _vp, _vp, _vp, _i64, _vp]),
    "fmoe_noisy_gate_backward": (_int, [_vp, _vp, _vp, ctypes.c_double, _i64, _i64, _i64, _int, _vp, _vp, _vp, _vp, _vp,
                                        _vp, _vp, _vp, _vp]),
    "fmoe_limit_by_capacity": (_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "fmoe_prune_gate_by_capacity": (_int, [_vp, _vp, _vp, _i64, _i64, _vp, _i64, _vp]),
    "fmoe_gather_rows": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "fmoe_gather_rows_div": (_int, [_vp, _vp, _i64, _vp, _i64, _i64, _i64, _int, _vp]),
    "fmoe_invert_index": (_int, [_vp, _i64, _vp, _i64, _vp]),
    "fmoe_reduce_slots": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "fmoe_index_add_workspace_bytes": (_i64, [_i64, _i64]),
    "fmoe_index_add_rows": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp, _i64, _vp]),
    "fmoe_mask_restore": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "fmoe_mask_scale_grad": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "fmoe_linear_forward": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "fmoe_linear_backward": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "fmoe_linear_act_forward": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _vp]),
    "fmoe_linear_dact_backward": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _vp]),
    "fmoe_segment_table_bytes": (_i64, [_i64, _i64]),
    "fmoe_segment_table_build": (_int, [_vp, _i64, _i64, _vp, _i64, _vp]),
    "fmoe_linear_dev_supported": (_int, [_i64, _i64, _int]),
    "fmoe_linear_dev_workspace_bytes": (_i64, [_i64, _int]),
    "fmoe_linear_forward_dev": (_int, [_vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp,
                                       _i64, _vp]),
    "fmoe_linear_dgrad_dev": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp, _i64, _vp]),
    "fmoe_linear_wgrad_dev": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "fmoe_gemm_tail_plan": (_int, [_i64, _i64, _int, _vp]),
    "fmoe_fused_chunk_bounds": (_int, [_vp, _i64, _int, _i64, _i64, _int, _vp]),
    "fmoe_fused_mlp_forward": (_int, [ctypes.POINTER(MlpParams), _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                                      _vp, _vp, _vp, _vp, _vp, _int, _vp]),
    "fmoe_fused_mlp_backward": (_int, [ctypes.POINTER(MlpParams), _vp, _vp, _vp, _vp, _i64, _i64, _i64,
                                       _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _vp]),
    "fmoe_fused_scatter_in_loader": (_int, [ctypes.POINTER(MlpParams), _vp, _i64]),
    "fmoe_combine_forward": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "fmoe_combine_backward": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "fmoe_gather_combine_forward": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "fmoe_gather_combine_backward": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "fmoe_profile_enable": (_int, [_int]),
    "fmoe_profile_classes": (_int, []),
    "fmoe_profile_collect": (_int, [_vp, _vp, _vp, _int]),
}

PROFILE_CLASSES = ["gemm_fwd", "gemm_dgrad", "gemm_wgrad", "bias_grad", "gather_rows", "scatter_rows",
                   "reduce_slots", "index_add", "combine"]

F32, BF16, F16, F64 = 0, 1, 2, 3
ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2

_lib = None


def load():
    """Loads the shared library once and types every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP kernels have not been built "
            "(run `python -m fastermoe_amd.build`); there is no fallback path")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


class FmoeHipError(RuntimeError):
    pass


def check(rc):
    """Turns a negative status of the C ABI into a Python exception."""
    if rc != 0:
        msg = load().fmoe_last_error()
        raise FmoeHipError(f"libfmoe_hip error {rc}: {msg.decode() if msg else '?'}")


def profile_enable(on):
    check(load().fmoe_profile_enable(1 if on else 0))


def profile_collect():
    """{class name: (launches, milliseconds, work)} since the last collect."""
    lib = load()
    n = lib.fmoe_profile_classes()
    cnt = (ctypes.c_int64 * n)()
    ms = (ctypes.c_double * n)()
    work = (ctypes.c_double * n)()
    check(lib.fmoe_profile_collect(ctypes.cast(cnt, _vp), ctypes.cast(ms, _vp), ctypes.cast(work, _vp), n))
    return {PROFILE_CLASSES[i]: (cnt[i], ms[i], work[i]) for i in range(n)}
