"""ctypes binding of libgalvatron_moe.so (C ABI declared in include/galvatron_moe.h).

The library is the only compute backend of this package: there is no Python or CPU fallback, and
`lib()` raises if the shared object has not been built (`python hetu-galvatron_amd/build.py`).
"""
from __future__ import annotations

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
# GALVATRON_MOE_LIB selects another build of the same ABI (e.g. a tuning variant)
LIB_PATH = os.environ.get("GALVATRON_MOE_LIB") or os.path.join(_HERE, "_lib", "libgalvatron_moe.so")
ABI_VERSION = 10

GMOE_F32, GMOE_BF16, GMOE_F16, GMOE_F8E4M3 = 0, 1, 2, 3
SCORE_SOFTMAX, SCORE_SIGMOID, SCORE_IDENTITY = 0, 1, 2
ACT_SILU, ACT_GELU = 0, 1

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_f32 = ctypes.c_float

# name -> (restype, argtypes); must list every function declared in include/galvatron_moe.h
PROTOTYPES = {
    "gmoe_abi_version": (_int, []),
    "gmoe_status_string": (ctypes.c_char_p, [_int]),
    "gmoe_route_workspace_bytes": (_i64, [_i64, _int]),
    "gmoe_route_topk": (_int, [_vp, _int, _i64, _int, _int, _int, _int, _f32, _vp, _vp, _int, _int,
                               _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "gmoe_seq_aux_loss": (_int, [_vp, _int, _vp, _i64, _int, _int, _int, _int, _f32, _vp, _vp, _vp, _vp]),
    "gmoe_seq_aux_loss_bwd": (_int, [_vp, _int, _i64, _int, _int, _int, _int, _vp, _f32, _vp, _vp, _vp]),
    "gmoe_score_stats": (_int, [_vp, _int, _i64, _int, _int, _int, _vp, _vp, _vp]),
    "gmoe_score_stats_bwd": (_int, [_vp, _int, _i64, _int, _int, _int, _vp, _f32, _f32, _vp, _vp, _vp]),
    "gmoe_sinkhorn": (_int, [_vp, _int, _i64, _int, _f32, _int, _vp, _vp, _vp]),
    "gmoe_router_bookkeeping": (_int, [_vp, _vp, _int, _f32, _f32, _vp, _vp, _vp, _f32, _vp, _f32, _vp,
                                       _vp]),
    "gmoe_expert_bias_update": (_int, [_vp, _vp, _i64, _int, _f32, _vp, _vp]),
    "gmoe_route_topk_bwd": (_int, [_vp, _int, _i64, _int, _int, _int, _int, _f32, _vp, _vp, _vp,
                                   _f32, _f32, _vp, _vp, _vp]),
    "gmoe_capacity_select": (_int, [_vp, _int, _vp, _i64, _int, _i64, _int, _int, _vp, _vp, _vp]),
    "gmoe_permute_plan_workspace_bytes": (_i64, [_i64, _int]),
    "gmoe_permute_plan": (_int, [_vp, _i64, _int, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp]),
    "gmoe_permute_plan_static_max_slots": (_i64, []),
    "gmoe_permute_plan_static": (_int, [_vp, _i64, _int, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _vp]),
    "gmoe_permute_rows": (_int, [_vp, _int, _i64, _i64, _int, _vp, _i64, _vp, _vp, _int, _vp, _vp]),
    "gmoe_unpermute_rows": (_int, [_vp, _int, _i64, _i64, _int, _vp, _i64, _vp, _int, _vp, _vp,
                                   _vp, _vp, _vp, _vp]),
    "gmoe_unpermute_rows_bwd": (_int, [_vp, _vp, _int, _i64, _i64, _int, _vp, _i64, _vp, _int,
                                       _vp, _vp, _vp]),
    "gmoe_scatter_add_rows": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _int, _i64, _vp, _vp]),
    "gmoe_cast_rows": (_int, [_vp, _i64, _int, _vp, _vp]),
    "gmoe_sort_chunks": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _int, _vp, _vp, _vp]),
    "gmoe_scatter_rows_by_map": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _vp]),
    "gmoe_glu_fwd": (_int, [_vp, _int, _i64, _i64, _int, _vp, _vp]),
    "gmoe_glu_bwd": (_int, [_vp, _vp, _int, _i64, _i64, _int, _vp, _vp]),
    "gmoe_glu_fwd_fp8store": (_int, [_vp, _int, _i64, _i64, _int, _vp, _vp, _vp]),
    "gmoe_glu_bwd_fp8in": (_int, [_vp, _vp, _int, _i64, _i64, _int, _vp, _vp]),
    "gmoe_bias_rows": (_int, [_vp, _vp, _int, _i64, _i64, _vp, _int, _vp, _vp]),
    "gmoe_bias_rows_bwd": (_int, [_vp, _int, _i64, _i64, _vp, _int, _vp, _vp]),
    "gmoe_gmm_workspace_bytes": (_i64, [_int, _i64, _i64, _i64, _int, _int, _int]),
    "gmoe_gmm": (_int, [_vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _int, _int, _int, _vp, _i64,
                        _vp]),
    "gmoe_gmm_glu": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _int, _vp]),
    "gmoe_gmm_glu_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _int, _vp]),
    "gmoe_gmm_fp8w": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _vp]),
    "gmoe_quantize_fp8_block": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _vp]),
    "gmoe_quantize_fp8_rows": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _vp]),
    "gmoe_glu_fwd_quantize_fp8_rows": (_int, [_vp, _int, _i64, _i64, _int, _vp, _vp, _vp]),
    "gmoe_glu_bwd_quantize_fp8_rows": (_int, [_vp, _vp, _int, _i64, _i64, _int, _vp, _vp, _vp]),
    "gmoe_gmm_fp8a": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _int, _vp]),
    "gmoe_gate_fwd_workspace_bytes": (_i64, [_i64, _i64, _int, _int]),
    "gmoe_gate_fwd": (_int, [_vp, _vp, _i64, _i64, _int, _int, _vp, _int, _vp, _i64, _vp]),
    "gmoe_gate_bwd_input_workspace_bytes": (_i64, [_i64, _i64, _int, _int, _int]),
    "gmoe_gate_bwd_input": (_int, [_vp, _int, _vp, _i64, _i64, _int, _int, _vp, _vp, _i64, _vp]),
    "gmoe_gate_bwd_workspace_rows": (_i64, [_i64, _i64, _int, _int]),
    "gmoe_gate_bwd_weight": (_int, [_vp, _int, _vp, _i64, _i64, _int, _int, _vp, _vp, _i64, _vp]),
    "gmoe_rmsnorm_fwd": (_int, [_vp, _vp, _i64, _i64, _f32, _int, _vp, _vp, _vp]),
    "gmoe_rmsnorm_bwd_workspace_rows": (_i64, [_i64, _i64, _int]),
    "gmoe_rmsnorm_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _int, _vp, _vp, _vp, _i64, _vp]),
}

_lib = None
_lock = threading.Lock()


class LibraryMissingError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """The loaded shared library (loaded once per process)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise LibraryMissingError(
                    "HIP library %s is missing: build it with `python %s`. This package has no "
                    "fallback path." % (LIB_PATH, os.path.join(_HERE, "build.py")))
            handle = ctypes.CDLL(LIB_PATH)
            for name, (restype, argtypes) in PROTOTYPES.items():
                fn = getattr(handle, name)  # AttributeError if the export is missing
                fn.restype = restype
                fn.argtypes = argtypes
            got = handle.gmoe_abi_version()
            if got != ABI_VERSION:
                raise RuntimeError("libgalvatron_moe.so ABI %d, Python expects %d: rebuild" %
                                   (got, ABI_VERSION))
            _lib = handle
    return _lib


def check(status: int, what: str) -> None:
    """Turn a negative gmoe_status into a RuntimeError."""
    if status != 0:
        msg = lib().gmoe_status_string(status).decode()
        raise RuntimeError("%s failed: %s (status %d)" % (what, msg, status))
