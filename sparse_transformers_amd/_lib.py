"""ctypes loader for libsparse_mlp_amd.so (the C ABI declared in include/sparse_mlp_amd.h).

The library is looked up next to this file.  There is no CPU fallback: if it is
missing, or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libsparse_mlp_amd.so")

ST_OK = 0
ST_ERR_ARG = -1
ST_ERR_NO_ACTIVE = -2
ST_ERR_HIP = -3
ST_ERR_INVALID = -4

ST_F32, ST_F16, ST_BF16, ST_F64 = 0, 1, 2, 3
ACT_CODES = {"relu": 0, "silu": 1, "gelu_pytorch_tanh": 2, "sigmoid": 3, "identity": 4}

STATE_N_ACTIVE, STATE_N_CHANGED, STATE_STATUS, STATE_VALID = 0, 1, 2, 3
STATE_N_ADDED, STATE_N_REMOVED, STATE_SERIAL, STATE_EPOCH, STATE_WORDS = 4, 5, 6, 7, 16


class CacheBuffers(C.Structure):
    _fields_ = [
        ("gate_pool", C.c_void_p), ("up_pool", C.c_void_p), ("downT_pool", C.c_void_p),
        ("gate_active", C.c_void_p), ("up_active", C.c_void_p), ("down_active", C.c_void_p),
        ("indices", C.c_void_p), ("cur_mask", C.c_void_p), ("state", C.c_void_p),
    ]


# name -> (restype, argtypes); every symbol include/sparse_mlp_amd.h declares
_vp, _i64, _ci, _f = C.c_void_p, C.c_int64, C.c_int, C.c_float
SIGNATURES = {
    "st_version": (_ci, []),
    "st_last_error": (C.c_char_p, []),
    "st_mlp_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "st_mlp_f64_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "st_mlp_forward": (_ci, [_vp, _i64, _i64, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _vp, _i64, _vp, _i64, _ci, _ci, _ci,
                             _vp]),
    "st_mlp_static_scratch_bytes": (_i64, []),
    "st_mlp_forward_static": (_ci, [_vp, _i64, _i64, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _vp, _i64, _ci, _ci, _ci, _vp]),
    "st_predictor_mask": (_ci, [_vp, _i64, _i64, _vp, _i64, _vp, _i64, _ci, _f, _ci, _vp, _vp, _vp, _vp]),
    "st_predictor_mask_ex": (_ci, [_vp, _i64, _i64, _vp, _i64, _vp, _i64, _ci, _f, _ci, _ci, _vp, _vp, _vp, _vp]),
    "st_mask_select_workspace_bytes": (_i64, [_i64, _i64]),
    "st_mask_select": (_ci, [_vp, _i64, _i64, _ci, _i64, _f, _vp, _vp, _vp, _i64, _vp]),
    "st_approx_topk_threshold": (_ci, [_vp, _i64, _i64, _i64, _vp, _vp]),
    "st_approx_topk_threshold_f64": (_ci, [_vp, _i64, _i64, _i64, _vp, _vp]),
    "st_cache_max_intermediate": (_i64, []),
    "st_cache_create": (_vp, [C.POINTER(CacheBuffers), _i64, _i64, _ci, _ci]),
    "st_cache_destroy": (None, [_vp]),
    "st_cache_load_weights": (_ci, [_vp, _vp, _vp, _vp, _vp]),
    "st_cache_update_async": (_ci, [_vp, _vp, _vp]),
    "st_cache_update_forward": (_ci, [_vp, _vp, _vp, _i64, _i64, _vp, _vp, _i64, _vp, _i64, _ci, _vp]),
    "st_cache_sync_state": (_ci, [_vp, _vp, _vp]),
    "st_cache_materialize_concat": (_ci, [_vp, _vp, _i64, _vp]),
    "st_profile_enable": (_ci, [_ci]),
    "st_profile_disable": (_ci, []),
    "st_profile_collect": (_ci, [_vp, _vp, _ci]),
}

KERNEL_KINDS = ["mlp_decode", "mlp_reduce", "cache_update", "mask_select", "pred_down", "pred_up_mask",
                "mlp_prefill_gateup", "mlp_prefill_down", "mlp_batch_gateup", "mlp_batch_down",
                "cache_update_decode"]

_lib = None


class NativeLibraryMissing(ImportError):
    pass


def lib() -> C.CDLL:
    """Load the HIP library once; raise loudly when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NativeLibraryMissing(
                f"{LIB_PATH} not found: build it with `python -m sparse_transformers_amd.build` "
                "(this package has no CPU fallback)")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error() -> str:
    return lib().st_last_error().decode("utf-8", "replace")


def check(rc: int, what: str) -> None:
    """Translate a negative st_status into the exception the reference would raise."""
    if rc == ST_OK:
        return
    msg = last_error()
    if rc == ST_ERR_NO_ACTIVE:
        raise RuntimeError("No active weights")
    if rc == ST_ERR_INVALID:
        raise RuntimeError("Cache is not valid")
    if rc == ST_ERR_ARG:
        raise ValueError(f"{what}: {msg}")
    raise RuntimeError(f"{what}: {msg} (status {rc})")
