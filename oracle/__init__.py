"""CPU oracle for the sparse-MLP decode path.  TEST INFRASTRUCTURE ONLY.

ctypes bindings over ``liboracle.so`` (built from ``sparse_mlp_oracle.c`` by
``oracle/Makefile``) plus a loader for the reference's own C++ operator when it
has been compiled into ``oracle/_ref``.  Only the test-suite, the smoke check
and the benchmark's CPU-baseline leg may import this package; the product
package ``sparse_transformers_amd`` never does.

Reference files each binding mirrors are cited in ``sparse_mlp_oracle.c``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
REF_SO_PATH = os.path.join(_HERE, "_ref", "sparse_transformers_ref.so")

ACT_CODES = {"relu": 0, "silu": 1, "gelu_pytorch_tanh": 2, "sigmoid": 3, "identity": 4}

ERR_NO_ACTIVE = 1


def build(with_ref: bool = True) -> None:
    """Compile liboracle.so (and oracle/_ref when the reference checkout is present)."""
    targets = ["oracle"] + (["ref"] if with_ref else [])
    subprocess.run(["make", "-C", _HERE, "-B"] + targets, check=True, stdout=subprocess.DEVNULL)


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build(with_ref=False)
        L = C.CDLL(_LIB_PATH)
        vp, i64, ci = C.c_void_p, C.c_int64, C.c_int
        L.orc_cache_create.restype = vp
        L.orc_cache_create.argtypes = [vp, i64, i64, vp, vp, vp, ci, C.POINTER(ci)]
        L.orc_cache_destroy.argtypes = [vp]
        L.orc_cache_update.restype = ci
        L.orc_cache_update.argtypes = [vp, vp]
        L.orc_cache_num_active.restype = i64
        L.orc_cache_num_active.argtypes = [vp]
        L.orc_cache_valid.restype = ci
        L.orc_cache_valid.argtypes = [vp]
        L.orc_cache_indices.argtypes = [vp, vp]
        for name in ("orc_cache_concat", "orc_cache_down_active", "orc_cache_gate_active", "orc_cache_up_active"):
            getattr(L, name).restype = vp
            getattr(L, name).argtypes = [vp]
        L.orc_mlp_forward.argtypes = [vp, i64, i64, vp, i64, vp, vp, vp, ci, ci]
        L.orc_predictor_scores.argtypes = [vp, i64, i64, vp, i64, vp, i64, vp]
        L.orc_mask_threshold.argtypes = [vp, i64, i64, C.c_float, ci, vp]
        L.orc_mask_topk.argtypes = [vp, i64, i64, i64, vp]
        L.orc_mask_statistical.argtypes = [vp, i64, i64, C.c_float, vp, vp]
        L.orc_approx_topk_threshold.argtypes = [vp, i64, i64, i64, vp]
        L.orc_approx_topk_threshold_f64.argtypes = [vp, i64, i64, i64, vp]
        _lib = L
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a).astype(np.uint8))


def _p(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


class NoActiveWeights(RuntimeError):
    pass


class OracleWeightCache:
    """Host-memory differential weight cache with the reference's semantics."""

    def __init__(self, init_mask, hidden_size, gate_weight, up_weight, down_weight, has_gate=True):
        up = _f32(up_weight)
        down = _f32(down_weight)
        self.I, self.H = int(up.shape[0]), int(hidden_size)
        assert up.shape == (self.I, self.H) and down.shape == (self.H, self.I)
        self.has_gate = bool(has_gate)
        gate = _f32(gate_weight) if self.has_gate else None
        err = C.c_int(0)
        m = _u8(init_mask)
        self._h = lib().orc_cache_create(_p(m), self.I, self.H, _p(gate) if gate is not None else None, _p(up),
                                         _p(down), int(self.has_gate), C.byref(err))
        if err.value == ERR_NO_ACTIVE:
            raise NoActiveWeights("No active weights")

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _lib is not None:
            _lib.orc_cache_destroy(h)

    def update_active_weights(self, mask) -> None:
        m = _u8(mask)
        assert m.shape == (self.I,)
        if lib().orc_cache_update(self._h, _p(m)) == ERR_NO_ACTIVE:
            raise NoActiveWeights("No active weights")

    @property
    def num_active(self) -> int:
        return int(lib().orc_cache_num_active(self._h))

    def get_active_indices(self) -> np.ndarray:
        out = np.empty(self.num_active, dtype=np.int64)
        lib().orc_cache_indices(self._h, _p(out))
        return out

    def _view(self, fn, rows) -> np.ndarray:
        ptr = getattr(lib(), fn)(self._h)
        buf = (C.c_float * (rows * self.H)).from_address(ptr)
        return np.frombuffer(buf, dtype=np.float32).reshape(rows, self.H)

    def _check_valid(self):
        if not lib().orc_cache_valid(self._h):
            raise RuntimeError("Cache is not valid")

    def get_concat_weight(self) -> np.ndarray:
        """[2n,H] gate rows then up rows ([n,H] when ungated); a copy."""
        self._check_valid()
        n = self.num_active
        return self._view("orc_cache_concat", (2 if self.has_gate else 1) * n).copy()

    def get_active_down_weight(self) -> np.ndarray:
        """[H,n] with strides (1,H) elements, like the reference's transposed view; a copy."""
        self._check_valid()
        return self._view("orc_cache_down_active", self.num_active).copy().T


def mlp_forward(x, concat_weight, active_down_weight, act="silu", has_gate=True):
    """Returns (out[B,H], combined[B,2n or n]).  active_down_weight is [H,n]."""
    x2 = _f32(x).reshape(-1, np.asarray(x).shape[-1])
    B, H = x2.shape
    cw = _f32(concat_weight)
    n = cw.shape[0] // 2 if has_gate else cw.shape[0]
    dn = _f32(np.asarray(active_down_weight, dtype=np.float32).T)  # packed [n,H]
    assert dn.shape == (n, H) and cw.shape[1] == H
    out = np.empty((B, H), dtype=np.float32)
    comb = np.empty((B, cw.shape[0]), dtype=np.float32)
    lib().orc_mlp_forward(_p(x2), B, H, _p(cw), n, _p(dn), _p(out), _p(comb), ACT_CODES[act], int(has_gate))
    return out.reshape(np.asarray(x).shape), comb


def _round_storage(a: np.ndarray, storage: str) -> np.ndarray:
    """float32 -> nearest value of the storage type (round to nearest even) -> float32."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    if storage == "float16":
        return a.astype(np.float16).astype(np.float32)
    if storage == "bfloat16":
        u = a.view(np.uint32).astype(np.uint64)
        r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
        out = (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32).copy()
        out[np.isnan(a)] = np.nan
        return out
    raise ValueError(f"unknown storage type {storage!r}")


def predictor_scores(x, A, Bm, storage=None) -> np.ndarray:
    """scores = (x @ A^T) @ Bm^T (src/modeling_skip.py:52-53).  ``storage`` ("float16" / "bfloat16"): the two maps as
    modules of a half-precision model compute them -- each output rounded to the storage type (products summed in
    higher precision first, as the BLAS kernels do)."""
    if storage in ("float16", "bfloat16"):
        x2 = np.asarray(x, dtype=np.float64).reshape(-1, np.asarray(x).shape[-1])
        t = _round_storage((x2 @ np.asarray(A, dtype=np.float64).T).astype(np.float32), storage)
        return _round_storage((t.astype(np.float64) @ np.asarray(Bm, dtype=np.float64).T).astype(np.float32), storage)
    x2 = _f32(x).reshape(-1, np.asarray(x).shape[-1])
    A, Bm = _f32(A), _f32(Bm)
    B, H = x2.shape
    r, I = A.shape[0], Bm.shape[0]
    assert A.shape == (r, H) and Bm.shape == (I, r)
    s = np.empty((B, I), dtype=np.float32)
    lib().orc_predictor_scores(_p(x2), B, H, _p(A), r, _p(Bm), I, _p(s))
    return s


def mask_threshold(scores, thr=0.0, ge=True) -> np.ndarray:
    s = _f32(scores)
    m = np.empty(s.shape[1], dtype=np.uint8)
    lib().orc_mask_threshold(_p(s), s.shape[0], s.shape[1], float(thr), int(ge), _p(m))
    return m.astype(bool)


def mask_topk(scores, k) -> np.ndarray:
    s = _f32(scores)
    m = np.empty(s.shape[1], dtype=np.uint8)
    lib().orc_mask_topk(_p(s), s.shape[0], s.shape[1], int(k), _p(m))
    return m.astype(bool)


def mask_statistical(scores, z):
    s = _f32(scores)
    m = np.empty(s.shape[1], dtype=np.uint8)
    cut = np.empty(s.shape[0], dtype=np.float32)
    lib().orc_mask_statistical(_p(s), s.shape[0], s.shape[1], float(z), _p(m), _p(cut))
    return m.astype(bool), cut


def approx_topk_threshold(scores, k) -> np.ndarray:
    """Per-row sketch threshold [B] (sparse_transformers/csrc/approx_topk.h:10-88).  float64 scores give a float64
    threshold (the reference dispatches on the scores' type), anything else is evaluated in float32."""
    f64 = isinstance(scores, np.ndarray) and scores.dtype == np.float64
    s = np.ascontiguousarray(scores, dtype=np.float64) if f64 else _f32(scores)
    if s.ndim != 2:
        raise ValueError("Input scores must be 2D tensor [batch_size, features]")
    if k <= 0:
        raise ValueError("k must be positive")
    if k > s.shape[1]:
        raise ValueError("k cannot be larger than feature size")
    if s.shape[1] < 4:
        raise ValueError("feature size below 4: the reference divides by a sketch width of zero")
    thr = np.empty(s.shape[0], dtype=s.dtype)
    fn = lib().orc_approx_topk_threshold_f64 if f64 else lib().orc_approx_topk_threshold
    fn(_p(s), s.shape[0], s.shape[1], int(k), _p(thr))
    return thr


# ---------------------------------------------------------------------------
# The reference's own operator, compiled from its sources into oracle/_ref.
# ---------------------------------------------------------------------------
_ref_loaded = None


def load_reference():
    """Load oracle/_ref/sparse_transformers_ref.so; returns (WeightCache class, forward op) or None."""
    global _ref_loaded
    if _ref_loaded is None:
        _ref_loaded = False
        if os.path.exists(REF_SO_PATH):
            import torch

            try:
                torch.classes.load_library(REF_SO_PATH)
                _ref_loaded = (torch.classes.sparse_mlp.WeightCache, torch.ops.sparse_mlp.forward)
            except Exception:  # pragma: no cover - e.g. libtorch mismatch on another host
                _ref_loaded = False
    return _ref_loaded or None
