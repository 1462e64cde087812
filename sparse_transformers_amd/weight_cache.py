"""HBM-resident differential weight cache with the reference's class surface.

Mirrors ``torch.classes.sparse_mlp.WeightCache`` (sparse_transformers/csrc/weight_cache.h:13-381,
registered in sparse_mlp_op.cpp:198-202): same six constructor arguments, ``update_active_weights``,
``get_concat_weight``, ``get_active_down_weight``.  All storage is device memory owned by torch
tensors; the bookkeeping (ordered active list, mask diff, pairing, swap-with-last) runs in HIP kernels.
"""
from __future__ import annotations

import ctypes as C
import weakref
from typing import Optional

import torch

from . import _lib
from .ops import (_check_workspace, check_mlp_args, combined_for_launch, current_stream_ptr, dtype_code,
                  mlp_forward_rows, mlp_workspace, mlp_workspace_bytes, require_gpu)


class ConcatWeightHandle(torch.Tensor):
    """What ``WeightCache.get_concat_weight()`` returns: a tensor of shape ``[2n,H]`` (``[n,H]`` ungated) that
    owns no memory until something reads it.  ``sparse_mlp_forward`` recognises it and reads the cache's packed
    gate / up rows in place, so the reference's call sequence costs no ``[2n,H]`` copy (the reference pays a
    ``torch::cat`` per update, weight_cache.h:138).  Any other torch operation on it (``.t()``, ``matmul``,
    indexing, ``.cpu()`` ...) first materialises the contiguous tensor with one device copy and then runs on
    that.  Like the reference's tensor it describes the cache as of the update it was fetched after: a handle that is
    still alive when the next update is enqueued through this object is filled first (one device copy), so it stays a
    snapshot as the reference's ``torch::cat`` result does; when nobody holds it any more -- the usual case, a handle
    fetched for one forward -- nothing is copied.  Updates that bypass this object's methods (a replayed HIP graph)
    cannot do that: a handle that was not filled before such an update raises when it is used, instead of silently
    showing newer rows under the old shape."""

    @staticmethod
    def __new__(cls, cache: "WeightCache", n: int, serial: int):
        rows = (2 if cache.has_gate else 1) * n
        t = torch.Tensor._make_wrapper_subclass(cls, (rows, cache.hidden_size), dtype=cache.dtype,
                                                device=cache.device, requires_grad=False)
        t._cache, t._n, t._serial, t._real = cache, n, serial, None
        return t

    def fresh(self) -> bool:
        """True while no update has changed the cache since this handle was fetched."""
        c = self._cache
        return not c._dirty and c._host_state[_lib.STATE_SERIAL] == self._serial

    def materialize(self) -> torch.Tensor:
        if self._real is None:
            c = self._cache
            if not self.fresh():
                raise RuntimeError("this concat weight was fetched before the cache's last update; "
                                   "call get_concat_weight() again")
            buf = torch.empty(self.shape[0], c.hidden_size, dtype=c.dtype, device=c.device)
            if self._n > 0:
                rc = _lib.lib().st_cache_materialize_concat(c._h, buf.data_ptr(), self._n, current_stream_ptr(c.device))
                _lib.check(rc, "st_cache_materialize_concat")
            self._real = buf
        return self._real

    def __repr__(self):
        return f"ConcatWeightHandle(shape={tuple(self.shape)}, dtype={self.dtype}, materialized={self._real is not None})"

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        from torch.utils._pytree import tree_map

        def real(t):
            return t.materialize() if isinstance(t, cls) else t
        return func(*tree_map(real, args), **tree_map(real, kwargs or {}))


class WeightCache:
    """Drop-in for the reference WeightCache, plus a zero-copy fast path.

    Reference-compatible calls (each may read a few state words back from the device):
      ``update_active_weights(mask)``, ``get_concat_weight()``, ``get_active_down_weight()``.
    Fast path (nothing is read back, everything is stream-ordered):
      ``update_active_weights_async(mask)`` then ``forward(x, act, ...)``; the kernels take the active
      count from device memory.
    ``lazy_updates = True`` (off by default; the drop-in ``SkipMLP`` module switches it on for its cache) makes
    ``update_active_weights(mask)`` only remember the mask: the update then runs with the next ``forward`` as ONE
    fused update + MLP launch (``update_and_forward``) -- the order a decoder layer produces, where the mask is
    computed before attention and the MLP runs after it (src/modeling_skip.py:234-261) -- or, if a getter or
    another update comes first, on its own.  The caller must leave the mask tensor alone until then, and "No active
    weights" is reported by the next call that synchronises instead of by ``update_active_weights`` itself.
    """

    def __init__(self, init_mask: torch.Tensor, hidden_size: int, gate_weight: Optional[torch.Tensor],
                 up_weight: torch.Tensor, down_weight: torch.Tensor, has_gate: bool = True):
        self.has_gate = bool(has_gate)
        if self.has_gate and gate_weight is None:
            raise ValueError("has_gate=True needs gate_weight")
        dev = require_gpu(up_weight, down_weight, gate_weight if self.has_gate else None)
        self.device = dev
        self.dtype = up_weight.dtype
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(up_weight.size(0))
        I, H = self.intermediate_size, self.hidden_size
        if tuple(up_weight.shape) != (I, H) or tuple(down_weight.shape) != (H, I):
            raise ValueError(f"up must be [I,H] and down [H,I]; got {tuple(up_weight.shape)}, {tuple(down_weight.shape)}")
        if self.has_gate and tuple(gate_weight.shape) != (I, H):
            raise ValueError(f"gate must be [{I},{H}], got {tuple(gate_weight.shape)}")
        if down_weight.dtype != self.dtype or (self.has_gate and gate_weight.dtype != self.dtype):
            raise TypeError("gate, up and down weights must share one dtype")
        if self.dtype == torch.float64:
            raise TypeError("the weight cache holds float32, float16 or bfloat16 rows (float64 is served by "
                            "sparse_mlp_forward on caller-owned rows only)")
        code = dtype_code(up_weight)
        L = _lib.lib()
        if I > L.st_cache_max_intermediate():
            raise ValueError(f"intermediate size {I} exceeds the supported maximum {L.st_cache_max_intermediate()}")

        def wbuf():
            return torch.empty(I, H, dtype=self.dtype, device=dev)

        self.gate_pool = wbuf() if self.has_gate else None
        self.up_pool = wbuf()
        self.downT_pool = wbuf()
        self.gate_active = wbuf() if self.has_gate else None
        self.up_active = wbuf()
        self.down_active = wbuf()
        # bookkeeping is double-buffered on the device; state[STATE_EPOCH] says which half is current
        self.indices = torch.empty(2, I, dtype=torch.int32, device=dev)
        self.cur_mask = torch.empty(2, I, dtype=torch.uint8, device=dev)
        self.state = torch.empty(_lib.STATE_WORDS, dtype=torch.int32, device=dev)
        self.n_active_dev = self.state[_lib.STATE_N_ACTIVE:_lib.STATE_N_ACTIVE + 1]

        bufs = _lib.CacheBuffers(
            self.gate_pool.data_ptr() if self.has_gate else None, self.up_pool.data_ptr(), self.downT_pool.data_ptr(),
            self.gate_active.data_ptr() if self.has_gate else None, self.up_active.data_ptr(),
            self.down_active.data_ptr(), self.indices.data_ptr(), self.cur_mask.data_ptr(), self.state.data_ptr())
        self._h = L.st_cache_create(C.byref(bufs), I, H, code, int(self.has_gate))
        if not self._h:
            raise ValueError(_lib.last_error())

        up_c = up_weight.detach().contiguous()
        down_c = down_weight.detach().contiguous()
        gate_c = gate_weight.detach().contiguous() if self.has_gate else None
        rc = L.st_cache_load_weights(self._h, gate_c.data_ptr() if self.has_gate else None, up_c.data_ptr(),
                                     down_c.data_ptr(), current_stream_ptr(dev))
        _lib.check(rc, "st_cache_load_weights")
        self._host_state = (C.c_int32 * _lib.STATE_WORDS)()
        self._host_serial = -1      # serial the host copy of the state belongs to
        self._dirty = True          # updates enqueued since the last read-back
        self.lazy_updates = False
        self._pending_mask: Optional[torch.Tensor] = None
        self._concat_ref = None     # weak reference to the handle get_concat_weight() handed out last
        self._concat_serial = -1
        # weight_cache.h:226: the constructor ends with update_active_weights(init_mask)
        self.update_active_weights(init_mask)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _lib._lib is not None:
            _lib._lib.st_cache_destroy(h)

    # ------------------------------------------------------------------ updates
    def _mask_arg(self, mask: torch.Tensor) -> torch.Tensor:
        if mask.device != self.device:
            mask = mask.to(self.device)
        if mask.dtype not in (torch.bool, torch.uint8):
            mask = mask != 0
        if mask.numel() != self.intermediate_size:
            raise ValueError(f"mask must have {self.intermediate_size} elements, got {mask.numel()}")
        return mask if mask.is_contiguous() else mask.contiguous()

    def _keep_snapshot(self) -> None:
        """Before an update overwrites packed rows: a concat handle somebody still holds is filled now (the
        reference's tensor is a copy and survives later updates, weight_cache.h:138)."""
        h = self._concat_ref() if self._concat_ref is not None else None
        if h is not None and h._real is None and h.fresh():
            h.materialize()

    def _flush_pending(self) -> None:
        """A remembered mask (``lazy_updates``) that no forward has consumed is applied now, on its own."""
        m, self._pending_mask = self._pending_mask, None
        if m is not None:
            self.update_active_weights_async(m)

    def update_active_weights_async(self, mask: torch.Tensor) -> None:
        """Enqueue the differential update on the current stream; never waits for the device."""
        m = self._mask_arg(mask)
        self._flush_pending()
        self._keep_snapshot()
        rc = _lib.lib().st_cache_update_async(self._h, m.data_ptr(), current_stream_ptr(self.device))
        _lib.check(rc, "st_cache_update_async")
        self._dirty = True

    def update_active_weights(self, mask: torch.Tensor) -> None:
        """weight_cache.h:229: raises RuntimeError("No active weights") when the mask empties the cache."""
        if self.lazy_updates:
            self._flush_pending()
            self._pending_mask = self._mask_arg(mask)
            return
        known = not self._dirty
        serial = int(self._host_state[_lib.STATE_SERIAL])
        self.update_active_weights_async(mask)
        try:
            self.sync_state()
        except RuntimeError as exc:
            # The "emptied" status stays in the state words until an update changes something.  An update with an
            # unchanged mask touches nothing and returns silently in the reference (weight_cache.h:237-240), also
            # right after the update that emptied the cache: only an update that did something may raise.
            if str(exc) == "No active weights" and known and int(self._host_state[_lib.STATE_SERIAL]) == serial:
                return
            raise

    def sync_state(self) -> dict:
        """Read the state words back (waits for the current stream)."""
        self._flush_pending()
        if self._dirty:
            rc = _lib.lib().st_cache_sync_state(self._h, self._host_state, current_stream_ptr(self.device))
            self._dirty = False
            _lib.check(rc, "st_cache_sync_state")
        s = self._host_state
        return {"n_active": s[_lib.STATE_N_ACTIVE], "n_changed": s[_lib.STATE_N_CHANGED],
                "status": s[_lib.STATE_STATUS], "valid": s[_lib.STATE_VALID], "n_added": s[_lib.STATE_N_ADDED],
                "n_removed": s[_lib.STATE_N_REMOVED], "serial": s[_lib.STATE_SERIAL],
                "epoch": s[_lib.STATE_EPOCH]}

    # ------------------------------------------------------------------ getters
    def get_num_active(self) -> int:
        return int(self.sync_state()["n_active"])

    def get_active_indices(self) -> torch.Tensor:
        """Ordered active list (the reference's ``active_indices``) as int64[n]."""
        st = self.sync_state()
        return self.indices[int(st["epoch"]), : int(st["n_active"])].to(torch.int64)

    def _require_valid(self) -> dict:
        st = self.sync_state()
        if not st["valid"]:
            raise RuntimeError("Cache is not valid")
        return st

    def get_concat_weight(self) -> torch.Tensor:
        """``[2n,H]`` (gate rows then up rows; ``[n,H]`` when ungated), valid until the next update.  Returned
        as a ``ConcatWeightHandle``: no copy is made unless something other than ``sparse_mlp_forward`` reads it."""
        st = self._require_valid()
        h = self._concat_ref() if self._concat_ref is not None else None
        if h is None or self._concat_serial != st["serial"]:
            h = ConcatWeightHandle(self, int(st["n_active"]), st["serial"])
            self._concat_ref, self._concat_serial = weakref.ref(h), st["serial"]
        return h

    def get_active_down_weight(self) -> torch.Tensor:
        """[H,n] view with strides (1,H) over the packed down rows (zero-copy)."""
        st = self._require_valid()
        return self.down_active[: int(st["n_active"])].t()

    # ---------------------------------------------------------------- fast path
    def _x_rows(self, x: torch.Tensor) -> torch.Tensor:
        H = self.hidden_size
        if x.shape[-1] != H:
            raise ValueError(f"x must have {H} columns, got {tuple(x.shape)}")
        if x.dtype != self.dtype or x.device != self.device:
            raise TypeError(f"x must be {self.dtype} on {self.device}, got {x.dtype} on {x.device}")
        x2 = x.reshape(-1, H)
        return x2 if x2.is_contiguous() else x2.contiguous()

    def update_and_forward(self, mask: torch.Tensor, x: torch.Tensor, act: str = "silu",
                           out: Optional[torch.Tensor] = None, combined: Optional[torch.Tensor] = None,
                           n_hint: Optional[int] = None, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``update_active_weights(mask)`` followed by the sparse MLP on x, enqueued as one call and never
        touching the host.  For one row of x this is a single kernel that takes the rows whose index
        changed straight from the pool (and writes them back to the active buffers on the way); the
        cache state and the result equal those of the two separate calls bit for bit.  ``n_hint`` (default:
        the last count the host saw) only steers what the kernel requests before it knows the true count.
        ``workspace``: a caller-owned uint8 buffer of ``mlp_workspace_bytes(B, H, I)`` bytes (default: one
        kept per device and stream)."""
        m = self._mask_arg(mask)
        self._flush_pending()
        H, I = self.hidden_size, self.intermediate_size
        x2 = self._x_rows(x)
        B = x2.size(0)
        if out is None:
            out = torch.empty_like(x2)
        # the count after the update is not known on the host: `combined` must hold the largest possible one
        check_mlp_args(x2, out, combined, self.dtype, self.device, H, (2 if self.has_gate else 1) * I)
        need = mlp_workspace_bytes(B, H, I)
        ws = mlp_workspace(self.device, B, H, I) if workspace is None else _check_workspace(workspace, self.device, need)
        if act not in _lib.ACT_CODES:
            raise ValueError(f"unknown activation {act!r}; expected one of {sorted(_lib.ACT_CODES)}")
        combined, copy_back = combined_for_launch(combined, B, I)
        self._keep_snapshot()
        rc = _lib.lib().st_cache_update_forward(
            self._h, m.data_ptr(), x2.data_ptr(), B,
            int(self._host_state[_lib.STATE_N_ACTIVE]) if n_hint is None else int(n_hint), out.data_ptr(),
            combined.data_ptr() if combined is not None else None, combined.stride(0) if combined is not None else 0,
            ws.data_ptr(), ws.numel(), _lib.ACT_CODES[act], current_stream_ptr(self.device))
        _lib.check(rc, "st_cache_update_forward")
        self._dirty = True
        if copy_back is not None:
            copy_back.copy_(combined)
        return out.view(x.shape)

    def forward(self, x: torch.Tensor, act: str = "silu", out: Optional[torch.Tensor] = None,
                combined: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Sparse MLP on the cache's packed rows; the active count is read on the device."""
        if self._pending_mask is not None:      # lazy_updates: the remembered update and this forward as one call
            m, self._pending_mask = self._pending_mask, None
            if combined is None or combined.size(-1) >= (2 if self.has_gate else 1) * self.intermediate_size:
                return self.update_and_forward(m, x, act, out=out, combined=combined, workspace=workspace)
            self.update_active_weights_async(m)   # `combined` is sized for the current count only: two calls
        x2 = self._x_rows(x)
        if out is None:
            out = torch.empty_like(x2)
        # the last count the host saw is only a prefetch hint; the kernels read the true one on the device
        # (mlp_forward_rows checks out / combined against the cache's dtype, device and capacity I)
        mlp_forward_rows(x2, self.gate_active, self.up_active, self.down_active, self.intermediate_size,
                         self.n_active_dev, out, combined, act, self.has_gate,
                         n_hint=int(self._host_state[_lib.STATE_N_ACTIVE]), workspace=workspace)
        return out.view(x.shape)
