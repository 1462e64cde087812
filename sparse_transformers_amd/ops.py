"""Operator-level host API: sparse_mlp_forward and the LoRA predictor mask.

Mirrors the operator surface of NimbleEdge/sparse_transformers:
  * ``sparse_mlp_forward(x, concat_weight, active_down_weight, down_proj_buffer,
    combined_proj_buffer, act, has_gate=True)`` — sparse_transformers/csrc/sparse_mlp_op.cpp:53-76,
    README.md:108-116 (six-argument call).
  * ``predictor_mask`` / ``predictor_scores`` — FastLoRAProjection.forward and
    SkipDecoderLayer._compute_binary_mask, src/modeling_skip.py:52-53,204-214.
  * ``mask_select`` — the "topk" and "statistical_topk" methods of the same function
    (src/modeling_skip.py:197-202,208-214).
  * ``approx_topk_threshold(scores, k)`` — sparse_transformers/csrc/approx_topk.h:10-88
    (registered in sparse_mlp_op.cpp:208).

torch is used for device memory and the current stream only; all arithmetic is
done by the HIP kernels behind the C ABI.
"""
from __future__ import annotations

import warnings
from typing import Optional

import torch

from . import _lib

_DTYPES = {torch.float32: _lib.ST_F32, torch.float16: _lib.ST_F16, torch.bfloat16: _lib.ST_BF16,
           torch.float64: _lib.ST_F64}   # (double precision: the stand-alone forward only)


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}; expected float32, float16, bfloat16 or float64") from None


def require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "sparse_transformers_amd runs on an AMD GPU only: got a tensor on "
                f"{t.device} (there is no CPU fallback)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def current_stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


_workspaces: dict = {}


def mlp_workspace_bytes(B: int, H: int, n: int, dtype: Optional[torch.dtype] = None) -> int:
    if dtype == torch.float64:
        return int(_lib.lib().st_mlp_f64_workspace_bytes(B, H, n))
    return int(_lib.lib().st_mlp_workspace_bytes(B, H, n))


def mlp_workspace(device: torch.device, B: int, H: int, n: int, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Scratch for one forward on the current stream of ``device``.

    One list of buffers per (device, stream): two streams never share scratch, and a buffer that has been
    handed out is kept for the life of the process -- a HIP graph captured earlier may have its address
    baked in, so growing must not free it.  Callers that replay graphs or know their largest batch should
    own a buffer instead (``torch.empty(mlp_workspace_bytes(B, H, I), dtype=torch.uint8)``) and pass it as
    ``workspace=``."""
    need = mlp_workspace_bytes(B, H, n, dtype)
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    bufs = _workspaces.setdefault(key, [])
    if not bufs or bufs[-1].numel() < need:
        grow = max(need, 2 * bufs[-1].numel() if bufs else 0)
        bufs.append(torch.empty(grow, dtype=torch.uint8, device=device))
    return bufs[-1]


def _check_workspace(ws: torch.Tensor, device: torch.device, need: int) -> torch.Tensor:
    if ws.dtype != torch.uint8 or not ws.is_cuda or ws.device != device or not ws.is_contiguous():
        raise ValueError("workspace must be a contiguous uint8 tensor on the cache's GPU")
    if ws.numel() < need:
        raise ValueError(f"workspace holds {ws.numel()} bytes, this call needs {need}")
    return ws


def check_mlp_args(x2: torch.Tensor, out: torch.Tensor, combined: Optional[torch.Tensor], dtype: torch.dtype,
                   device: torch.device, H: int, min_cols: int) -> None:
    """Host-side checks shared by every MLP launch: the kernels index x, out and combined as [B,H] / [B,ldc]
    arrays of the weights' element type, so a wrong dtype or a short buffer must never reach them."""
    B = x2.size(0)
    for name, t in (("x", x2), ("out", out), ("combined", combined)):
        if t is None:
            continue
        if t.dtype != dtype:
            raise TypeError(f"{name} has dtype {t.dtype}, the weights are {dtype}")
        if t.device != device:
            raise RuntimeError(f"{name} is on {t.device}, the weights are on {device}")
    if x2.dim() != 2 or x2.size(1) != H or not x2.is_contiguous():
        raise ValueError(f"x must be a contiguous [B,{H}] tensor, got {tuple(x2.shape)}")
    if out.dim() != 2 or tuple(out.shape) != (B, H) or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous [{B},{H}] tensor, got {tuple(out.shape)}")
    if combined is not None:
        if combined.dim() != 2 or combined.size(0) < B or combined.stride(1) != 1 or combined.size(1) < min_cols \
                or combined.stride(0) < combined.size(1):
            raise ValueError(f"combined must be [>={B}, >={min_cols}] with unit column stride, got "
                             f"{tuple(combined.shape)} strides {combined.stride()}")


def combined_for_launch(combined: Optional[torch.Tensor], B: int, n: int):
    """The tensor to hand to the C entry points as ``combined`` and the view to copy it back into afterwards (or
    None).  With 32 or more rows of x in fp16 / bf16 the GEMM kernels may keep their intermediate in ``combined``
    when its row stride has room for n rounded up to a multiple of 128, and then zero the columns between n and
    that width.  The C ABI describes the buffer by its stride alone; a column slice of a wider tensor whose own
    width ends before the padded one would have its parent's columns zeroed, so such a view goes through a
    contiguous stand-in of its own width (whose stride is too short for the padding, so nothing is written
    outside it)."""
    if combined is None or B < 32 or combined.dtype in (torch.float32, torch.float64):
        return combined, None
    padded = (int(n) + 127) // 128 * 128
    if combined.stride(0) == combined.size(1) or combined.size(1) >= padded:
        return combined, None
    return torch.empty(B, combined.size(1), dtype=combined.dtype, device=combined.device), combined[:B]


def mlp_forward_rows(x2: torch.Tensor, gate_rows: Optional[torch.Tensor], up_rows: torch.Tensor,
                     down_rows: torch.Tensor, n: int, n_dev: Optional[torch.Tensor], out: torch.Tensor,
                     combined: Optional[torch.Tensor], act: str, has_gate: bool, n_hint: int = 0,
                     workspace: Optional[torch.Tensor] = None) -> None:
    """Raw launch on packed rows: gate/up/down are [>=n, H] row-major, x2/out are [B, H].
    With ``n_dev`` (device int32 count) the kernels use min(*n_dev, n); ``n_hint`` is the count the host
    expects, used only to request rows before the device count has arrived."""
    dev = require_gpu(x2, gate_rows, up_rows, down_rows, out, combined, n_dev)
    if x2.dim() != 2:
        raise ValueError(f"x must be [B,H], got {tuple(x2.shape)}")
    B, H = x2.shape
    n = int(n)
    for name, t in (("gate_rows", gate_rows if has_gate else None), ("up_rows", up_rows), ("down_rows", down_rows)):
        if t is None:
            if name == "gate_rows" and has_gate:
                raise ValueError("has_gate=True needs gate_rows")
            continue
        if t.dim() != 2 or t.size(1) != H or t.size(0) < n or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous [>={n},{H}] tensor, got {tuple(t.shape)}")
        if t.dtype != x2.dtype:
            raise TypeError(f"{name} has dtype {t.dtype}, x is {x2.dtype}")
    if has_gate and gate_rows is None:
        raise ValueError("has_gate=True needs gate_rows")
    check_mlp_args(x2, out, combined, up_rows.dtype, dev, H, (2 if has_gate else 1) * n)
    if n_dev is not None and (n_dev.dtype != torch.int32 or n_dev.numel() < 1):
        raise TypeError("n_dev must be an int32 GPU tensor")
    need = mlp_workspace_bytes(B, H, n, x2.dtype)
    ws = mlp_workspace(dev, B, H, n, x2.dtype) if workspace is None else _check_workspace(workspace, dev, need)
    if act not in _lib.ACT_CODES:
        raise ValueError(f"unknown activation {act!r}; expected one of {sorted(_lib.ACT_CODES)}")
    combined, copy_back = combined_for_launch(combined, B, n)
    rc = _lib.lib().st_mlp_forward(
        x2.data_ptr(), B, H, gate_rows.data_ptr() if has_gate else None, up_rows.data_ptr(), down_rows.data_ptr(),
        n, n_dev.data_ptr() if n_dev is not None else None, int(n_hint), out.data_ptr(),
        combined.data_ptr() if combined is not None else None, combined.stride(0) if combined is not None else 0,
        ws.data_ptr(), ws.numel(), _lib.ACT_CODES[act], dtype_code(x2), int(bool(has_gate)), current_stream_ptr(dev))
    _lib.check(rc, "st_mlp_forward")
    if copy_back is not None:
        copy_back.copy_(combined)


_warned_layout = False


def sparse_mlp_forward(x: torch.Tensor, concat_weight: torch.Tensor, active_down_weight: torch.Tensor,
                       down_proj_buffer: torch.Tensor, combined_proj_buffer: torch.Tensor, act: str = "silu",
                       has_gate: bool = True) -> torch.Tensor:
    """out = (act(x @ Wg^T) * (x @ Wu^T)) @ Wd^T on the active rows.

    x: [..., H]; concat_weight: [2n, H] (gate rows then up rows; [n, H] when ``has_gate`` is False);
    active_down_weight: [H, n], normally the cache's transposed view with strides (1, H).
    ``down_proj_buffer`` is resized in place to [B, H] and returned viewed to x's shape (it aliases the
    result, as in the reference); ``combined_proj_buffer`` is resized to [B, concat_weight.size(0)] and
    left holding act(gate)*up in its first n columns.  Unlike sparse_mlp_op.cpp:157, ``act`` is honoured:
    "relu" reproduces that operator, "silu" reproduces src/modeling_skip.py:114-117.
    """
    global _warned_layout
    from .weight_cache import ConcatWeightHandle
    handle = concat_weight if isinstance(concat_weight, ConcatWeightHandle) and concat_weight._real is None else None
    if isinstance(concat_weight, ConcatWeightHandle) and handle is None:
        concat_weight = concat_weight.materialize()
    dev = require_gpu(x, concat_weight, active_down_weight, down_proj_buffer, combined_proj_buffer)
    H = x.shape[-1]
    rows = concat_weight.size(0)
    if has_gate and rows % 2:
        raise ValueError("concat_weight must hold gate rows followed by as many up rows")
    n = rows // 2 if has_gate else rows
    if concat_weight.dim() != 2 or concat_weight.size(1) != H:
        raise ValueError(f"concat_weight must be [rows, {H}], got {tuple(concat_weight.shape)}")
    if tuple(active_down_weight.shape) != (H, n):
        raise ValueError(f"active_down_weight must be [{H}, {n}], got {tuple(active_down_weight.shape)}")
    for name, t in (("concat_weight", concat_weight), ("active_down_weight", active_down_weight),
                    ("down_proj_buffer", down_proj_buffer), ("combined_proj_buffer", combined_proj_buffer)):
        if t.dtype != x.dtype:
            raise TypeError(f"{name} has dtype {t.dtype}, expected {x.dtype}")
    x2 = x.reshape(-1, H)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    B = x2.size(0)
    # [H, n] with strides (1, H) is a packed [n, H] buffer underneath
    if n > 0 and active_down_weight.stride() == (1, H):
        down_rows = active_down_weight.t()
    else:
        if not _warned_layout:
            warnings.warn("active_down_weight is not the cache's transposed [n,H] view; repacking it "
                          "(one extra device copy per call)")
            _warned_layout = True
        down_rows = active_down_weight.t().contiguous()
    if down_proj_buffer.dim() != 2 or down_proj_buffer.size(0) != B or down_proj_buffer.size(1) != H:
        down_proj_buffer.resize_(B, H)
    if combined_proj_buffer.dim() != 2 or combined_proj_buffer.size(0) != B or combined_proj_buffer.size(1) != rows:
        combined_proj_buffer.resize_(B, rows)
    if handle is not None:
        # the cache's own handle: its packed gate / up rows are read in place (no [2n,H] copy)
        cache = handle._cache
        if has_gate != cache.has_gate:
            raise ValueError("has_gate does not match the cache the concat weight comes from")
        if not handle.fresh():
            raise RuntimeError("concat_weight was fetched before the cache's last update; call get_concat_weight() again")
        gate_rows = cache.gate_active if has_gate else None
        up_rows = cache.up_active
    else:
        if not concat_weight.is_contiguous():
            concat_weight = concat_weight.contiguous()
        gate_rows = concat_weight[:n] if has_gate else None
        up_rows = concat_weight[n:] if has_gate else concat_weight
    mlp_forward_rows(x2, gate_rows, up_rows, down_rows, n, None, down_proj_buffer, combined_proj_buffer, act,
                     has_gate)
    return down_proj_buffer.view(x.shape) if x.dim() != 2 else down_proj_buffer


def predictor_mask(x: torch.Tensor, down_weight: torch.Tensor, up_weight: torch.Tensor, thr: float = 0.0,
                   ge: bool = True, return_scores: bool = False, out: Optional[torch.Tensor] = None,
                   t_ws: Optional[torch.Tensor] = None, scores_out: Optional[torch.Tensor] = None,
                   round_to_storage: bool = False):
    """mask[i] = any over rows b of ((x @ down^T) @ up^T)[b, i] >= thr  (``>`` when ``ge`` is False).

    x: [..., H]; down_weight: [r, H] (FastLoRAProjection.down.weight); up_weight: [I, r].
    Returns a bool[I] tensor (and the fp32 scores [B, I] when ``return_scores`` or ``scores_out`` is given;
    ``scores_out`` is a caller-owned buffer, for loops that must not allocate).
    thr = 0, ge = True is the reference's "naive" method (src/modeling_skip.py:206-207).
    ``round_to_storage``: round the rank-r intermediate and the scores to x's dtype before they are used, as the
    reference's two half-precision modules do (by default both stay in fp32).
    """
    dev = require_gpu(x, down_weight, up_weight, out)
    H = x.shape[-1]
    x2 = x.reshape(-1, H)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    B = x2.size(0)
    r, I = down_weight.size(0), up_weight.size(0)
    if tuple(down_weight.shape) != (r, H) or tuple(up_weight.shape) != (I, r):
        raise ValueError(f"predictor weights must be [r,{H}] and [I,r]; got {tuple(down_weight.shape)}, "
                         f"{tuple(up_weight.shape)}")
    if down_weight.dtype != x.dtype or up_weight.dtype != x.dtype:
        raise TypeError("predictor weights and x must share one dtype")
    down_weight = down_weight if down_weight.is_contiguous() else down_weight.contiguous()
    up_weight = up_weight if up_weight.is_contiguous() else up_weight.contiguous()
    if t_ws is None:
        t_ws = torch.empty(B, r, dtype=torch.float32, device=dev)
    elif t_ws.dtype != torch.float32 or t_ws.numel() < B * r or not t_ws.is_cuda:
        raise ValueError("t_ws must be a float32 GPU tensor with at least B*r elements")
    scores = None
    if scores_out is not None:
        if scores_out.dtype != torch.float32 or scores_out.numel() < B * I or not scores_out.is_cuda or \
                not scores_out.is_contiguous():
            raise ValueError("scores_out must be a contiguous float32 GPU tensor with at least B*I elements")
        scores = scores_out.view(-1)[:B * I].view(B, I)
    elif return_scores:
        scores = torch.empty(B, I, dtype=torch.float32, device=dev)
    mask = out if out is not None else torch.empty(I, dtype=torch.bool, device=dev)
    if mask.dtype != torch.bool or mask.numel() != I or not mask.is_contiguous():
        raise ValueError("out must be a contiguous bool[I] tensor")
    rc = _lib.lib().st_predictor_mask_ex(
        x2.data_ptr(), B, H, down_weight.data_ptr(), r, up_weight.data_ptr(), I, dtype_code(x2), float(thr), int(ge),
        1 if round_to_storage else 0, t_ws.data_ptr(), scores.data_ptr() if scores is not None else None,
        mask.data_ptr(), current_stream_ptr(dev))
    _lib.check(rc, "st_predictor_mask_ex")
    return (mask, scores) if (return_scores or scores_out is not None) else mask


def predictor_scores(x: torch.Tensor, down_weight: torch.Tensor, up_weight: torch.Tensor,
                     round_to_storage: bool = False) -> torch.Tensor:
    """fp32 scores [B, I] of the LoRA predictor (FastLoRAProjection.forward); with ``round_to_storage`` they hold
    values of x's dtype (see predictor_mask)."""
    return predictor_mask(x, down_weight, up_weight, 0.0, True, return_scores=True,
                          round_to_storage=round_to_storage)[1]


MASK_METHODS = {"topk": 0, "statistical_topk": 1}
_select_workspaces: dict = {}


def _select_workspace(device: torch.device, B: int, I: int) -> torch.Tensor:
    """Zero-initialised once; every call leaves the ticket word at the front zero again."""
    need = int(_lib.lib().st_mask_select_workspace_bytes(B, I))
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    ws = _select_workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.zeros(need, dtype=torch.uint8, device=device)
        _select_workspaces[key] = ws
    return ws


def select_workspace(device: torch.device, B: int, I: int) -> Optional[torch.Tensor]:
    """A workspace for ``mask_select`` with B rows (None for B = 1), zeroed as the first call needs it.  For
    callers that keep their own (one per stream of overlapping calls; allocate it outside graph capture)."""
    if B <= 1:
        return None
    return torch.zeros(int(_lib.lib().st_mask_select_workspace_bytes(B, I)), dtype=torch.uint8, device=device)


def mask_select(scores: torch.Tensor, method: str, k: int = 0, std_multiplier: float = 0.0,
                out: Optional[torch.Tensor] = None, return_cutoff: bool = False,
                workspace: Optional[torch.Tensor] = None):
    """Union over rows of the per-row selection on fp32 ``scores`` [B, I].

    ``topk``: the k largest scores of every row (src/modeling_skip.py:208-211; equal scores are taken in
    index order).  ``statistical_topk``: score > mean + std * std_multiplier with the population standard
    deviation (src/modeling_skip.py:197-202).  Returns bool[I] (and the per-row cutoffs [B] on request).
    """
    dev = require_gpu(scores, out)
    if method not in MASK_METHODS:
        raise ValueError(f"unknown sparsity method {method!r}")
    if scores.dim() != 2 or scores.dtype != torch.float32:
        raise ValueError("scores must be a float32 [B, I] tensor")
    scores = scores if scores.is_contiguous() else scores.contiguous()
    B, I = scores.shape
    mask = out if out is not None else torch.empty(I, dtype=torch.bool, device=dev)
    if mask.dtype != torch.bool or mask.numel() != I or not mask.is_contiguous():
        raise ValueError("out must be a contiguous bool[I] tensor")
    cutoff = torch.empty(B, dtype=torch.float32, device=dev) if return_cutoff else None
    ws = None
    if B > 1:
        ws = workspace if workspace is not None else _select_workspace(dev, B, I)
        if ws.dtype != torch.uint8 or not ws.is_cuda:
            raise ValueError("workspace must be a uint8 GPU tensor (see select_workspace)")
    rc = _lib.lib().st_mask_select(
        scores.data_ptr(), B, I, MASK_METHODS[method], int(k), float(std_multiplier), mask.data_ptr(),
        cutoff.data_ptr() if cutoff is not None else None, ws.data_ptr() if ws is not None else None,
        ws.numel() if ws is not None else 0, current_stream_ptr(dev))
    _lib.check(rc, "st_mask_select")
    return (mask, cutoff) if return_cutoff else mask


def approx_topk_threshold(scores: torch.Tensor, k: int) -> torch.Tensor:
    """Per-row approximate top-k threshold [B, 1] from four max-sketches
    (sparse_transformers/csrc/approx_topk.h:10-88).  ``scores`` is a float32 or float64 [B, F] GPU tensor; the
    threshold has its dtype (the reference dispatches on the scores' type, :33)."""
    dev = require_gpu(scores)
    if scores.dim() != 2:
        raise RuntimeError("Input scores must be 2D tensor [batch_size, features]")
    if scores.dtype not in (torch.float32, torch.float64):
        raise TypeError("approx_topk_threshold: scores must be float32 or float64")
    if k <= 0:
        raise RuntimeError("k must be positive")
    if k > scores.size(1):
        raise RuntimeError("k cannot be larger than feature size")
    scores = scores if scores.is_contiguous() else scores.contiguous()
    B, F = scores.shape
    thr = torch.empty(B, 1, dtype=scores.dtype, device=dev)
    fn = _lib.lib().st_approx_topk_threshold if scores.dtype == torch.float32 else _lib.lib().st_approx_topk_threshold_f64
    rc = fn(scores.data_ptr(), B, F, int(k), thr.data_ptr(), current_stream_ptr(dev))
    _lib.check(rc, "st_approx_topk_threshold")
    return thr
