"""Host-side mirror of the reference's callers of the sparse-MLP path.

  * ``FastLoRAProjection`` — src/modeling_skip.py:32-53 (the importance predictor's two bias-free maps)
  * ``SkipMLP``            — src/modeling_skip.py:55-128 (buffers, ``initialize_weight_cache``, sparse forward)
  * ``SparseDecodeLayer`` / ``SparseMLPStack`` — the per-layer order of SkipDecoderLayer.forward
    (src/modeling_skip.py:204-219,234-261): predictor -> mask -> union -> cache update -> sparse MLP,
    without attention or normalisation, which are outside this path.

No HuggingFace dependency; parameters are plain tensors on the GPU.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from .ops import (mask_select, mlp_workspace_bytes, predictor_mask, predictor_scores, select_workspace,
                  sparse_mlp_forward)
from .weight_cache import WeightCache


class FastLoRAProjection:
    """scores = (x @ down.weight^T) @ up.weight^T with down.weight [r,H], up.weight [I,r]."""

    def __init__(self, down_weight: torch.Tensor, up_weight: torch.Tensor):
        self.down_weight = down_weight.contiguous()
        self.up_weight = up_weight.contiguous()
        self.lora_size, self.hidden_size = self.down_weight.shape
        self.intermediate_size = self.up_weight.size(0)

    @classmethod
    def from_state_dict(cls, sd: dict, device=None, dtype=None) -> "FastLoRAProjection":
        """Accepts the reference's predictor checkpoints: keys ``down.weight`` and ``up.weight``
        (src/trainer.py:570-585)."""
        d, u = sd["down.weight"], sd["up.weight"]
        return cls(d.to(device=device, dtype=dtype), u.to(device=device, dtype=dtype))

    @classmethod
    def from_file(cls, path: str, device=None, dtype=None) -> "FastLoRAProjection":
        """One trained predictor as the reference's trainer saves it (``torch.save(state_dict)``,
        src/trainer.py:570-585).  Loaded with ``weights_only=True``: nothing in the file is executed."""
        sd = torch.load(path, map_location="cpu", weights_only=True)
        return cls.from_state_dict(sd, device=device, dtype=dtype)

    @staticmethod
    def checkpoint_name(layer_idx: int, lora_pct: float) -> str:
        """File name the reference gives layer ``layer_idx``'s final predictor (src/trainer.py:573,904)."""
        return f"final_predictor_layer_{layer_idx}_lora_{lora_pct:.1f}pct.pt"

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return predictor_scores(x, self.down_weight, self.up_weight)

    __call__ = forward

    def mask(self, x: torch.Tensor, method: str = "naive", thr: float = 0.0, ge: bool = True, k: int = 0,
             std_multiplier: float = 0.0, out: Optional[torch.Tensor] = None,
             t_ws: Optional[torch.Tensor] = None, scores_ws: Optional[torch.Tensor] = None,
             select_ws: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Union-over-rows boolean mask, src/modeling_skip.py:204-214.

        ``naive`` (score >= 0) and ``threshold`` (score >= thr, or > thr) are fused into the predictor
        kernel.  ``topk`` and ``statistical_topk`` need a statistic of the whole row: the predictor kernel
        leaves its fp32 scores and a selection kernel (one block per row) finishes.  ``scores_ws`` (float32,
        B*I elements) and, for several rows, ``select_ws`` (``ops.select_workspace``) make the call
        allocation-free.
        """
        if method == "naive":
            return predictor_mask(x, self.down_weight, self.up_weight, 0.0, True, out=out, t_ws=t_ws)
        if method == "threshold":
            return predictor_mask(x, self.down_weight, self.up_weight, thr, ge, out=out, t_ws=t_ws)
        if method not in ("topk", "statistical_topk"):
            raise ValueError(f"unknown sparsity method {method!r}")
        if scores_ws is None:
            scores = self.forward(x)
        else:   # caller-owned buffers: nothing is allocated (what a captured decode loop needs)
            scores = predictor_mask(x, self.down_weight, self.up_weight, 0.0, True, out=out, t_ws=t_ws,
                                    scores_out=scores_ws)[1]
        return mask_select(scores, method, k=k, std_multiplier=std_multiplier, out=out, workspace=select_ws)


def load_predictors(directory: str, num_layers: int, lora_pct: float, device=None, dtype=None) -> List["FastLoRAProjection"]:
    """The per-layer predictors of a trained model, from the directory the reference's trainer writes
    (consumed by benchmark.py:460-468 in the reference)."""
    import os

    return [FastLoRAProjection.from_file(os.path.join(directory, FastLoRAProjection.checkpoint_name(l, lora_pct)),
                                         device=device, dtype=dtype) for l in range(num_layers)]


class SkipMLP:
    """Gated (or ungated) MLP whose decode path runs on the differential weight cache."""

    def __init__(self, gate_weight: Optional[torch.Tensor], up_weight: torch.Tensor, down_weight: torch.Tensor,
                 sparsity: float = 0.5, act_fn: str = "silu", has_gate: bool = True):
        self.gate_weight, self.up_weight, self.down_weight = gate_weight, up_weight, down_weight
        self.intermediate_size, self.hidden_size = up_weight.shape
        self.sparsity = sparsity
        self.act_fn_name = act_fn
        self.has_gate = has_gate
        dev, dt = up_weight.device, up_weight.dtype
        self.init_mask = torch.ones(self.intermediate_size, dtype=torch.bool, device=dev)
        self.weight_cache: Optional[WeightCache] = None
        cols = (2 if has_gate else 1) * int(self.intermediate_size * sparsity)
        self.down_proj_buffer = torch.zeros(1, self.hidden_size, dtype=dt, device=dev)
        self.combined_proj_buffer = torch.zeros(1, max(cols, 1), dtype=dt, device=dev)

    def initialize_weight_cache(self) -> None:
        if self.weight_cache is None:
            self.weight_cache = WeightCache(self.init_mask, self.hidden_size, self.gate_weight, self.up_weight,
                                            self.down_weight, self.has_gate)

    def reset_cache(self) -> None:
        """Back to the all-ones mask of a fresh cache (every row active, order 0..I-1)."""
        self.weight_cache = None
        self.initialize_weight_cache()

    def forward(self, x: torch.Tensor, use_sparse: bool = True) -> torch.Tensor:
        if not use_sparse:
            raise NotImplementedError("the dense (prefill) MLP is outside this package's path")
        wc = self.weight_cache
        if wc is None:
            raise RuntimeError("call initialize_weight_cache() first")
        return sparse_mlp_forward(x, wc.get_concat_weight(), wc.get_active_down_weight(), self.down_proj_buffer,
                                  self.combined_proj_buffer, self.act_fn_name, self.has_gate)

    __call__ = forward


class SparseDecodeLayer:
    """predictor -> mask -> cache update -> sparse MLP for one layer, all stream-ordered."""

    def __init__(self, predictor: FastLoRAProjection, cache: WeightCache, act: str = "silu", thr: float = 0.0,
                 ge: bool = True, method: str = "threshold", k: int = 0, std_multiplier: float = 0.0):
        """``method`` is one of SkipDecoderLayer's sparsity methods (src/modeling_skip.py:204-213): "naive",
        "topk" (``k`` per row), "statistical_topk" (``std_multiplier`` = Normal(0,1).icdf(sparsity)), or
        "threshold" (score >= ``thr``; ``ge=False`` for a strict comparison)."""
        if method not in ("naive", "threshold", "topk", "statistical_topk"):
            raise ValueError(f"unknown sparsity method {method!r}")
        self.predictor, self.cache, self.act, self.thr, self.ge = predictor, cache, act, thr, ge
        self.method, self.k, self.std_multiplier = method, k, std_multiplier
        self.mask = torch.zeros(cache.intermediate_size, dtype=torch.bool, device=cache.device)
        self._scores_ws: Optional[torch.Tensor] = None
        self._select_ws: Optional[torch.Tensor] = None

    @classmethod
    def from_sparsity(cls, predictor: FastLoRAProjection, cache: WeightCache, sparsity: float,
                      sparsity_method: str = "naive", act: str = "silu") -> "SparseDecodeLayer":
        """The layer as SkipDecoderLayer.__init__ configures it from ``config.sparsities[layer_idx]``
        (src/modeling_skip.py:138-143): "statistical_topk" takes its multiplier from the inverse normal CDF
        at ``sparsity``; "topk" keeps ``int(hidden_size * (1 - sparsity))`` scores per row -- the reference
        sets ``self.intermediate_size = config.hidden_size`` (:134), so the count follows the hidden size."""
        k, z = 0, 0.0
        if sparsity_method == "statistical_topk":
            z = float(torch.distributions.normal.Normal(0, 1).icdf(torch.tensor(float(sparsity))))
        elif sparsity_method == "topk":
            k = int(cache.hidden_size * (1 - sparsity))
        return cls(predictor, cache, act=act, method=sparsity_method, k=k, std_multiplier=z)

    def predict_mask(self, x_pred: torch.Tensor, t_ws: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The layer's mask for ``x_pred`` into ``self.mask``.  The buffers the row-statistic methods need are
        created on the first call with a given batch size (so: before a graph capture, not inside one)."""
        if self.method in ("topk", "statistical_topk"):
            B, I = x_pred.reshape(-1, x_pred.shape[-1]).size(0), self.cache.intermediate_size
            if self._scores_ws is None or self._scores_ws.numel() < B * I:
                self._scores_ws = torch.empty(B * I, dtype=torch.float32, device=self.cache.device)
                self._select_ws = select_workspace(self.cache.device, B, I)
        return self.predictor.mask(x_pred, self.method, self.thr, self.ge, k=self.k,
                                   std_multiplier=self.std_multiplier, out=self.mask, t_ws=t_ws,
                                   scores_ws=self._scores_ws, select_ws=self._select_ws)

    def compute_mask_and_update(self, x_pred: torch.Tensor, mask_override: Optional[torch.Tensor] = None,
                                t_ws: Optional[torch.Tensor] = None) -> None:
        self.predict_mask(x_pred, t_ws)
        self.cache.update_active_weights_async(self.mask if mask_override is None else mask_override)

    def mlp(self, x: torch.Tensor, out: Optional[torch.Tensor] = None,
            workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
        return self.cache.forward(x, self.act, out=out, workspace=workspace)

    def step(self, x_pred: torch.Tensor, x: torch.Tensor, mask_override: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None, t_ws: Optional[torch.Tensor] = None,
             workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Predictor mask, then cache update and MLP in one call (``WeightCache.update_and_forward``)."""
        self.predict_mask(x_pred, t_ws)
        return self.cache.update_and_forward(self.mask if mask_override is None else mask_override, x, self.act,
                                             out=out, workspace=workspace)


class SparseMLPStack:
    """A stack of sparse layers stepped one token at a time (the decode loop of the reference,
    src/modeling_skip.py:383-402, restricted to the sparse-MLP path)."""

    def __init__(self, layers: Sequence[SparseDecodeLayer]):
        self.layers: List[SparseDecodeLayer] = list(layers)

    # ---- staged / graph-replayed stepping: fixed device buffers, no allocation, no host reads ----
    def prepare(self, batch: int, overlap: bool = False, fused: bool = True) -> None:
        c0 = self.layers[0].cache
        dev, dt, H, I = c0.device, c0.dtype, c0.hidden_size, c0.intermediate_size
        L = len(self.layers)
        self.x_stage = torch.empty(batch, H, dtype=dt, device=dev)
        self.xp_stage = torch.empty(L, batch, H, dtype=dt, device=dev)
        self.mask_stage = torch.empty(L, I, dtype=torch.bool, device=dev)
        self._pingpong = [torch.empty(batch, H, dtype=dt, device=dev) for _ in range(2)]
        rmax = max(layer.predictor.lora_size for layer in self.layers)
        self._t_ws = torch.empty(batch * rmax, dtype=torch.float32, device=dev)
        # the stack owns its MLP scratch: a captured step keeps this address, whatever other callers do later
        self._mlp_ws = torch.empty(mlp_workspace_bytes(batch, H, I), dtype=torch.uint8, device=dev)
        self.out = self._pingpong[0]
        self.graph = None
        self.use_trace_masks = True
        self.overlap = overlap
        self.fused = fused and not overlap   # update + MLP as one call per layer
        self._side = torch.cuda.Stream(device=dev) if overlap else None   # default priority
        self._ev_fork = torch.cuda.Event()
        self._ev_upd = [torch.cuda.Event() for _ in range(L)]

    def _enqueue(self) -> None:
        """One decode step.  With ``overlap`` the predictor + cache update of every layer run on a side
        stream (they depend on the staged predictor inputs / masks only, as in the reference where the
        mask is computed from the pre-attention state, src/modeling_skip.py:235-238) and each layer's
        MLP waits for its own update; the two streams join at the end of the step."""
        x = self.x_stage
        main = torch.cuda.current_stream(self.x_stage.device)
        side = self._side if self.overlap else None
        if side is not None:
            self._ev_fork.record(main)
            side.wait_event(self._ev_fork)
        for l, layer in enumerate(self.layers):
            mask = self.mask_stage[l] if self.use_trace_masks else None
            if self.fused:
                out = self._pingpong[l & 1]
                layer.step(self.xp_stage[l], x, mask, out=out, t_ws=self._t_ws, workspace=self._mlp_ws)
                x = out
                continue
            if side is not None:
                with torch.cuda.stream(side):
                    layer.compute_mask_and_update(self.xp_stage[l], mask, t_ws=self._t_ws)
                    self._ev_upd[l].record(side)
                main.wait_event(self._ev_upd[l])
            else:
                layer.compute_mask_and_update(self.xp_stage[l], mask, t_ws=self._t_ws)
            out = self._pingpong[l & 1]
            layer.cache.forward(x, layer.act, out=out, workspace=self._mlp_ws)
            x = out
        self.out = x

    def capture(self) -> None:
        """Record one decode step into a HIP graph (call after at least one eager step)."""
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self._enqueue()
        self.graph = g

    def step_staged(self, x: torch.Tensor, x_pred: torch.Tensor, masks: Optional[torch.Tensor] = None,
                    replay: bool = False) -> torch.Tensor:
        """x [B,H], x_pred [L,B,H], masks bool [L,I] (trace-driven cache masks; ignored when
        ``use_trace_masks`` is False).  Copies the inputs into the staging buffers and either replays
        the captured graph or launches the kernels eagerly."""
        self.x_stage.copy_(x)
        self.xp_stage.copy_(x_pred)
        if masks is not None:
            self.mask_stage.copy_(masks)
        if replay:
            self.graph.replay()
            for layer in self.layers:
                layer.cache._dirty = True
        else:
            self._enqueue()
        return self.out

    def decode_step(self, x: torch.Tensor, x_pred: Optional[Sequence[torch.Tensor]] = None,
                    mask_override: Optional[Sequence[torch.Tensor]] = None) -> torch.Tensor:
        """x: [B,H].  Layer l's predictor sees ``x_pred[l]`` (default: the layer's own input), its MLP
        sees the previous layer's output."""
        for l, layer in enumerate(self.layers):
            xp = x if x_pred is None else x_pred[l]
            x = layer.step(xp, x, None if mask_override is None else mask_override[l])
        return x
