"""Host-side mirror of the reference's callers of the sparse-MLP path.

  * ``FastLoRAProjection`` — src/modeling_skip.py:32-53 (the importance predictor's two bias-free maps)
  * ``SkipMLP`` / ``OPTSkipMLP`` — src/modeling_skip.py:55-128, src/models/opt/modelling_opt_skip.py:60-119
    (``nn.Module`` with the reference's sub-modules and buffers, ``initialize_weight_cache``, ``reset_cache``)
  * ``SparseDecodeLayer`` / ``SparseMLPStack`` — the per-layer order of SkipDecoderLayer.forward
    (src/modeling_skip.py:204-219,234-261): predictor -> mask -> union -> cache update -> sparse MLP,
    without attention or normalisation, which are outside this path.

No HuggingFace dependency.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from .ops import (mask_select, mlp_workspace_bytes, predictor_mask, predictor_scores, select_workspace,
                  sparse_mlp_forward)
from .weight_cache import WeightCache


class FastLoRAProjection:
    """scores = (x @ down.weight^T) @ up.weight^T with down.weight [r,H], up.weight [I,r]."""

    def __init__(self, down_weight: torch.Tensor, up_weight: torch.Tensor, round_to_storage: bool = False):
        """``round_to_storage``: round the rank-r intermediate and the scores to the weights' dtype, as the reference's
        ``up(down(x))`` does when the model runs in fp16 / bf16 (default: both stay in fp32)."""
        self.down_weight = down_weight.contiguous()
        self.up_weight = up_weight.contiguous()
        self.round_to_storage = bool(round_to_storage)
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
        return predictor_scores(x, self.down_weight, self.up_weight, self.round_to_storage)

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
            return predictor_mask(x, self.down_weight, self.up_weight, 0.0, True, out=out, t_ws=t_ws,
                                  round_to_storage=self.round_to_storage)
        if method == "threshold":
            return predictor_mask(x, self.down_weight, self.up_weight, thr, ge, out=out, t_ws=t_ws,
                                  round_to_storage=self.round_to_storage)
        if method not in ("topk", "statistical_topk"):
            raise ValueError(f"unknown sparsity method {method!r}")
        if scores_ws is None:
            scores = self.forward(x)
        else:   # caller-owned buffers: nothing is allocated (what a captured decode loop needs)
            scores = predictor_mask(x, self.down_weight, self.up_weight, 0.0, True, out=out, t_ws=t_ws,
                                    scores_out=scores_ws, round_to_storage=self.round_to_storage)[1]
        return mask_select(scores, method, k=k, std_multiplier=std_multiplier, out=out, workspace=select_ws)


def load_predictors(directory: str, num_layers: int, lora_pct: float, device=None, dtype=None) -> List["FastLoRAProjection"]:
    """The per-layer predictors of a trained model, from the directory the reference's trainer writes
    (consumed by benchmark.py:460-468 in the reference)."""
    import os

    return [FastLoRAProjection.from_file(os.path.join(directory, FastLoRAProjection.checkpoint_name(l, lora_pct)),
                                         device=device, dtype=dtype) for l in range(num_layers)]


_TORCH_ACTS = {
    "relu": torch.relu,
    "silu": torch.nn.functional.silu,
    "gelu_pytorch_tanh": lambda v: torch.nn.functional.gelu(v, approximate="tanh"),
    "sigmoid": torch.sigmoid,
    "identity": lambda v: v,
}


class SkipMLP(torch.nn.Module):
    """Drop-in for the reference's ``SkipMLP`` (src/modeling_skip.py:55-128) and, with ``has_gate=False``, for
    ``OPTSkipMLP`` (src/models/opt/modelling_opt_skip.py:60-119): same constructor arguments, the same
    sub-modules ``gate_proj`` / ``up_proj`` / ``down_proj`` (bias-free by default) and registered buffers
    ``init_mask``, ``down_proj_buffer``, ``combined_proj_buffer`` -- so a checkpoint of the reference loads
    with ``load_state_dict`` -- and the same methods.

    ``forward(x, use_sparse=True)`` runs the HIP decode kernels on the cache's packed rows
    (``WeightCache.forward``: no host read-back, no ``[2n,H]`` copy).  The reference's own sparse forward
    multiplies ``x`` with ``get_concat_weight()`` in torch (src/modeling_skip.py:114-117) and therefore never
    reaches ``sparse_mlp_forward``; replacing the module is what puts the kernels on the path.
    ``use_sparse=False`` is the dense MLP in torch, which is what the reference runs for prefill.
    Like the reference's cache path, the sparse forward ignores biases.

    ``lazy_cache_updates`` (class attribute, default True): the module's cache only remembers the mask handed to
    ``weight_cache.update_active_weights`` -- the decoder layer's call, made before attention
    (src/modeling_skip.py:217,235-238) -- and applies it together with this module's forward as one fused
    update + MLP launch.  The price: an update that leaves nothing active is reported by the next synchronising
    call instead of by ``update_active_weights``.  Set it to False for the reference's timing of that error."""

    lazy_cache_updates = True

    def __init__(self, hidden_size: int, intermediate_size: int, sparsity: float, bias: bool = False,
                 act_fn: str = "silu", use_weight_cache: bool = True, has_gate: bool = True):
        super().__init__()
        if act_fn not in _TORCH_ACTS:
            raise ValueError(f"unknown activation {act_fn!r}; expected one of {sorted(_TORCH_ACTS)}")
        self.has_gate = bool(has_gate)
        if self.has_gate:
            self.gate_proj = torch.nn.Linear(hidden_size, intermediate_size, bias=bias)
        self.up_proj = torch.nn.Linear(hidden_size, intermediate_size, bias=bias)
        self.down_proj = torch.nn.Linear(intermediate_size, hidden_size, bias=bias)
        self.sparsity = sparsity
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.act_fn_name = act_fn
        self.act_fn = _TORCH_ACTS[act_fn]
        self.use_weight_cache = use_weight_cache
        self.weight_mask: Optional[torch.Tensor] = None      # only used by the cache-less debugging forward
        self.weight_cache: Optional[WeightCache] = None
        self.register_buffer("init_mask", torch.ones(self.intermediate_size, dtype=torch.bool))
        cols = (2 if self.has_gate else 1) * int(self.intermediate_size * sparsity)
        self.register_buffer("down_proj_buffer", torch.zeros(1, self.hidden_size))
        self.register_buffer("combined_proj_buffer", torch.zeros(1, max(cols, 1)))

    @classmethod
    def from_weights(cls, gate_weight: Optional[torch.Tensor], up_weight: torch.Tensor, down_weight: torch.Tensor,
                     sparsity: float = 0.5, act_fn: str = "silu", has_gate: bool = True) -> "SkipMLP":
        """The module around existing weight tensors (gate/up [I,H], down [H,I]); device and dtype follow them."""
        I, H = up_weight.shape
        with torch.device("meta"):
            m = cls(H, I, sparsity, False, act_fn, True, has_gate)
        m = m.to_empty(device=up_weight.device).to(up_weight.dtype)
        with torch.no_grad():
            if has_gate:
                m.gate_proj.weight.copy_(gate_weight)
            m.up_proj.weight.copy_(up_weight)
            m.down_proj.weight.copy_(down_weight)
            m.init_mask.fill_(True)
            m.down_proj_buffer.zero_()
            m.combined_proj_buffer.zero_()
        return m

    def initialize_weight_cache(self) -> None:
        """Builds the cache from the current weights (they are copied), all rows active: called once the weights
        are loaded and the module sits on its GPU, as the reference does from ``post_init``."""
        if self.weight_cache is None and self.use_weight_cache:
            self.weight_cache = WeightCache(self.init_mask, self.hidden_size,
                                            self.gate_proj.weight if self.has_gate else None, self.up_proj.weight,
                                            self.down_proj.weight, self.has_gate)
            self.weight_cache.lazy_updates = bool(self.lazy_cache_updates)

    def reset_cache(self) -> None:
        """What the reference's model-level ``reset_cache`` does per layer (src/modeling_skip.py:492-497): drop
        the cache and build a fresh one (every row active, order 0..I-1)."""
        self.weight_cache = None
        self.initialize_weight_cache()

    def _apply(self, fn, *args, **kwargs):
        # .to() / .half() / .cuda(): parameters and the registered buffers move with the module; a cache built
        # on the old device or dtype no longer matches them and has to be rebuilt
        out = super()._apply(fn, *args, **kwargs)
        wc = self.weight_cache
        if wc is not None and (wc.device != self.up_proj.weight.device or wc.dtype != self.up_proj.weight.dtype):
            self.weight_cache = None
        return out

    def forward(self, x: torch.Tensor, use_sparse: bool = True) -> torch.Tensor:
        if not use_sparse:
            return self._forward_dense(x)
        if self.use_weight_cache:
            return self._forward_sparse_weight_cache(x)
        return self._forward_sparse_no_cache(x)

    def _forward_sparse_weight_cache(self, x: torch.Tensor) -> torch.Tensor:
        wc = self.weight_cache
        if wc is None:
            raise RuntimeError("call initialize_weight_cache() first")
        return wc.forward(x, self.act_fn_name)

    def _forward_sparse_no_cache(self, x: torch.Tensor) -> torch.Tensor:
        up = self.up_proj(x)
        h = self.act_fn(self.gate_proj(x)) * up if self.has_gate else self.act_fn(up)
        if self.weight_mask is not None:
            h = h * self.weight_mask
        return self.down_proj(h)

    def _forward_dense(self, x: torch.Tensor) -> torch.Tensor:
        up = self.up_proj(x)
        return self.down_proj(self.act_fn(self.gate_proj(x)) * up if self.has_gate else self.act_fn(up))


class OPTSkipMLP(SkipMLP):
    """The ungated variant (src/models/opt/modelling_opt_skip.py:60-119): ``up_proj`` / ``down_proj`` only,
    ReLU by default."""

    def __init__(self, hidden_size: int, intermediate_size: int, sparsity: float, bias: bool = False,
                 act_fn: str = "relu", use_weight_cache: bool = True):
        super().__init__(hidden_size, intermediate_size, sparsity, bias, act_fn, use_weight_cache, has_gate=False)


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
