"""MI355X-native sparse-MLP decode path (LoRA predictor -> mask -> differential weight cache ->
fused gate/up/activation/down) behind the operator API of NimbleEdge/sparse_transformers.

Unlike the reference's ``sparse_transformers/__init__.py`` nothing global is changed at import
(no thread-count or JIT settings).  The HIP library is loaded on first use and there is no CPU
fallback: without the built library, or without a GPU tensor, calls raise.
"""
from .ops import approx_topk_threshold, mask_select, predictor_mask, predictor_scores, sparse_mlp_forward
from .skip_mlp import FastLoRAProjection, OPTSkipMLP, SkipMLP, SparseDecodeLayer, SparseMLPStack, load_predictors
from .weight_cache import WeightCache

__all__ = [
    "sparse_mlp_forward",
    "WeightCache",
    "predictor_mask",
    "predictor_scores",
    "mask_select",
    "approx_topk_threshold",
    "FastLoRAProjection",
    "SkipMLP",
    "OPTSkipMLP",
    "SparseDecodeLayer",
    "SparseMLPStack",
    "load_predictors",
]
