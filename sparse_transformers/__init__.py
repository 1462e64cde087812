"""Import-name compatibility: `from sparse_transformers import WeightCache` (as src/modeling_skip.py:23 of
NimbleEdge/sparse_transformers does) resolves to the MI355X implementation in `sparse_transformers_amd`.
Unlike the reference's package, importing this one changes no global thread or JIT settings."""
from sparse_transformers_amd import WeightCache, approx_topk_threshold, sparse_mlp_forward  # noqa: F401

# the reference registers approx_topk_threshold (sparse_mlp_op.cpp:208) but keeps its re-export commented out
# (sparse_transformers/__init__.py:29-33); it is offered here under the same name
__all__ = ["WeightCache", "sparse_mlp_forward", "approx_topk_threshold"]
