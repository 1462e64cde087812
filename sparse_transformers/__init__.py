"""Import-name compatibility: `from sparse_transformers import WeightCache` (as src/modeling_skip.py:23 of
NimbleEdge/sparse_transformers does) resolves to the MI355X implementation in `sparse_transformers_amd`.
Unlike the reference's package, importing this one changes no global thread or JIT settings."""
from sparse_transformers_amd import WeightCache, sparse_mlp_forward  # noqa: F401

__all__ = ["WeightCache", "sparse_mlp_forward"]
