"""The C-ABI library loads and exports every symbol include/sparse_mlp_amd.h declares; argument
validation works without touching a GPU.  No compute calls here."""
import ctypes as C
import os
import re

import pytest

from sparse_transformers_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "sparse_mlp_amd.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(st_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 14 and "st_mlp_forward" in names and "st_cache_update_async" in names
    L = _lib.lib()
    for name in names:
        assert hasattr(L, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes signature table and header disagree"


def test_header_cites_reference_interfaces():
    text = open(HEADER).read()
    for cite in ("sparse_mlp_op.cpp:53-76", "weight_cache.h:229-359", "src/modeling_skip.py:52-53"):
        assert cite in text


def test_version_and_limits():
    L = _lib.lib()
    assert L.st_version() >= 1
    assert 14336 <= L.st_cache_max_intermediate() < 65535


def test_argument_validation_without_gpu():
    L = _lib.lib()
    # null pointers / bad shapes are rejected before any HIP call
    rc = L.st_mlp_forward(None, 1, 64, None, None, None, 4, None, 0, None, None, 0, None, 0, 1, 0, 1, None)
    assert rc == _lib.ST_ERR_ARG and "null" in _lib.last_error()
    rc = L.st_predictor_mask(None, 1, 64, None, 8, None, 16, 0, 0.0, 1, None, None, None, None)
    assert rc == _lib.ST_ERR_ARG
    assert not L.st_cache_create(None, 16, 8, 0, 1)
    bufs = _lib.CacheBuffers()
    assert not L.st_cache_create(C.byref(bufs), 10 ** 6, 8, 0, 1)
    assert "range" in _lib.last_error()
    with pytest.raises(ValueError):
        _lib.check(_lib.ST_ERR_ARG, "x")
    with pytest.raises(RuntimeError, match="No active weights"):
        _lib.check(_lib.ST_ERR_NO_ACTIVE, "x")
    with pytest.raises(RuntimeError, match="Cache is not valid"):
        _lib.check(_lib.ST_ERR_INVALID, "x")
