"""Shared fixtures.  `-m "not gpu"` runs on a CPU-only box: the oracle against its golden vectors,
host logic, and the C-ABI export check.  `-m gpu` tests are the parity tests proper: HIP path vs the
oracle on the same seeded inputs, called through the C ABI."""
import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _gpu_available() -> bool:
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def golden_traces():
    with open(os.path.join(GOLDEN, "cache_traces.json")) as f:
        return json.load(f)["traces"]


@pytest.fixture(scope="session")
def golden_mlp():
    with open(os.path.join(GOLDEN, "mlp_forward.json")) as f:
        return json.load(f)["cases"]


def bits_to_mask(s: str) -> np.ndarray:
    return np.frombuffer(s.encode(), dtype=np.uint8) == ord("1")


def golden_weights(I: int, H: int):
    """The recognisable weights tests/golden/make_golden.py used for the cache traces."""
    gate = (np.arange(I * H, dtype=np.float32).reshape(I, H) + 0.25)
    up = -(np.arange(I * H, dtype=np.float32).reshape(I, H) + 0.5)
    down = (np.arange(H * I, dtype=np.float32).reshape(H, I) * 2.0 + 1.0)
    return gate, up, down


def round_to(a: np.ndarray, dtype: str) -> np.ndarray:
    """Round float32 data to the storage type and back (what the GPU kernels actually read)."""
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32))
    return t.to(getattr(torch, dtype)).to(torch.float32).numpy()


# tolerances of the north star: fp32 1e-5 relative; fp16/bf16 2e-2 absolute / 1e-2 relative
TOL = {"float32": dict(rtol=1e-5, atol_rel=1e-5), "float16": dict(rtol=1e-2, atol=2e-2),
       "bfloat16": dict(rtol=1e-2, atol=2e-2),
       # double precision against a float64 library evaluation: summation order only
       "float64": dict(rtol=1e-12, atol_rel=1e-12)}


def assert_close(got: np.ndarray, want: np.ndarray, dtype: str, what: str = ""):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    t = TOL[dtype]
    scale = float(np.max(np.abs(want))) if want.size else 0.0
    atol = t.get("atol", t.get("atol_rel", 0.0) * max(scale, 1e-30))
    err = np.abs(got - want)
    bad = err > atol + t["rtol"] * np.abs(want)
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.size} outside tolerance; max err {err.max():.3e}, scale {scale:.3e}"
