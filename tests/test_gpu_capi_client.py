"""The C ABI used without torch: tests/capi/capi_client.cpp links only the library and the HIP runtime,
allocates its buffers with hipMalloc and checks cache order, MLP output, the fused call, the empty-mask
error, the predictor mask and top-k against loops of its own.  The binary is built by
`python -m sparse_transformers_amd.build` (in-tree, beside its source)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
EXE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "capi", "capi_client")


def test_c_abi_client_without_torch():
    if not os.path.exists(EXE):
        pytest.fail(f"{EXE} not built: run python -m sparse_transformers_amd.build")
    run = subprocess.run([EXE], capture_output=True, text=True, timeout=100)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "capi_client: OK" in run.stdout
