"""The entry point that allocates nothing (st_mlp_forward_static, scratch inside the library image) against
st_mlp_forward with a caller workspace: same kernels, so the outputs must agree bit for bit.  Two calls in a row,
the second on a smaller input, so that whatever the first call left in the shared scratch is still there."""
import numpy as np
import pytest
import torch

import oracle
from sparse_transformers_amd import _lib
from conftest import assert_close, round_to

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _call(static, x, gate, up, down, n, act, has_gate, comb=None):
    L = _lib.lib()
    B, H = x.shape
    out = torch.full((B, H), float("nan"), dtype=x.dtype, device=DEV)
    code = {torch.float32: _lib.ST_F32, torch.float16: _lib.ST_F16, torch.bfloat16: _lib.ST_BF16}[x.dtype]
    stream = torch.cuda.current_stream().cuda_stream
    common = (x.data_ptr(), B, H, gate.data_ptr() if has_gate else None, up.data_ptr(), down.data_ptr(), n, None, 0,
              out.data_ptr(), comb.data_ptr() if comb is not None else None, comb.stride(0) if comb is not None else 0)
    if static:
        rc = L.st_mlp_forward_static(*common, _lib.ACT_CODES[act], code, int(has_gate), stream)
    else:
        ws = torch.empty(int(L.st_mlp_workspace_bytes(B, H, n)), dtype=torch.uint8, device=DEV)
        rc = L.st_mlp_forward(*common, ws.data_ptr(), ws.numel(), _lib.ACT_CODES[act], code, int(has_gate), stream)
    _lib.check(rc, "st_mlp_forward_static" if static else "st_mlp_forward")
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype,H", [("float16", 3072), ("bfloat16", 4096), ("float32", 2048)])
@pytest.mark.parametrize("has_gate", [True, False])
def test_static_scratch_forward_matches_workspace_forward(dtype, H, has_gate):
    tdt = getattr(torch, dtype)
    rng = np.random.default_rng(17)
    n_max = 1500
    w = {k: round_to(rng.standard_normal((n_max, H)).astype(np.float32) * 0.05, dtype) for k in ("gate", "up", "down")}
    t = {k: torch.from_numpy(v).to(DEV, tdt) for k, v in w.items()}
    act = "silu" if has_gate else "relu"
    # first call: two rows of x on all rows; second call: one row of x on fewer rows (smaller in both respects)
    for B, n in ((2, n_max), (1, 411)):
        xh = round_to(rng.standard_normal((B, H)).astype(np.float32), dtype)
        x = torch.from_numpy(xh).to(DEV, tdt)
        comb_s = torch.zeros(B, 2 * n, dtype=tdt, device=DEV)
        comb_w = torch.zeros_like(comb_s)
        got = _call(True, x, t["gate"], t["up"], t["down"], n, act, has_gate, comb_s)
        ref = _call(False, x, t["gate"], t["up"], t["down"], n, act, has_gate, comb_w)
        assert torch.equal(got, ref), (B, n, (got.float() - ref.float()).abs().max().item())
        assert torch.equal(comb_s, comb_w), (B, n)
        concat = np.concatenate([w["gate"][:n], w["up"][:n]]) if has_gate else w["up"][:n]
        want, _ = oracle.mlp_forward(xh, concat, np.ascontiguousarray(w["down"][:n].T), act, has_gate)
        assert_close(got.float().cpu().numpy(), want, dtype, f"B={B} n={n}")


def test_static_scratch_forward_under_graph_capture():
    """What the entry point is for: a caller that records a HIP graph.  After one eager call on the device (which
    resolves the address of the library's scratch array; nothing but launches happens afterwards) the call is
    captured, replayed with other work between the replays, and every replay equals the eager result."""
    L = _lib.lib()
    H, n, B = 3072, 900, 1
    tdt = torch.float16
    g = torch.Generator(device=DEV)
    g.manual_seed(5)
    w = [(torch.randn(n, H, generator=g, device=DEV) * 0.05).to(tdt) for _ in range(3)]
    x = torch.randn(B, H, generator=g, device=DEV).to(tdt)
    out = torch.zeros(B, H, dtype=tdt, device=DEV)

    def call():
        rc = L.st_mlp_forward_static(x.data_ptr(), B, H, w[0].data_ptr(), w[1].data_ptr(), w[2].data_ptr(), n, None, 0,
                                     out.data_ptr(), None, 0, _lib.ACT_CODES["silu"], _lib.ST_F16, 1,
                                     torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "st_mlp_forward_static")

    call()                                   # eager: also the first call on this device
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(4):
        x.copy_(torch.randn(B, H, generator=g, device=DEV).to(tdt))
        call()
        torch.cuda.synchronize()
        eager = out.clone()
        out.zero_()
        other = _call(False, x, w[0], w[1], w[2], n // 2, "silu", True)    # unrelated work between the replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
        del other


def test_static_scratch_limits():
    L = _lib.lib()
    assert L.st_mlp_static_scratch_bytes() == 8 << 20
    x = torch.zeros(3, 256, dtype=torch.float16, device=DEV)
    w = torch.zeros(8, 256, dtype=torch.float16, device=DEV)
    out = torch.zeros_like(x)
    s = torch.cuda.current_stream().cuda_stream
    # three rows of x, and a hidden size whose partial rows do not fit: both refused with a message
    rc = L.st_mlp_forward_static(x.data_ptr(), 3, 256, w.data_ptr(), w.data_ptr(), w.data_ptr(), 8, None, 0, out.data_ptr(),
                                 None, 0, 1, _lib.ST_F16, 1, s)
    assert rc == _lib.ST_ERR_ARG and "B=3" in _lib.last_error()
    rc = L.st_mlp_forward_static(x.data_ptr(), 2, 16384, w.data_ptr(), w.data_ptr(), w.data_ptr(), 8, None, 0,
                                 out.data_ptr(), None, 0, 1, _lib.ST_F16, 1, s)
    assert rc == _lib.ST_ERR_ARG and "scratch" in _lib.last_error()
