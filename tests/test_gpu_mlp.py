"""Fused sparse MLP on the GPU vs the oracle (float64-accumulating CPU restatement), through the C ABI.

Tolerances (north star): fp32 1e-5 relative; fp16 / bf16 2e-2 absolute, 1e-2 relative, against an fp32
evaluation of the dtype-rounded weights and inputs."""
import numpy as np
import pytest
import torch

import oracle
import sparse_transformers_amd as st
from sparse_transformers_amd.ops import mlp_forward_rows
from conftest import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(seed, B, H, n, dtype, has_gate, std=0.02, lead_shape=None):
    g = torch.Generator().manual_seed(seed)
    tdt = getattr(torch, dtype)
    cw = (torch.randn((2 if has_gate else 1) * n, H, generator=g) * std).to(tdt)
    dn = (torch.randn(n, H, generator=g) * std).to(tdt)
    x = torch.randn(*(lead_shape or (B,)), H, generator=g).to(tdt)
    return x, cw, dn


def _run(x, cw, dn, act, has_gate):
    H = x.shape[-1]
    db = torch.zeros(1, H, dtype=x.dtype, device=DEV)
    cb = torch.zeros(1, 2, dtype=x.dtype, device=DEV)
    out = st.sparse_mlp_forward(x.to(DEV), cw.to(DEV), dn.to(DEV).t(), db, cb, act, has_gate)
    torch.cuda.synchronize()
    return out, db, cb


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("act", ["silu", "relu", "gelu_pytorch_tanh", "sigmoid"])
@pytest.mark.parametrize("has_gate", [True, False])
def test_forward_vs_oracle_small(dtype, act, has_gate):
    for seed, (B, H, n) in enumerate([(1, 64, 5), (1, 256, 300), (2, 128, 77), (3, 1024, 129), (5, 512, 1000)]):
        x, cw, dn = _case(seed, B, H, n, dtype, has_gate, std=0.05)
        out, db, cb = _run(x, cw, dn, act, has_gate)
        want, wantc = oracle.mlp_forward(x.float().numpy(), cw.float().numpy(), dn.float().numpy().T, act, has_gate)
        assert out.shape == x.shape and out.data_ptr() == db.data_ptr()        # aliases down_proj_buffer
        assert tuple(db.shape) == (B, H) and tuple(cb.shape) == (B, cw.shape[0])  # buffers resized in place
        assert_close(out.float().cpu().numpy(), want, dtype, f"out B={B} H={H} n={n}")
        assert_close(cb.float().cpu().numpy(), wantc, dtype, "combined_proj_buffer")


@pytest.mark.parametrize("name,B,H,n,dtype,act,has_gate", [
    ("llama-1b layer fp32", 1, 2048, 2457, "float32", "silu", True),
    ("llama-3b layer fp16", 1, 3072, 2867, "float16", "silu", True),
    ("llama-3b bf16, 4 rows, union of masks", 4, 3072, 4620, "bfloat16", "silu", True),
    ("llama-3b bf16, 8 rows, union of masks", 8, 3072, 6300, "bfloat16", "silu", True),
    ("mistral-7b layer", 1, 4096, 3584, "bfloat16", "silu", True),
    ("mistral-7b layer, 2 rows", 2, 4096, 3584, "bfloat16", "silu", True),
    ("relu-llama-7b gated", 1, 4096, 1100, "float16", "relu", True),
    ("relu-llama-7b ungated", 1, 4096, 1100, "float16", "relu", False),
    ("fp32 wide rows (two chunks per thread)", 1, 4096, 700, "float32", "silu", True),
    ("fp32 8192 hidden", 1, 8192, 300, "float32", "relu", True),
    ("fp16 8192 hidden", 3, 8192, 900, "float16", "silu", True),
])
def test_forward_vs_oracle_config_shapes(name, B, H, n, dtype, act, has_gate):
    x, cw, dn = _case(11, B, H, n, dtype, has_gate, lead_shape=(B, 1))
    out, _, cb = _run(x, cw, dn, act, has_gate)
    want, wantc = oracle.mlp_forward(x.float().numpy(), cw.float().numpy(), dn.float().numpy().T, act, has_gate)
    assert out.shape == (B, 1, H)
    assert_close(out.float().cpu().numpy(), want, dtype, name)
    assert_close(cb.float().cpu().numpy(), wantc, dtype, name + " combined")


@pytest.mark.parametrize("act", ["silu", "relu", "gelu_pytorch_tanh", "sigmoid"])
@pytest.mark.parametrize("has_gate", [True, False])
def test_forward_float64(act, has_gate):
    """Double precision (the reference's operator is dtype-generic, sparse_mlp_op.cpp:151-161): against numpy's
    float64 matrix products (1e-12 of the output's scale: only the order of the sums differs) and, on inputs that
    float32 holds exactly, against the oracle (whose sums are in double and whose outputs are rounded to float32)."""
    acts = {"silu": lambda v: v / (1 + np.exp(-v)), "relu": lambda v: np.maximum(v, 0), "sigmoid": lambda v: 1 / (1 + np.exp(-v)),
            "gelu_pytorch_tanh": lambda v: 0.5 * v * (1 + np.tanh(np.sqrt(2 / np.pi) * (v + 0.044715 * v ** 3)))}
    for seed, (B, H, n) in enumerate([(1, 64, 5), (1, 3072, 700), (3, 256, 300), (8, 130, 77), (9, 1024, 129), (19, 512, 1000)]):
        x, cw, dn = _case(seed, B, H, n, "float32", has_gate, std=0.05)      # float32 values, held in double
        out, db, cb = _run(x.double(), cw.double(), dn.double(), act, has_gate)
        assert out.dtype == torch.float64 and tuple(cb.shape) == (B, cw.shape[0])
        xd, cwd, dnd = x.double().numpy(), cw.double().numpy(), dn.double().numpy()
        up = xd @ cwd[n:].T if has_gate else xd @ cwd.T
        h = acts[act](xd @ cwd[:n].T) * up if has_gate else acts[act](up)
        assert_close(out.cpu().numpy(), h @ dnd, "float64", f"float64 out B={B} H={H} n={n}")
        assert_close(cb.cpu().numpy()[:, :n], h, "float64", "float64 combined")
        if has_gate:
            assert_close(cb.cpu().numpy()[:, n:], up, "float64", "float64 combined, up half")
        want, wantc = oracle.mlp_forward(x.numpy(), cw.numpy(), dn.numpy().T, act, has_gate)
        assert_close(out.cpu().numpy(), want, "float32", "float64 against the oracle")
        assert_close(cb.cpu().numpy(), wantc, "float32", "float64 combined against the oracle")
    # an odd hidden size has rows that are not 16-byte multiples
    x, cw, dn = _case(3, 1, 33, 8, "float32", True)
    with pytest.raises(ValueError, match="16-byte"):
        _run(x.double(), cw.double(), dn.double(), "silu", True)
    # caches and the predictor do not take double
    with pytest.raises(TypeError, match="float64"):
        st.WeightCache(torch.ones(8, dtype=torch.bool, device=DEV), 16, torch.zeros(8, 16, dtype=torch.float64, device=DEV),
                       torch.zeros(8, 16, dtype=torch.float64, device=DEV), torch.zeros(16, 8, dtype=torch.float64, device=DEV))


def test_matches_reference_operator_vectors(golden_mlp):
    """Outputs of the reference's compiled ReLU operator (tests/golden/mlp_forward.json)."""
    for case in golden_mlp:
        H, n, hg = case["H"], case["n"], case["has_gate"]
        x = torch.tensor(case["x"]).reshape(case["x_shape"])
        cw = torch.tensor(case["concat"]).reshape(-1, H)
        dn = torch.tensor(case["down_rows"]).reshape(n, H)
        out, _, cb = _run(x, cw, dn, "relu", hg)
        np.testing.assert_allclose(out.cpu().numpy().ravel(), np.array(case["out"], np.float32), rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(cb.cpu().numpy().ravel(), np.array(case["combined"], np.float32), rtol=2e-5,
                                   atol=2e-5)


def test_device_count_and_hint_paths():
    """With a device-side count the result must not depend on the host's hint (too low, exact, too
    high, absent) nor on rows beyond the count."""
    I, H, n = 4096, 3072, 1500
    g = torch.Generator().manual_seed(2)
    gate = (torch.randn(I, H, generator=g) * 0.02).half().to(DEV)
    up = (torch.randn(I, H, generator=g) * 0.02).half().to(DEV)
    dn = (torch.randn(I, H, generator=g) * 0.02).half().to(DEV)
    x = torch.randn(1, H, generator=g).half().to(DEV)
    n_dev = torch.tensor([n], dtype=torch.int32, device=DEV)
    ref = torch.empty(1, H, dtype=torch.float16, device=DEV)
    mlp_forward_rows(x, gate, up, dn, n, None, ref, None, "silu", True)
    want, _ = oracle.mlp_forward(x.float().cpu().numpy(), torch.cat([gate[:n], up[:n]]).float().cpu().numpy(),
                                 dn[:n].float().cpu().numpy().T, "silu", True)
    assert_close(ref.float().cpu().numpy(), want, "float16", "host count")
    for hint in (0, 1, 700, n, n + 500, I):
        out = torch.full((1, H), float("nan"), dtype=torch.float16, device=DEV)
        mlp_forward_rows(x, gate, up, dn, I, n_dev, out, None, "silu", True, n_hint=hint)
        assert torch.equal(out, ref), f"hint {hint}"
    n_dev.fill_(0)
    out = torch.full((1, H), 1.0, dtype=torch.float16, device=DEV)
    mlp_forward_rows(x, gate, up, dn, I, n_dev, out, None, "silu", True, n_hint=n)
    assert not out.any()                                       # empty active set -> zeros


@pytest.mark.parametrize("B,H,dt", [(4, 3072, "float16"), (20, 2048, "bfloat16"), (6, 1536, "bfloat16")])
def test_batch_device_count_and_hint_paths(B, H, dt):
    """The batch kernels deal rows to blocks for the count the host expects before the device's count has arrived:
    whatever that guess (absent, too low, exact, too high), the result carries the bits of a call with the exact host
    count, and an empty set gives zeros."""
    I, n = 4096, 1777
    dtype = getattr(torch, dt)
    g = torch.Generator().manual_seed(5)
    gate = (torch.randn(I, H, generator=g) * 0.02).to(dtype).to(DEV)
    up = (torch.randn(I, H, generator=g) * 0.02).to(dtype).to(DEV)
    dn = (torch.randn(I, H, generator=g) * 0.02).to(dtype).to(DEV)
    x = torch.randn(B, H, generator=g).to(dtype).to(DEV)
    n_dev = torch.tensor([n], dtype=torch.int32, device=DEV)
    ref = torch.empty(B, H, dtype=dtype, device=DEV)
    mlp_forward_rows(x, gate, up, dn, n, None, ref, None, "silu", True)
    want, _ = oracle.mlp_forward(x.float().cpu().numpy(), torch.cat([gate[:n], up[:n]]).float().cpu().numpy(),
                                 dn[:n].float().cpu().numpy().T, "silu", True)
    assert_close(ref.float().cpu().numpy(), want, dt, "host count")
    for hint in (0, 1, 900, n - 1, n, n + 1, n + 700, I):
        out = torch.full((B, H), float("nan"), dtype=dtype, device=DEV)
        mlp_forward_rows(x, gate, up, dn, I, n_dev, out, None, "silu", True, n_hint=hint)
        assert torch.equal(out, ref), f"hint {hint}"
    n_dev.fill_(0)
    out = torch.full((B, H), 1.0, dtype=dtype, device=DEV)
    mlp_forward_rows(x, gate, up, dn, I, n_dev, out, None, "silu", True, n_hint=n)
    assert not out.any()                                       # empty active set -> zeros


def test_float64_device_count_and_empty_set():
    """Double precision with the count on the device: rows beyond it are ignored, the result carries the same bits
    as with the host's count (fixed summation order), and an empty set gives zeros."""
    I, H, n = 700, 256, 333
    g = torch.Generator().manual_seed(4)
    gate = torch.randn(I, H, generator=g, dtype=torch.float64).to(DEV)
    up = torch.randn(I, H, generator=g, dtype=torch.float64).to(DEV)
    dn = torch.randn(I, H, generator=g, dtype=torch.float64).to(DEV)
    x = torch.randn(3, H, generator=g, dtype=torch.float64).to(DEV)
    ref = torch.empty(3, H, dtype=torch.float64, device=DEV)
    mlp_forward_rows(x, gate, up, dn, n, None, ref, None, "silu", True)
    gu = x @ gate[:n].T
    want = ((gu / (1 + torch.exp(-gu))) * (x @ up[:n].T)) @ dn[:n]
    assert_close(ref.cpu().numpy(), want.cpu().numpy(), "float64", "float64, host count")
    n_dev = torch.tensor([n], dtype=torch.int32, device=DEV)
    out = torch.full((3, H), float("nan"), dtype=torch.float64, device=DEV)
    comb = torch.zeros(3, 2 * I, dtype=torch.float64, device=DEV)
    mlp_forward_rows(x, gate, up, dn, I, n_dev, out, comb, "silu", True)
    assert_close(out.cpu().numpy(), want.cpu().numpy(), "float64", "float64, device count")
    n_dev.fill_(0)
    mlp_forward_rows(x, gate, up, dn, I, n_dev, out, None, "silu", True)
    assert not out.any()
    out.fill_(1.0)
    mlp_forward_rows(x, gate, up, dn, 0, None, out, None, "silu", True)
    assert not out.any()


def test_run_to_run_determinism_and_linearity_full_size():
    x, cw, dn = _case(5, 1, 3072, 2867, "float16", True)
    a, _, _ = _run(x, cw, dn, "silu", True)
    b, _, _ = _run(x, cw, dn, "silu", True)
    assert torch.equal(a, b)                                   # fixed summation order
    # identity activation, ungated: the op is linear in x
    xs = torch.randn(2, 3072, generator=torch.Generator().manual_seed(1)).float()
    cwu, dnf = cw[2867:].float(), dn.float()
    y0, _, _ = _run(xs[:1], cwu, dnf, "identity", False)
    y0 = y0.clone()
    y1, _, _ = _run(xs[1:], cwu, dnf, "identity", False)
    y1 = y1.clone()
    ys, _, _ = _run(xs[:1] + xs[1:], cwu, dnf, "identity", False)
    assert_close((y0 + y1).cpu().numpy(), ys.cpu().numpy(), "float32", "linearity")


def test_argument_errors():
    x, cw, dn = _case(0, 1, 64, 8, "float32", True)
    db = torch.zeros(1, 64, device=DEV)
    cb = torch.zeros(1, 2, device=DEV)
    with pytest.raises(ValueError):
        st.sparse_mlp_forward(x.to(DEV), cw.to(DEV)[:-1], dn.to(DEV).t(), db, cb, "silu")      # odd row count
    with pytest.raises(ValueError):
        st.sparse_mlp_forward(x.to(DEV), cw.to(DEV), dn.to(DEV)[:-1].t(), db, cb, "silu")      # n mismatch
    with pytest.raises(ValueError):
        st.sparse_mlp_forward(x.to(DEV), cw.to(DEV), dn.to(DEV).t(), db, cb, "tanh")           # unknown act
    with pytest.raises(TypeError):
        st.sparse_mlp_forward(x.to(DEV), cw.to(DEV).half(), dn.to(DEV).t(), db, cb, "silu")    # dtype mismatch
    # a contiguous [H, n] down matrix (not the cache's view) still gives the right answer
    dwc = dn.to(DEV).t().contiguous()
    with pytest.warns(UserWarning):
        out = st.sparse_mlp_forward(x.to(DEV), cw.to(DEV), dwc, db, cb, "silu")
    want, _ = oracle.mlp_forward(x.numpy(), cw.numpy(), dn.numpy().T, "silu", True)
    assert_close(out.cpu().numpy(), want, "float32", "repacked down")


@pytest.mark.parametrize("name,M,H,n,dtype,act,has_gate", [
    ("small ragged", 130, 256, 200, "float16", "silu", True),
    ("one row tile, n below a K step", 32, 128, 20, "bfloat16", "relu", True),
    ("ungated", 77, 512, 333, "float16", "relu", False),
    ("llama-3b prefill shape, part of the active set", 512, 3072, 1000, "bfloat16", "silu", True),
    ("wide hidden", 96, 4096, 600, "float16", "gelu_pytorch_tanh", True),
    ("narrow tiles, two K groups, many tiles", 100, 512, 7000, "bfloat16", "silu", True),
    ("64-row weight tiles, two K groups", 512, 256, 2457, "float16", "silu", True),
    ("narrow tiles, one K group (more tiles than CUs, one row tile)", 64, 256, 17000, "float16", "silu", True),
    ("the same, ungated", 500, 384, 2300, "bfloat16", "relu", False),
    ("up to 64 rows of x: four K groups", 50, 768, 900, "bfloat16", "silu", True),
    ("four K groups, ungated", 64, 512, 333, "float16", "sigmoid", False),
    ("one active row", 40, 256, 1, "float16", "silu", True),
    ("three active rows, several row tiles", 300, 256, 3, "bfloat16", "silu", True),
])
def test_prefill_mfma_vs_oracle(name, M, H, n, dtype, act, has_gate):
    """More than 32 rows (32 where the batch kernels do not apply) in fp16 / bf16 run on the MFMA GEMM kernels; same
    tolerance as decode."""
    x, cw, dn = _case(21, M, H, n, dtype, has_gate)
    out, _, cb = _run(x, cw, dn, act, has_gate)
    want, wantc = oracle.mlp_forward(x.float().numpy(), cw.float().numpy(), dn.float().numpy().T, act, has_gate)
    assert_close(out.float().cpu().numpy(), want, dtype, name)
    assert_close(cb.float().cpu().numpy()[:, :n], wantc[:, :n], dtype, name + " combined[:, :n]")


@pytest.mark.parametrize("M", [40, 200, 512])
def test_prefill_device_count(M):
    """The GEMM kernels with the active count read on the device: the tile geometry is laid out for the host's
    upper bound, rows beyond the device count may hold anything (here NaN), and the result is the one for the
    exact count."""
    I, H, n = 6144, 1024, 1500
    g = torch.Generator().manual_seed(31)
    gate = (torch.randn(I, H, generator=g) * 0.02).half().to(DEV)
    up = (torch.randn(I, H, generator=g) * 0.02).half().to(DEV)
    dn = (torch.randn(I, H, generator=g) * 0.02).half().to(DEV)
    x = torch.randn(M, H, generator=g).half().to(DEV)
    ref = torch.empty(M, H, dtype=torch.float16, device=DEV)
    mlp_forward_rows(x, gate, up, dn, n, None, ref, None, "silu", True)
    for t in (gate, up, dn):
        t[n:] = float("nan")
    n_dev = torch.tensor([n], dtype=torch.int32, device=DEV)
    out = torch.full((M, H), float("nan"), dtype=torch.float16, device=DEV)
    mlp_forward_rows(x, gate, up, dn, I, n_dev, out, None, "silu", True)
    torch.cuda.synchronize()
    assert_close(out.float().cpu().numpy(), ref.float().cpu().numpy(), "float16", f"device count, {M} rows")
    want, _ = oracle.mlp_forward(x[:4].float().cpu().numpy(), torch.cat([gate[:n], up[:n]]).float().cpu().numpy(),
                                 dn[:n].float().cpu().numpy().T, "silu", True)
    assert_close(out[:4].float().cpu().numpy(), want, "float16", "device count vs oracle")
    n_dev.fill_(0)
    out.fill_(1.0)
    mlp_forward_rows(x, gate, up, dn, I, n_dev, out, None, "silu", True)
    assert not out.any()                                       # empty active set -> zeros


def test_prefill_agrees_with_decode_kernel():
    """The MFMA path (B = 40) and the streaming path (the same rows, 4 at a time) agree to rounding."""
    x, cw, dn = _case(22, 40, 1024, 700, "float16", True)
    big, _, _ = _run(x, cw, dn, "silu", True)
    big = big.clone()
    for b0 in range(0, 40, 8):
        small, _, _ = _run(x[b0:b0 + 8], cw, dn, "silu", True)
        assert_close(small.float().cpu().numpy(), big[b0:b0 + 8].float().cpu().numpy(), "float16", f"rows {b0}")


@pytest.mark.parametrize("name,M,H,n,dtype,act,has_gate", [
    ("ragged rows and columns, K loop with whole groups and a tail", 300, 1152, 6000, "bfloat16", "silu", True),
    ("ungated, K loop shorter than one group", 260, 256, 8500, "float16", "relu", False),
    ("llama-3b prefill, every row active", 512, 3072, 8192, "bfloat16", "silu", True),
    ("ragged 256-row tile through both wide kernels, intermediate kept in the combined buffer", 448, 1024, 4096, "float16", "silu", True),
    ("the same with an odd count: combined rows not 16-byte aligned, intermediate in the workspace", 448, 1024, 3001, "bfloat16", "silu", True),
    ("ungated, combined buffer exactly as wide as the padded intermediate", 512, 512, 5120, "float16", "relu", False),
    ("more 256-row tiles than CUs: down projection without a K split", 2800, 3072, 640, "bfloat16", "silu", True),
    ("two K stages in gate/up; down projection with splits that have nothing to do", 512, 128, 8200, "float16", "silu", True),
])
def test_prefill_wide_blocks(name, M, H, n, dtype, act, has_gate):
    """With more 128-row tiles than CUs the gate/up kernel switches to 256-row blocks, and from 256 rows on the down
    projection to 256-row tiles with the K range split over the CUs.  Every row of the output and of the
    intermediate is held against the oracle; a sample of row groups is also compared with the streaming decode
    kernel."""
    x, cw, dn = _case(23, M, H, n, dtype, has_gate)
    out, _, cb = _run(x, cw, dn, act, has_gate)
    out, cb = out.float().cpu().numpy().copy(), cb.float().cpu().numpy().copy()
    xf, cwf, dnf = x.float().numpy(), cw.float().numpy(), np.ascontiguousarray(dn.float().numpy().T)
    for r0 in range(0, M, 128):
        rows = slice(r0, min(M, r0 + 128))
        want, wantc = oracle.mlp_forward(xf[rows], cwf, dnf, act, has_gate)
        assert_close(out[rows], want, dtype, f"{name} rows {rows}")
        assert_close(cb[rows, :n], wantc[:, :n], dtype, f"{name} combined rows {rows}")
    step = 8
    for b0 in range(0, M, 64):   # a sample of row groups through the streaming kernel
        small, _, cs = _run(x[b0:b0 + step], cw, dn, act, has_gate)
        assert_close(out[b0:b0 + step], small.float().cpu().numpy(), dtype, f"{name} rows {b0}.. vs decode kernel")
        assert_close(cb[b0:b0 + step, :n], cs.float().cpu().numpy()[:, :n], dtype, f"{name} combined rows {b0}..")


def test_prefill_leaves_the_parent_of_a_column_slice_alone():
    """`combined` given as a column slice of a wider tensor (ungated, 64 rows of x, n not a multiple of 128): the
    GEMM kernels keep their intermediate in a buffer whose row stride has room for n rounded up to 128 and zero the
    padding, which must not happen to the parent's columns."""
    B, H, n = 64, 512, 700
    x, cw, dn = _case(29, B, H, n, "float16", False)
    parent = torch.full((B, 1024), 7.0, dtype=torch.float16, device=DEV)
    out = torch.empty(B, H, dtype=torch.float16, device=DEV)
    mlp_forward_rows(x.to(DEV), None, cw.to(DEV), dn.to(DEV), n, None, out, parent[:, :n], "relu", False)
    torch.cuda.synchronize()
    assert bool((parent[:, n:] == 7.0).all()), "columns outside the view were written"
    want, wantc = oracle.mlp_forward(x.float().numpy(), cw.float().numpy(), np.ascontiguousarray(dn.float().numpy().T),
                                     "relu", False)
    assert_close(out.float().cpu().numpy(), want, "float16", "out")
    assert_close(parent[:, :n].float().cpu().numpy(), wantc[:, :n], "float16", "combined view")


# ---- MFMA batch kernels (3 <= B <= 32, fp16 / bf16, hidden sizes that are multiples of 256) ----
@pytest.mark.parametrize("name,B,H,n,dtype,act,has_gate", [
    ("llama-3b bf16, 4 rows", 4, 3072, 4620, "bfloat16", "silu", True),
    ("llama-3b bf16, 16 rows", 16, 3072, 7660, "bfloat16", "silu", True),
    ("mistral-7b bf16, 8 rows", 8, 4096, 3584, "bfloat16", "silu", True),
    ("4096-wide fp16, 4 rows, ungated relu", 4, 4096, 1100, "float16", "relu", False),
    ("two passes of 16 + ragged tail", 19, 2048, 1237, "float16", "gelu_pytorch_tanh", True),
    ("31 rows, fewer active rows than blocks", 31, 3072, 97, "bfloat16", "sigmoid", True),
    ("32 rows: two full passes", 32, 3072, 2867, "float16", "silu", True),
    ("one active row", 5, 2048, 1, "float16", "silu", True),
    ("33 rows per block (two tiles)", 3, 2048, 8450, "float16", "silu", False),
    # hidden sizes without a kernel instantiated for them (run-time K loop; x from LDS up to 4096 columns, from memory beyond)
    ("qwen2-7b width 3584, 8 rows", 8, 3584, 2500, "bfloat16", "silu", True),
    ("width 5120, 4 rows (x straight from memory)", 4, 5120, 1800, "float16", "silu", True),
    ("opt-125m width 768, 16 rows, ungated relu", 16, 768, 1111, "float16", "relu", False),
    ("qwen2-1.5b width 1536, 20 rows (two passes of 16 + 4)", 20, 1536, 3000, "bfloat16", "silu", True),
    ("width 8192, 3 rows, ragged tiles", 3, 8192, 1031, "float16", "gelu_pytorch_tanh", True),
    ("width 256, 5 rows: a single k-step per wave", 5, 256, 300, "float16", "silu", True),
])
def test_batch_mfma_vs_oracle(name, B, H, n, dtype, act, has_gate):
    x, cw, dn = _case(4242 + B + n, B, H, n, dtype, has_gate)
    out, db, cb = _run(x, cw, dn, act, has_gate)
    want, wantc = oracle.mlp_forward(x.float().numpy(), cw.float().numpy(), dn.float().numpy().T, act, has_gate)
    assert tuple(out.shape) == (B, H) and tuple(cb.shape) == (B, cw.shape[0])
    assert_close(out.float().cpu().numpy(), want, dtype, name)
    assert_close(cb.float().cpu().numpy(), wantc, dtype, name + " combined")


def test_batch_mfma_device_count_and_determinism():
    """The batch kernels take the active count from device memory (rows past it may hold anything, here NaN),
    and repeat bit-identically."""
    B, H, I, n = 8, 3072, 2000, 1333
    x, cw, dn = _case(99, B, H, I, "float16", True)
    gate, up = cw[:I].clone(), cw[I:].clone()
    gate[n:], up[n:], dn[n:] = float("nan"), float("nan"), float("nan")
    xg, gg, ug, dg = x.to(DEV), gate.to(DEV), up.to(DEV), dn.to(DEV)
    n_dev = torch.tensor([n], dtype=torch.int32, device=DEV)
    outs = []
    for _ in range(3):
        out = torch.full((B, H), float("nan"), dtype=torch.float16, device=DEV)
        mlp_forward_rows(xg, gg, ug, dg, I, n_dev, out, None, "silu", True)
        torch.cuda.synchronize()
        outs.append(out.cpu())
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    want, _ = oracle.mlp_forward(x.float().numpy(), torch.cat([gate[:n], up[:n]]).float().numpy(),
                                 dn[:n].float().numpy().T, "silu", True)
    assert_close(outs[0].float().numpy(), want, "float16", "device count")
    # an empty active set gives zeros
    n_dev.zero_()
    out = torch.full((B, H), float("nan"), dtype=torch.float16, device=DEV)
    mlp_forward_rows(xg, gg, ug, dg, I, n_dev, out, None, "silu", True)
    torch.cuda.synchronize()
    assert torch.count_nonzero(out).item() == 0


def test_batch_mfma_agrees_with_streaming_kernel():
    """Same inputs through the MFMA batch kernels (4 rows at once) and the streaming kernel (row by row)."""
    H, n = 3072, 2867
    x, cw, dn = _case(7, 4, H, n, "bfloat16", True)
    out4, _, _ = _run(x, cw, dn, "silu", True)
    ref = torch.cat([_run(x[i:i + 1], cw, dn, "silu", True)[0].clone() for i in range(4)]).float().cpu().numpy()
    assert_close(out4.float().cpu().numpy(), ref, "bfloat16", "batch vs streaming")
