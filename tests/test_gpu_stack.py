"""The per-layer sequence (predictor -> mask -> union -> cache update -> sparse MLP) over a small stack,
GPU vs the oracle pipeline, eager and replayed from a HIP graph."""
import numpy as np
import pytest
import torch

import oracle
import sparse_transformers_amd as st
from sparse_transformers_amd import synthetic as syn
from conftest import assert_close, round_to

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _build(dtype, L=3, H=256, I=640, r=16, B=1, has_gate=True, act="silu", seed=0):
    rng = np.random.default_rng(seed)
    tdt = getattr(torch, dtype)
    layers, oracles = [], []
    for _ in range(L):
        w = syn.layer_weights(rng, H, I, r, std=0.05, has_gate=has_gate)
        w = {k: (None if v is None else round_to(v, dtype)) for k, v in w.items()}
        t = {k: (None if v is None else torch.from_numpy(v).to(DEV, tdt)) for k, v in w.items()}
        init = np.ones(I, bool)
        cache = st.WeightCache(torch.from_numpy(init).to(DEV), H, t["gate"], t["up"], t["down"], has_gate)
        layers.append(st.SparseDecodeLayer(st.FastLoRAProjection(t["A"], t["Bm"]), cache, act, 0.0, True))
        oracles.append((oracle.OracleWeightCache(init, H, w["gate"], w["up"], w["down"], has_gate), w))
    return st.SparseMLPStack(layers), oracles


def _oracle_step(oracles, x, x_pred, thr, act, has_gate, dtype):
    masks = []
    for l, (oc, w) in enumerate(oracles):
        s = oracle.predictor_scores(x_pred[l], w["A"], w["Bm"])
        m = oracle.mask_threshold(s, thr[l], True)
        masks.append((m, s))
        oc.update_active_weights(m)
        y, _ = oracle.mlp_forward(x, oc.get_concat_weight(), oc.get_active_down_weight(), act, has_gate)
        x = round_to(y, dtype)            # the GPU path stores each layer's output in the storage type
    return x, masks


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("has_gate", [True, False])
def test_predictor_driven_decode_steps(dtype, has_gate):
    L, H, I, B = 3, 256, 640, 2
    act = "silu" if has_gate else "relu"
    stack, oracles = _build(dtype, L, H, I, 16, B, has_gate, act)
    rng = np.random.default_rng(1)
    tdt = getattr(torch, dtype)
    for step in range(6):
        x = round_to(rng.standard_normal((B, H)).astype(np.float32), dtype)
        x_pred = round_to(rng.standard_normal((L, B, H)).astype(np.float32), dtype)
        # per-layer thresholds in a wide score gap so that the masks are unambiguous
        thr = []
        for l, (oc, w) in enumerate(oracles):
            s = oracle.predictor_scores(x_pred[l], w["A"], w["Bm"])
            thr.append(syn.threshold_for_fraction(s.max(0), 0.4))
            stack.layers[l].thr = thr[l]
        want, masks = _oracle_step(oracles, x, x_pred, thr, act, has_gate, dtype)
        got = stack.decode_step(torch.from_numpy(x).to(DEV, tdt), [torch.from_numpy(x_pred[l]).to(DEV, tdt)
                                                                    for l in range(L)])
        for l, (oc, _) in enumerate(oracles):
            m, s = masks[l]
            near = (np.abs(s - thr[l]) < 1e-5 * np.abs(s).max()).any(0)
            assert not near.any(), "threshold inside the guard band"
            assert np.array_equal(stack.layers[l].mask.cpu().numpy(), m), (step, l)
            assert stack.layers[l].cache.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist()
        assert_close(got.float().cpu().numpy(), want, dtype, f"step {step}")


@pytest.mark.parametrize("overlap", [False, True])
def test_graph_replay_equals_eager(overlap):
    """Replays of the captured step (with eager work and synchronisations in between) reproduce the
    eager results and index lists exactly."""
    L, H, I, B = 4, 512, 1024, 1
    stack_g, _ = _build("float16", L, H, I, 32, B, seed=5)
    stack_e, _ = _build("float16", L, H, I, 32, B, seed=5)
    trace = torch.from_numpy(syn.mask_trace(3, L, I, 400, 12, 0.05, 0.2)).to(DEV)
    gen = torch.Generator(device=DEV).manual_seed(0)
    xs = torch.randn(12, B, H, device=DEV, generator=gen).half()
    xp = torch.randn(12, L, B, H, device=DEV, generator=gen).half()
    for s in (stack_g, stack_e):
        s.prepare(B, overlap=overlap)
        s.step_staged(xs[0], xp[0], trace[0])
    torch.cuda.synchronize()
    stack_g.capture()
    for t in range(1, 12):
        a = stack_g.step_staged(xs[t], xp[t], trace[t], replay=True).clone()
        b = stack_e.step_staged(xs[t], xp[t], trace[t], replay=False).clone()
        torch.cuda.synchronize()
        assert torch.equal(a, b), t
        for lg, le in zip(stack_g.layers, stack_e.layers):
            assert torch.equal(lg.mask, le.mask)
            assert torch.equal(lg.cache.get_active_indices(), le.cache.get_active_indices())
            assert lg.cache.get_num_active() == 400
        _ = (xs[t].float() @ xs[t].float().t()).sum().item()   # unrelated eager work + a host sync between replays


def test_skip_mlp_module_surface():
    """SkipMLP mirrors the reference module (src/modeling_skip.py:55-128): constructor arguments, sub-modules,
    registered buffers, state-dict keys, initialize_weight_cache / reset_cache, the three forwards."""
    H, I = 128, 320
    g = torch.Generator().manual_seed(0)
    mlp = st.SkipMLP(H, I, 0.5, bias=False, act_fn="silu", use_weight_cache=True)
    assert isinstance(mlp, torch.nn.Module)
    assert sorted(mlp.state_dict()) == sorted(["gate_proj.weight", "up_proj.weight", "down_proj.weight", "init_mask",
                                               "down_proj_buffer", "combined_proj_buffer"])
    assert tuple(mlp.down_proj_buffer.shape) == (1, H) and tuple(mlp.combined_proj_buffer.shape) == (1, 2 * 160)
    assert mlp.init_mask.dtype == torch.bool and bool(mlp.init_mask.all())
    gate, up, down = (torch.randn(I, H, generator=g) * 0.05), (torch.randn(I, H, generator=g) * 0.05), \
        (torch.randn(H, I, generator=g) * 0.05)
    mlp.load_state_dict({"gate_proj.weight": gate, "up_proj.weight": up, "down_proj.weight": down}, strict=False)
    mlp = mlp.to(DEV)
    assert mlp.init_mask.is_cuda and mlp.down_proj_buffer.is_cuda and mlp.combined_proj_buffer.is_cuda
    with pytest.raises(RuntimeError):
        mlp(torch.randn(1, 1, H, device=DEV))
    mlp.initialize_weight_cache()
    wc0 = mlp.weight_cache
    mlp.initialize_weight_cache()
    assert mlp.weight_cache is wc0                        # only built once
    m = torch.rand(I, generator=g) < 0.5
    mlp.weight_cache.update_active_weights(m.to(DEV))
    x = torch.randn(2, 1, H, generator=g)
    out = mlp(x.to(DEV))
    assert out.shape == x.shape
    idx = torch.nonzero(m).flatten()
    oc = oracle.OracleWeightCache(np.ones(I, bool), H, gate.numpy(), up.numpy(), down.numpy(), True)
    oc.update_active_weights(m.numpy())
    want, _ = oracle.mlp_forward(x.numpy(), oc.get_concat_weight(), oc.get_active_down_weight(), "silu", True)
    assert_close(out.cpu().numpy(), want, "float32", "SkipMLP")
    assert sorted(mlp.weight_cache.get_active_indices().cpu().tolist()) == idx.tolist()
    # dense forward (the reference's prefill path) = the full MLP in torch
    dense = mlp(x.to(DEV), use_sparse=False).detach().cpu()
    ref = (torch.nn.functional.silu(x @ gate.t()) * (x @ up.t())) @ down.t()
    assert torch.allclose(dense, ref, rtol=1e-4, atol=1e-5)
    # reset_cache: back to every row active in order 0..I-1 (src/modeling_skip.py:492-497)
    mlp.reset_cache()
    assert mlp.weight_cache is not wc0
    assert mlp.weight_cache.get_active_indices().cpu().tolist() == list(range(I))
    # a move to another dtype invalidates the cache (its rows would no longer match the parameters)
    mlp = mlp.half()
    assert mlp.weight_cache is None and mlp.down_proj_buffer.dtype == torch.float16
    mlp.initialize_weight_cache()
    assert mlp.weight_cache.dtype == torch.float16
    # the cache-less debugging forward with a weight mask
    dbg = st.SkipMLP.from_weights(gate.to(DEV), up.to(DEV), down.to(DEV), 0.5, "silu")
    dbg.use_weight_cache = False
    dbg.weight_mask = m.to(DEV).float()
    assert_close(dbg(x.to(DEV)).detach().cpu().numpy(), want, "float32", "masked dense forward")


@pytest.mark.parametrize("variant", ["llama3b_gated_fp16", "opt_ungated_fp16"])
def test_skip_mlp_full_shape_vs_oracle(variant):
    """The module at a benchmark shape (H = 3072, I = 8192, 35 % active, fp16), gated with SiLU and OPT-style
    ungated with ReLU, decode with one row and with several: sparse forward against the oracle."""
    H, I, dtype = 3072, 8192, "float16"
    gated = variant.startswith("llama")
    rng = np.random.default_rng(12)
    w = syn.layer_weights(rng, H, I, 8, std=0.02, has_gate=gated)
    w = {k: (None if v is None else round_to(v, dtype)) for k, v in w.items()}
    if gated:
        mlp = st.SkipMLP(H, I, 0.65, act_fn="silu")
        mlp.gate_proj.weight.data = torch.from_numpy(w["gate"])
    else:
        mlp = st.OPTSkipMLP(H, I, 0.65)
        assert not hasattr(mlp, "gate_proj") and mlp.act_fn_name == "relu"
    mlp.up_proj.weight.data = torch.from_numpy(w["up"])
    mlp.down_proj.weight.data = torch.from_numpy(w["down"])
    mlp = mlp.to(DEV).half()
    mlp.initialize_weight_cache()
    oc = oracle.OracleWeightCache(np.ones(I, bool), H, w["gate"], w["up"], w["down"], gated)
    act = "silu" if gated else "relu"
    for step, B in enumerate((1, 1, 4, 1)):
        m = syn.initial_mask(rng, I, int(0.35 * I))
        mlp.weight_cache.update_active_weights(torch.from_numpy(m).to(DEV))
        oc.update_active_weights(m)
        x = round_to(rng.standard_normal((B, 1, H)).astype(np.float32), dtype)
        got = mlp(torch.from_numpy(x).to(DEV, torch.float16))
        want, _ = oracle.mlp_forward(x, oc.get_concat_weight(), oc.get_active_down_weight(), act, gated)
        assert_close(got.float().cpu().numpy(), want, dtype, f"{variant} step {step}")
        assert mlp.weight_cache.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist()


def test_lazy_cache_updates_fuse_with_the_next_forward():
    """The decoder layer's order (src/modeling_skip.py:234-261): update_active_weights(mask) early, the MLP later.
    With lazy updates the module's cache remembers the mask and runs update + MLP as one launch at the forward;
    outputs, ordered list and state equal those of a cache that updates at once, bit for bit; a getter or a second
    update in between applies the remembered mask first; an emptying mask is reported by the next synchronising call."""
    H, I = 1024, 2048
    g = torch.Generator().manual_seed(4)
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.05).half().to(DEV)
    gate, up, down = mk(I, H), mk(I, H), mk(H, I)
    lazy = st.SkipMLP.from_weights(gate, up, down, 0.5, "silu")
    eager = st.SkipMLP.from_weights(gate, up, down, 0.5, "silu")
    eager.lazy_cache_updates = False
    lazy.initialize_weight_cache()
    eager.initialize_weight_cache()
    assert lazy.weight_cache.lazy_updates and not eager.weight_cache.lazy_updates
    m = torch.rand(I, generator=g) < 0.4
    for step in range(6):
        m = m ^ (torch.rand(I, generator=g) < 0.1)
        md = m.to(DEV)
        x = mk(1 if step != 3 else 3, H)
        lazy.weight_cache.update_active_weights(md)
        eager.weight_cache.update_active_weights(md)
        assert lazy.weight_cache._pending_mask is not None
        if step == 2:      # a getter before the forward: the remembered update runs on its own
            assert lazy.weight_cache.get_num_active() == int(m.sum()) and lazy.weight_cache._pending_mask is None
        if step == 4:      # a second update before any forward: both are applied, in order
            m = m ^ (torch.rand(I, generator=g) < 0.1)
            md = m.to(DEV)
            lazy.weight_cache.update_active_weights(md)
            eager.weight_cache.update_active_weights(md)
        y_lazy, y_eager = lazy(x), eager(x)
        assert lazy.weight_cache._pending_mask is None
        assert torch.equal(y_lazy, y_eager), step
        assert torch.equal(lazy.weight_cache.get_active_indices(), eager.weight_cache.get_active_indices()), step
    lazy.weight_cache.update_active_weights(torch.zeros(I, dtype=torch.bool, device=DEV))   # accepted silently ...
    with pytest.raises(RuntimeError, match="No active weights"):
        lazy.weight_cache.get_num_active()                                                   # ... and reported here


def test_reference_call_sequence_reads_the_cache_in_place():
    """update_active_weights -> get_concat_weight -> get_active_down_weight -> sparse_mlp_forward, as a caller of
    the reference's operator writes it: the concat weight is a handle that sparse_mlp_forward resolves to the
    cache's packed rows (no [2n,H] copy); anything else that touches it gets the real contiguous tensor; a handle
    kept across a later update is refused."""
    H, I = 256, 512
    g = torch.Generator().manual_seed(2)
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.05).half().to(DEV)
    gate, up, down = mk(I, H), mk(I, H), mk(H, I)
    wc = st.WeightCache(torch.ones(I, dtype=torch.bool, device=DEV), H, gate, up, down, True)
    m = (torch.rand(I, generator=g) < 0.4).to(DEV)
    wc.update_active_weights(m)
    n = int(m.sum())
    cw, dw = wc.get_concat_weight(), wc.get_active_down_weight()
    assert tuple(cw.shape) == (2 * n, H) and cw.dtype == torch.float16 and cw.is_cuda and cw.is_contiguous()
    assert cw._real is None and wc.get_concat_weight() is cw
    x = mk(3, H)
    db, cb = torch.zeros(1, H, dtype=torch.float16, device=DEV), torch.zeros(1, 2, dtype=torch.float16, device=DEV)
    y = st.sparse_mlp_forward(x, cw, dw, db, cb, "silu").clone()
    assert cw._real is None                                   # still no copy
    order = wc.get_active_indices()
    real = cw + 0                                             # any torch op materialises it
    assert cw._real is not None and torch.equal(real, torch.cat([gate[order], up[order]]))
    assert torch.equal(cw.t().contiguous(), real.t().contiguous()) and torch.equal(cw[:n], gate[order])
    y2 = st.sparse_mlp_forward(x, cw, dw, db, cb, "silu")     # now through the materialised tensor: same bits
    assert torch.equal(y, y2)
    wc.update_active_weights(~m)
    stale = cw
    fresh = wc.get_concat_weight()
    assert fresh is not stale and tuple(fresh.shape) == (2 * (I - n), H)
    with pytest.raises(RuntimeError):
        st.sparse_mlp_forward(x, ConcatStale(stale, wc, n), dw, db, cb, "silu")
    # a handle that is still held when the next update comes is filled first and stays a snapshot of its update,
    # as the reference's torch::cat result does; one that nobody holds costs nothing
    order2 = wc.get_active_indices()
    held = wc.get_concat_weight()
    assert held._real is None
    wc.update_active_weights(m)
    assert held._real is not None and torch.equal(held + 0, torch.cat([gate[order2], up[order2]]))
    dropped = wc.get_concat_weight()
    assert dropped._real is None
    del dropped
    import gc
    gc.collect()
    assert wc._concat_ref() is None
    wc.update_active_weights(~m)      # nothing left to fill


def ConcatStale(stale, wc, n):
    """A handle fetched before the last update that has never been read."""
    from sparse_transformers_amd.weight_cache import ConcatWeightHandle
    return ConcatWeightHandle(wc, n, stale._serial)


@pytest.mark.parametrize("method,B", [("topk", 1), ("topk", 3), ("statistical_topk", 1), ("statistical_topk", 2)])
def test_row_statistic_methods_drive_the_stack(method, B):
    """The stack stepped with the top-k / statistical masks of SkipDecoderLayer._compute_binary_mask:
    masks (selected by the oracle from the same scores) and index order, outputs within tolerance, and a HIP-graph replay equal to
    the eager step (the layer's score and selection buffers are created before the capture)."""
    L, H, I, r = 3, 256, 640, 16
    dtype, act = "float16", "silu"
    k, z = 160, 0.5244
    stack, oracles = _build(dtype, L, H, I, r, B, True, act, seed=9)
    stack_g, _ = _build(dtype, L, H, I, r, B, True, act, seed=9)
    for s in (stack, stack_g):
        for layer in s.layers:
            layer.method, layer.k, layer.std_multiplier = method, k, z
    rng = np.random.default_rng(4)
    xs = round_to(rng.standard_normal((8, B, H)).astype(np.float32), dtype)
    xps = round_to(rng.standard_normal((8, L, B, H)).astype(np.float32), dtype)
    tx = torch.from_numpy(xs).to(DEV, torch.float16)
    txp = torch.from_numpy(xps).to(DEV, torch.float16)
    stack_g.prepare(B)
    stack_g.use_trace_masks = False
    for t in range(8):
        x = xs[t]
        want_masks = []
        for l, (oc, w) in enumerate(oracles):
            # the selection is checked on the kernel's own fp32 scores (which are checked against the oracle's
            # here and in test_gpu_predictor), so that a k-th score in a narrow gap cannot make the two diverge
            s = stack.layers[l].predictor(txp[t, l]).cpu().numpy()
            s_ref = oracle.predictor_scores(xps[t, l], w["A"], w["Bm"])
            assert np.abs(s - s_ref).max() <= 4e-6 * np.abs(s_ref).max()
            if method == "topk":
                m = oracle.mask_topk(s, k)
            else:
                m, cut = oracle.mask_statistical(s, z)
                assert (np.abs(s - cut[:, None]) > 1e-6 * np.abs(s).max()).all(), "score inside the guard band"
            want_masks.append(m)
            oc.update_active_weights(m)
            y, _ = oracle.mlp_forward(x, oc.get_concat_weight(), oc.get_active_down_weight(), act, True)
            x = round_to(y, dtype)
        got = stack.decode_step(tx[t], [txp[t, l] for l in range(L)])
        for l, (oc, _) in enumerate(oracles):
            assert np.array_equal(stack.layers[l].mask.cpu().numpy(), want_masks[l]), (t, l)
            assert stack.layers[l].cache.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist()
        assert_close(got.float().cpu().numpy(), x, dtype, f"step {t}")
        # the same step through the staged / captured path
        if t == 1:
            torch.cuda.synchronize()
            stack_g.capture()
        out_g = stack_g.step_staged(tx[t], txp[t], None, replay=t >= 1).clone()
        torch.cuda.synchronize()
        assert torch.equal(out_g, got), t
        for lg, le in zip(stack_g.layers, stack.layers):
            assert torch.equal(lg.mask, le.mask)
            assert torch.equal(lg.cache.get_active_indices(), le.cache.get_active_indices())


def test_captured_graph_survives_a_larger_forward_elsewhere():
    """A captured step keeps the address of the stack's own MLP scratch.  A later eager forward that needs far
    more scratch (512 rows of x through the same caches: the MFMA path) must not free or reuse it: replays after
    it still equal the eager stack bit for bit."""
    L, H, I, B = 3, 512, 1024, 1
    stack_g, _ = _build("float16", L, H, I, 32, B, seed=6)
    stack_e, _ = _build("float16", L, H, I, 32, B, seed=6)
    trace = torch.from_numpy(syn.mask_trace(5, L, I, 400, 10, 0.05, 0.2)).to(DEV)
    gen = torch.Generator(device=DEV).manual_seed(1)
    xs = torch.randn(10, B, H, device=DEV, generator=gen).half()
    xp = torch.randn(10, L, B, H, device=DEV, generator=gen).half()
    big = torch.randn(512, H, device=DEV, generator=gen).half()
    for s in (stack_g, stack_e):
        s.prepare(B)
        s.step_staged(xs[0], xp[0], trace[0])
    torch.cuda.synchronize()
    stack_g.capture()
    for t in range(1, 10):
        a = stack_g.step_staged(xs[t], xp[t], trace[t], replay=True).clone()
        b = stack_e.step_staged(xs[t], xp[t], trace[t], replay=False).clone()
        torch.cuda.synchronize()
        assert torch.equal(a, b), t
        if t in (2, 5):   # a prefill-sized forward on the default scratch, then some allocator churn
            y = stack_g.layers[0].cache.forward(big, "silu")
            junk = [torch.full((1 << 20,), 7.0, device=DEV) for _ in range(8)]
            torch.cuda.synchronize()
            assert torch.isfinite(y.float()).all()
            del junk
