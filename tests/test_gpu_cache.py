"""Differential weight cache on the GPU vs the oracle / golden traces: ordered index list and cache
layout must be bit-exact (integer and byte work)."""
import numpy as np
import pytest
import torch

import oracle
import sparse_transformers_amd as st
from sparse_transformers_amd import synthetic as syn
from conftest import bits_to_mask, golden_weights

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _t(a, dtype=torch.float32):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV, dtype)


def _check_layout(wc, oc_order, gate, up, down, has_gate):
    n = len(oc_order)
    assert wc.get_num_active() == n
    assert wc.get_active_indices().cpu().tolist() == list(oc_order)
    cw = wc.get_concat_weight()
    assert cw.is_contiguous() and cw.shape == ((2 if has_gate else 1) * n, up.shape[1])
    cw = cw.float().cpu().numpy()
    if has_gate:
        assert np.array_equal(cw[:n], gate[oc_order])
    assert np.array_equal(cw[-n:] if n else cw, up[oc_order])
    dw = wc.get_active_down_weight()
    assert dw.shape == (up.shape[1], n) and (n == 0 or dw.stride() == (1, up.shape[1]))
    assert np.array_equal(dw.float().cpu().numpy(), down[:, oc_order])


def test_golden_traces_from_reference(golden_traces):
    for trace in golden_traces:
        I, H, hg = trace["I"], trace["H"], trace["has_gate"]
        gate, up, down = golden_weights(I, H)
        wc = st.WeightCache(_t(bits_to_mask(trace["init_mask"]), torch.bool), H, _t(gate) if hg else None, _t(up),
                            _t(down), hg)
        _check_layout(wc, trace["init_order"], gate, up, down, hg)
        for step in trace["steps"]:
            m = _t(bits_to_mask(step["mask"]), torch.bool)
            if step["error"]:
                with pytest.raises(RuntimeError, match="No active weights"):
                    wc.update_active_weights(m)
                continue
            wc.update_active_weights(m)
            assert wc.get_active_indices().cpu().tolist() == step["order"], trace["seed"]
        _check_layout(wc, trace["steps"][-1]["order"], gate, up, down, hg)


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("has_gate", [True, False])
def test_ragged_traces_vs_oracle(dtype, has_gate):
    tdt = getattr(torch, dtype)
    rng = np.random.default_rng(7)
    for I, H in [(5, 8), (64, 8), (1000, 24), (2051, 16)]:
        g = torch.randn(I, H).to(tdt)
        u = torch.randn(I, H).to(tdt)
        d = torch.randn(H, I).to(tdt)
        gf, uf, df = g.float().numpy(), u.float().numpy(), d.float().numpy()
        trace = syn.ragged_mask_trace(int(rng.integers(1 << 30)), I, 80)
        oc = oracle.OracleWeightCache(trace[0], H, gf if has_gate else None, uf, df, has_gate)
        wc = st.WeightCache(_t(trace[0], torch.bool), H, g.to(DEV) if has_gate else None, u.to(DEV), d.to(DEV), has_gate)
        for t in range(1, len(trace)):
            oc.update_active_weights(trace[t])
            wc.update_active_weights(_t(trace[t], torch.bool))
            assert wc.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist(), (I, t)
            if t % 16 == 0:
                _check_layout(wc, oc.get_active_indices().tolist(), gf, uf, df, has_gate)
        _check_layout(wc, oc.get_active_indices().tolist(), gf, uf, df, has_gate)


@pytest.mark.parametrize("I,n,lo,hi", [(8192, 2867, 0.05, 0.15), (14336, 3584, 0.10, 0.10), (11008, 1100, 0.2, 0.2)])
def test_full_size_index_order(I, n, lo, hi):
    """Index order at the real intermediate sizes (the order does not depend on H, so H is kept small)."""
    H = 8
    rng = np.random.default_rng(1)
    g = rng.standard_normal((I, H)).astype(np.float32)
    u = rng.standard_normal((I, H)).astype(np.float32)
    d = rng.standard_normal((H, I)).astype(np.float32)
    trace = syn.mask_trace(5, 1, I, n, 128, lo, hi)[:, 0]
    oc = oracle.OracleWeightCache(np.ones(I, bool), H, g, u, d, True)
    wc = st.WeightCache(torch.ones(I, dtype=torch.bool, device=DEV), H, _t(g), _t(u), _t(d), True)
    for t in range(len(trace)):
        oc.update_active_weights(trace[t])
        wc.update_active_weights_async(_t(trace[t], torch.bool))   # no read-back between updates
        if t % 32 == 0 or t == len(trace) - 1:
            assert wc.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist(), t
    _check_layout(wc, oc.get_active_indices().tolist(), g, u, d, True)
    st_ = wc.sync_state()
    assert st_["n_active"] == n and st_["n_added"] == st_["n_removed"] > 0


@pytest.mark.parametrize("I,has_gate", [(28672, True), (32768, False), (22016, True)])
def test_large_intermediate_sizes(I, has_gate):
    """Intermediate sizes of the 70B-class models (28672), above what the index lists of the smaller kernels allow:
    index order and layout against the oracle over a trace that starts with every row active, shrinks to a quarter
    (thousands of sequential removals), then churns with the active count drifting both ways, with a no-op update,
    the error of an emptying mask and the state after it."""
    H = 16
    rng = np.random.default_rng(I)
    g = rng.standard_normal((I, H)).astype(np.float32)
    u = rng.standard_normal((I, H)).astype(np.float32)
    d = rng.standard_normal((H, I)).astype(np.float32)
    oc = oracle.OracleWeightCache(np.ones(I, bool), H, g if has_gate else None, u, d, has_gate)
    wc = st.WeightCache(torch.ones(I, dtype=torch.bool, device=DEV), H, _t(g) if has_gate else None, _t(u), _t(d), has_gate)
    assert wc.get_active_indices().cpu().tolist() == list(range(I))
    m = rng.random(I) < 0.25
    masks = [m.copy()]
    for t in range(24):
        m = m ^ (rng.random(I) < rng.choice([0.003, 0.02, 0.1]))
        masks.append(m.copy())
        if t == 9:
            masks.append(m.copy())           # unchanged mask
    for t, mk in enumerate(masks):
        oc.update_active_weights(mk)
        wc.update_active_weights(_t(mk, torch.bool))
        assert wc.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist(), (I, t)
        if t in (0, 5, len(masks) - 1):
            _check_layout(wc, oc.get_active_indices().tolist(), g, u, d, has_gate)
    with pytest.raises(RuntimeError, match="No active weights"):
        wc.update_active_weights(torch.zeros(I, dtype=torch.bool, device=DEV))
    with pytest.raises(RuntimeError):
        oc.update_active_weights(np.zeros(I, bool))
    # (the remembered mask is still the last good one: only indices outside it are added now)
    oc.update_active_weights(np.ones(I, bool))
    wc.update_active_weights(torch.ones(I, dtype=torch.bool, device=DEV))
    assert wc.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist()
    assert 0 < wc.get_num_active() < I
    # update + MLP in one call at this size (two launches underneath) against the oracle
    x = rng.standard_normal((1, H)).astype(np.float32)
    oc.update_active_weights(masks[7])
    y = wc.update_and_forward(_t(masks[7], torch.bool), _t(x), "silu" if has_gate else "relu")
    want, _ = oracle.mlp_forward(x, oc.get_concat_weight(), oc.get_active_down_weight(), "silu" if has_gate else "relu",
                                 has_gate)
    assert wc.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist()
    scale = np.abs(want).max()
    assert np.abs(y.cpu().numpy() - want).max() <= 1e-5 * scale + 1e-6


def test_full_size_layout_invariants_fp16():
    """cfg-2 shapes: every active row is a bit-copy of its pool row; set(indices) == nonzero(mask)."""
    I, H, n = 8192, 3072, 2867
    gen = torch.Generator(device=DEV).manual_seed(3)
    g = (torch.randn(I, H, device=DEV, generator=gen) * 0.02).half()
    u = (torch.randn(I, H, device=DEV, generator=gen) * 0.02).half()
    d = (torch.randn(H, I, device=DEV, generator=gen) * 0.02).half()
    wc = st.WeightCache(torch.ones(I, dtype=torch.bool, device=DEV), H, g, u, d, True)
    assert torch.equal(wc.get_concat_weight(), torch.cat([g, u]))          # init: all rows, ascending
    assert torch.equal(wc.get_active_down_weight(), d)
    trace = syn.mask_trace(9, 1, I, n, 12, 0.05, 0.15)[:, 0]
    for t in range(len(trace)):
        m = _t(trace[t], torch.bool)
        wc.update_active_weights(m)
        idx = wc.get_active_indices()
        assert idx.numel() == n and torch.equal(torch.sort(idx)[0], torch.nonzero(m).flatten())
        cw = wc.get_concat_weight()
        assert torch.equal(cw[:n], g[idx]) and torch.equal(cw[n:], u[idx])
        assert torch.equal(wc.get_active_down_weight(), d[:, idx])


def test_noop_and_error_semantics():
    I, H = 32, 8
    gate, up, down = golden_weights(I, H)
    m0 = np.zeros(I, bool)
    m0[[3, 5, 9]] = True
    wc = st.WeightCache(_t(m0, torch.bool), H, _t(gate), _t(up), _t(down), True)
    s0 = wc.sync_state()
    wc.update_active_weights(_t(m0, torch.bool))           # unchanged mask: nothing happens
    s1 = wc.sync_state()
    assert s1["serial"] == s0["serial"] and s1["n_changed"] == 0 and s1["n_active"] == 3
    with pytest.raises(RuntimeError, match="No active weights"):
        wc.update_active_weights(torch.zeros(I, dtype=torch.bool, device=DEV))
    # the remembered mask is still m0 (the reference stores the new mask only after a successful rebuild), so m0 is
    # an unchanged mask now: the reference returns before touching anything, and so does this -- no second error
    wc.update_active_weights(_t(m0, torch.bool))
    assert wc.get_num_active() == 0
    with pytest.raises(RuntimeError, match="No active weights"):      # all-false again differs from m0: it raises again
        wc.update_active_weights(torch.zeros(I, dtype=torch.bool, device=DEV))
    # an all-false init mask is an unchanged mask for the constructor's update (weight_cache.h:223-226,237-240):
    # nothing is built, and the getters then refuse like the reference's TORCH_CHECK(cache_valid)
    empty = st.WeightCache(torch.zeros(I, dtype=torch.bool, device=DEV), H, _t(gate), _t(up), _t(down), True)
    with pytest.raises(RuntimeError, match="Cache is not valid"):
        empty.get_concat_weight()
    with pytest.raises(RuntimeError, match="Cache is not valid"):
        empty.get_active_down_weight()
    empty.update_active_weights(_t(m0, torch.bool))
    assert empty.get_active_indices().cpu().tolist() == [3, 5, 9]
    with pytest.raises(ValueError):
        wc.update_active_weights(torch.ones(I + 1, dtype=torch.bool, device=DEV))
    # masks of other integer types and on the host are accepted like a bool tensor
    m1 = m0.copy()
    m1[[1, 2]] = True
    oc = oracle.OracleWeightCache(m0, H, gate, up, down, True)
    with pytest.raises(RuntimeError):
        oc.update_active_weights(np.zeros(I, bool))
    oc.update_active_weights(m1)
    wc.update_active_weights(torch.from_numpy(m1.astype(np.int64)))
    assert wc.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist()


def test_constructor_validation():
    I, H = 16, 8
    gate, up, down = golden_weights(I, H)
    ones = torch.ones(I, dtype=torch.bool, device=DEV)
    with pytest.raises(ValueError):
        st.WeightCache(ones, H, _t(gate), _t(up), _t(down.T.copy()), True)          # down must be [H, I]
    with pytest.raises(TypeError):
        st.WeightCache(ones, H, _t(gate), _t(up), _t(down).double(), True)
    with pytest.raises(ValueError):
        st.WeightCache(ones, H, None, _t(up), _t(down), True)
    wc = st.WeightCache(ones, H, None, _t(up), _t(down), False)                       # ungated: gate may be None
    assert wc.get_concat_weight().shape == (I, H)
    with pytest.raises(ValueError):                                                   # rows must be 16-byte multiples
        st.WeightCache(ones, 6, _t(gate[:, :6]), _t(up[:, :6]), _t(down[:6]), True)


def test_fast_path_argument_errors():
    """forward / update_and_forward check x, out and combined against the cache on the host: a wrong dtype, a
    short output or a combined buffer that cannot hold every possible count raises instead of reaching a kernel."""
    I, H = 256, 128
    g = torch.Generator().manual_seed(3)
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.05).half().to(DEV)
    cache = st.WeightCache(torch.ones(I, dtype=torch.bool, device=DEV), H, mk(I, H), mk(I, H), mk(H, I), True)
    mask = (torch.rand(I, generator=g) < 0.5).to(DEV)
    x = mk(1, H)
    for call in (lambda **kw: cache.forward(kw.pop("x", x), "silu", **kw),
                 lambda **kw: cache.update_and_forward(mask, kw.pop("x", x), "silu", **kw)):
        with pytest.raises(TypeError):
            call(x=x.float())                                   # fp32 x on an fp16 cache
        with pytest.raises(ValueError):
            call(x=mk(1, H // 2))                               # wrong hidden size
        with pytest.raises(TypeError):
            call(out=torch.empty(1, H, dtype=torch.float32, device=DEV))
        with pytest.raises(ValueError):
            call(out=torch.empty(1, H // 2, dtype=torch.float16, device=DEV))
        with pytest.raises(ValueError):
            call(combined=torch.empty(1, I, dtype=torch.float16, device=DEV))   # gated: needs 2*I columns
        with pytest.raises(ValueError):
            call(workspace=torch.empty(16, dtype=torch.uint8, device=DEV))
        with pytest.raises((TypeError, RuntimeError)):
            call(x=x.cpu())
    # and the C entry point itself refuses a short row pitch for `combined`
    from sparse_transformers_amd import _lib
    comb = torch.empty(1, I, dtype=torch.float16, device=DEV)
    out = torch.empty(1, H, dtype=torch.float16, device=DEV)
    ws = torch.empty(int(_lib.lib().st_mlp_workspace_bytes(1, H, I)), dtype=torch.uint8, device=DEV)
    rc = _lib.lib().st_cache_update_forward(cache._h, mask.data_ptr(), x.data_ptr(), 1, 0, out.data_ptr(), comb.data_ptr(),
                                            I, ws.data_ptr(), ws.numel(), 1, torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.ST_ERR_ARG and "ldc" in _lib.last_error()
    # nothing above changed the cache
    assert cache.get_num_active() == I
