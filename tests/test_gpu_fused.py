"""Cache update fused into the decode kernel (st_cache_update_forward) vs the two separate calls.

The fused kernel takes the rows whose index changed from the pool and writes them back on the way, so the
cache must end in exactly the state update_active_weights leaves (ordered list, counts, active rows), and its
arithmetic is that of the decode kernel, so the output must carry the same bits."""
import numpy as np
import pytest
import torch

import oracle
import sparse_transformers_amd as st
from sparse_transformers_amd import synthetic as syn
from conftest import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _pair(I, H, dtype, has_gate, seed, init_mask, std=0.05):
    g = torch.Generator().manual_seed(seed)
    tdt = getattr(torch, dtype)
    gate = (torch.randn(I, H, generator=g) * std).to(tdt)
    up = (torch.randn(I, H, generator=g) * std).to(tdt)
    down = (torch.randn(H, I, generator=g) * std).to(tdt)
    mk = lambda: st.WeightCache(init_mask.to(DEV), H, gate.to(DEV) if has_gate else None, up.to(DEV), down.to(DEV),
                                has_gate)
    return mk(), mk(), (gate, up, down), g


def _same_state(a, b, step):
    sa, sb = a.sync_state(), b.sync_state()
    for key in ("n_active", "n_changed", "n_added", "n_removed", "status", "valid"):
        assert sa[key] == sb[key], (step, key, sa, sb)
    n = sa["n_active"]
    assert torch.equal(a.get_active_indices(), b.get_active_indices()), step
    assert torch.equal(a.up_active[:n], b.up_active[:n]) and torch.equal(a.down_active[:n], b.down_active[:n]), step
    if a.has_gate:
        assert torch.equal(a.gate_active[:n], b.gate_active[:n]), step
    ea, eb = int(sa["epoch"]), int(sb["epoch"])
    assert torch.equal(a.cur_mask[ea], b.cur_mask[eb]), step


# I = 4096 / 9216 with about half the rows active: enough rows per block for the kernel variants that split the
# waves' roles
@pytest.mark.parametrize("dtype,H,I", [("float16", 3072, 4096), ("bfloat16", 1024, 4096), ("float32", 2048, 4096),
                                       ("float16", 4096, 4096), ("float16", 2048, 9216)])
@pytest.mark.parametrize("has_gate", [True, False])
def test_fused_equals_update_then_forward(dtype, H, I, has_gate):
    rng = np.random.default_rng(5)
    trace = syn.ragged_mask_trace(11 + H, I, 40)      # growth, shrinkage (sequential removals), no-ops, tiny sets
    fused, plain, (gate, up, down), g = _pair(I, H, dtype, has_gate, 3, torch.from_numpy(trace[0]))
    tdt = getattr(torch, dtype)
    for t in range(1, len(trace)):
        if not trace[t].any():
            continue
        m = torch.from_numpy(trace[t]).to(DEV)
        x = torch.randn(1, H, generator=g).to(tdt).to(DEV)
        comb_f = torch.zeros(1, 2 * I, dtype=tdt, device=DEV)
        comb_p = torch.zeros_like(comb_f)
        yf = fused.update_and_forward(m, x, "silu", combined=comb_f)
        plain.update_active_weights_async(m)
        yp = plain.forward(x, "silu", combined=comb_p)
        torch.cuda.synchronize()
        assert torch.equal(yf, yp), (t, (yf.float() - yp.float()).abs().max().item())
        assert torch.equal(comb_f, comb_p), t
        _same_state(fused, plain, t)
    # and against the oracle at the end: order, then the MLP on the final active set
    oc = oracle.OracleWeightCache(trace[0], H, gate.float().numpy() if has_gate else None, up.float().numpy(),
                                  down.float().numpy(), has_gate)
    for t in range(1, len(trace)):
        if trace[t].any():
            oc.update_active_weights(trace[t])
    assert fused.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist()
    want, _ = oracle.mlp_forward(x.float().cpu().numpy(), oc.get_concat_weight(), oc.get_active_down_weight(), "silu",
                                 has_gate)
    assert_close(yf.float().cpu().numpy(), want, dtype, "fused output vs oracle")


def test_fused_full_size_trace_and_errors():
    """The Llama-3.2-3B layer shape (H 3072, I 8192, 35 % active) with 5-15 % churn, then the corner cases: unchanged mask, an update that empties the
    cache (status reported at the next sync, zeros out), recovery from empty."""
    H, I, n = 3072, 8192, 2867
    trace = syn.mask_trace(21, 1, I, n, 12, 0.05, 0.15)[:, 0]
    fused, plain, _, g = _pair(I, H, "float16", True, 9, torch.from_numpy(trace[0]))
    x = torch.randn(1, H, generator=g).half().to(DEV)
    for t in range(1, len(trace)):
        m = torch.from_numpy(trace[t]).to(DEV)
        yf = fused.update_and_forward(m, x, "silu")
        plain.update_active_weights_async(m)
        yp = plain.forward(x, "silu")
        assert torch.equal(yf, yp), t
    _same_state(fused, plain, "trace end")
    # unchanged mask: nothing moves, same output again
    y2 = fused.update_and_forward(m, x, "silu")
    assert torch.equal(y2, yf) and fused.sync_state()["n_changed"] == 0
    # all-false mask: reference raises "No active weights" (weight_cache.h:117-118); here at the next sync
    none = torch.zeros(I, dtype=torch.bool, device=DEV)
    y0 = fused.update_and_forward(none, x, "silu")
    with pytest.raises(RuntimeError, match="No active weights"):
        fused.sync_state()
    assert torch.count_nonzero(y0).item() == 0
    with pytest.raises(RuntimeError, match="No active weights"):
        plain.update_active_weights(none)
    # the remembered mask survives the failed update (weight_cache.h:356-358 is never reached), so the same
    # mask again is "unchanged" and the cache stays empty; a different mask re-adds only what differs from it
    y0 = fused.update_and_forward(m, x, "silu")
    with pytest.raises(RuntimeError, match="No active weights"):
        fused.sync_state()
    assert torch.count_nonzero(y0).item() == 0
    m2 = m.clone()
    m2[(~m).nonzero().flatten()[:100]] = True       # 100 additions, no removals
    yf = fused.update_and_forward(m2, x, "silu")
    plain.update_active_weights_async(m2)
    yp = plain.forward(x, "silu")
    assert torch.equal(yf, yp)
    _same_state(fused, plain, "after recovery")
    assert fused.get_num_active() == 100


@pytest.mark.parametrize("dtype,H,I,B,has_gate", [
    ("bfloat16", 2048, 1024, 4, True), ("float16", 3072, 8192, 3, True), ("float16", 3072, 8192, 16, True),
    ("bfloat16", 4096, 14336, 8, True), ("float16", 4096, 11008, 4, False), ("bfloat16", 3072, 4096, 20, True),
    ("float16", 2048, 4096, 32, False), ("float32", 2048, 1024, 4, True), ("float16", 1024, 4096, 4, True)])
def test_fused_several_rows_of_x(dtype, H, I, B, has_gate):
    """3 <= B <= 32 rows of x through update_and_forward (one C call that enqueues the update and the MFMA batch
    kernels, or the streaming kernels where those do not apply, with the count read on the device).  Result,
    combined buffer and the cache state equal the two separate calls, bit for bit, over a ragged trace (growth,
    shrinkage with surplus removals, no-ops, tiny sets); order and output against the oracle at the end."""
    trace = syn.ragged_mask_trace(3 + H + B, I, 14)
    # (weights small enough that the outputs are O(1): the absolute tolerance of the 16-bit types assumes that)
    fused, plain, (gate, up, down), g = _pair(I, H, dtype, has_gate, 1, torch.from_numpy(trace[0]), std=0.012)
    tdt = getattr(torch, dtype)
    ncol = (2 if has_gate else 1) * I
    for t in range(1, len(trace)):
        if not trace[t].any():
            continue
        m = torch.from_numpy(trace[t]).to(DEV)
        x = torch.randn(B, H, generator=g).to(tdt).to(DEV)
        comb_f = torch.zeros(B, ncol, dtype=tdt, device=DEV)
        comb_p = torch.zeros_like(comb_f)
        yf = fused.update_and_forward(m, x, "silu", combined=comb_f)
        plain.update_active_weights_async(m)
        yp = plain.forward(x, "silu", combined=comb_p)
        torch.cuda.synchronize()
        assert torch.equal(yf, yp), (t, (yf.float() - yp.float()).abs().max().item())
        assert torch.equal(comb_f, comb_p), t
        _same_state(fused, plain, t)
    oc = oracle.OracleWeightCache(trace[0], H, gate.float().numpy() if has_gate else None, up.float().numpy(),
                                  down.float().numpy(), has_gate)
    for t in range(1, len(trace)):
        if trace[t].any():
            oc.update_active_weights(trace[t])
    assert fused.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist()
    want, _ = oracle.mlp_forward(x.float().cpu().numpy(), oc.get_concat_weight(), oc.get_active_down_weight(), "silu",
                                 has_gate)
    assert_close(yf.float().cpu().numpy(), want, dtype, "fused batch output vs oracle")


@pytest.mark.parametrize("dtype,H,I,n0", [("float16", 3072, 8192, 2867), ("bfloat16", 4096, 4096, 400),
                                          ("float32", 2048, 4096, 1500),
                                          # seven rows per thread group: the variants with seven rows in flight
                                          ("bfloat16", 4096, 14336, 3584), ("float16", 3072, 8192, 3500)])
def test_fused_result_does_not_depend_on_the_hint(dtype, H, I, n0):
    """The caller's guess of the active count decides which kernel variant runs, what is requested before
    the plan is known and how much of the index list is fetched up front; a wrong guess (far too low: the
    rest of the list is fetched in a second round trip; far too high; zero = unknown) must change nothing."""
    rng = np.random.default_rng(17)
    m = np.zeros(I, bool)
    m[rng.permutation(I)[:n0]] = True
    fused, plain, _, g = _pair(I, H, dtype, True, 5, torch.from_numpy(m))
    tdt = getattr(torch, dtype)
    for step, hint in enumerate((0, 1, 8, n0 // 3, n0 - 1, n0, n0 + 1000, I, 2 * I, 40, n0)):
        flip = rng.permutation(I)[: max(2, n0 // 8)]
        m = m.copy()
        m[flip] = ~m[flip]
        md = torch.from_numpy(m).to(DEV)
        x = torch.randn(1, H, generator=g).to(tdt).to(DEV)
        yf = fused.update_and_forward(md, x, "silu", n_hint=hint)
        plain.update_active_weights_async(md)
        yp = plain.forward(x, "silu")
        torch.cuda.synchronize()
        assert torch.equal(yf, yp), (step, hint)
        _same_state(fused, plain, step)


@pytest.mark.parametrize("dtype,H,I", [("float16", 3072, 4096), ("bfloat16", 4096, 4096), ("float32", 2048, 4096),
                                       ("float16", 1024, 4096)])
@pytest.mark.parametrize("has_gate", [True, False])
def test_fused_two_rows_of_x(dtype, H, I, has_gate):
    """Two rows of x go through the fused kernel too (one pass over the rows for both): result, the
    combined buffer and the cache state equal update followed by forward, bit for bit, over a ragged trace;
    and each row equals what the same row gives on its own."""
    trace = syn.ragged_mask_trace(23 + H, I, 24)
    fused, plain, _, g = _pair(I, H, dtype, has_gate, 7, torch.from_numpy(trace[0]))
    single, _, _, _ = _pair(I, H, dtype, has_gate, 7, torch.from_numpy(trace[0]))
    tdt = getattr(torch, dtype)
    for t in range(1, len(trace)):
        if not trace[t].any():
            continue
        m = torch.from_numpy(trace[t]).to(DEV)
        x = torch.randn(2, H, generator=g).to(tdt).to(DEV)
        comb_f = torch.zeros(2, 2 * I, dtype=tdt, device=DEV)
        comb_p = torch.zeros_like(comb_f)
        yf = fused.update_and_forward(m, x, "silu", combined=comb_f)
        plain.update_active_weights_async(m)
        yp = plain.forward(x, "silu", combined=comb_p)
        single.update_active_weights_async(m)
        y0, y1 = single.forward(x[0:1], "silu").clone(), single.forward(x[1:2], "silu").clone()
        torch.cuda.synchronize()
        assert torch.equal(yf, yp), (t, (yf.float() - yp.float()).abs().max().item())
        assert torch.equal(comb_f, comb_p), t
        assert torch.equal(yf[0:1], y0) and torch.equal(yf[1:2], y1), t
        if t % 6 == 0:
            _same_state(fused, plain, t)
    _same_state(fused, plain, "end")


@pytest.mark.parametrize("I,n0,hint_slack", [(4096, 2000, 0), (8192, 2867, 0), (512, 300, 0), (4096, 2000, -600),
                                             # the largest size the fused kernel takes: 64 positions per block
                                             (16384, 5000, 0)])
def test_fused_surplus_removals(I, n0, hint_slack):
    """More indices removed than added (weight_cache.h:310-353, swap with the last entry, one by one): the
    fused kernel places the entries of the list's end in one go.  Surpluses of 1 .. I/4 and beyond (the
    per-index plan takes over), removed indices drawn from all over the list, mostly from its end (surplus
    indices that sit in the last positions themselves travel with earlier moves), or ONLY from its end;
    with and without additions; a hint too low to fetch the list up front.  Order, counts, rows and output
    against update followed by forward, and the order against the oracle."""
    H, dtype = 1024, "float16"
    rng = np.random.default_rng(I + n0)
    m = np.zeros(I, bool)
    m[rng.permutation(I)[:n0]] = True
    fused, plain, (gate, up, down), g = _pair(I, H, dtype, True, 9, torch.from_numpy(m))
    oc = oracle.OracleWeightCache(m, H, gate.float().numpy(), up.float().numpy(), down.float().numpy(), True)
    x = torch.randn(1, H, generator=g).half().to(DEV)
    plans = [(1, 0, "any"), (5, 3, "end"), (40, 40, "end"), (64, 10, "only_end"), (65, 0, "any"), (300, 50, "end"),
             (I // 4, 0, "end"), (I // 4 + 1, 7, "any"), (17, 200, "only_end"), (2, 0, "only_end"), (120, 0, "only_end")]
    for step, (surplus, added, where) in enumerate(plans):
        order = oc.get_active_indices()
        n = order.size
        if n < n0 // 2:                  # grow the set back (additions only), then go on
            grow = rng.permutation(np.flatnonzero(~m))[: n0 - n]
            m = m.copy(); m[grow] = True
            md = torch.from_numpy(m).to(DEV)
            fused.update_and_forward(md, x, "silu"); plain.update_active_weights_async(md); oc.update_active_weights(m)
            order = oc.get_active_indices(); n = order.size
        surplus, added = min(surplus, n // 3), min(added, n // 8, I - n0)
        k = surplus + added
        if where == "any":
            out = rng.choice(order, k, replace=False)
        elif where == "end":          # three quarters of them from the last 2k positions
            end = order[max(0, n - 2 * k):]
            take = rng.choice(end, min(end.size, (3 * k) // 4), replace=False)
            rest = np.setdiff1d(order, take)
            out = np.concatenate([take, rng.choice(rest, k - take.size, replace=False)])
        else:                         # all of them among the last positions
            out = rng.choice(order[n - min(n, k + k // 4 + 1):], k, replace=False)
        m = m.copy()
        m[out] = False
        m[rng.permutation(np.flatnonzero(~m & ~np.isin(np.arange(I), out)))[:added]] = True
        md = torch.from_numpy(m).to(DEV)
        hint = max(0, n + hint_slack)
        yf = fused.update_and_forward(md, x, "silu", n_hint=hint)
        plain.update_active_weights_async(md)
        yp = plain.forward(x, "silu")
        oc.update_active_weights(m)
        torch.cuda.synchronize()
        assert torch.equal(yf, yp), (step, surplus, added, where)
        _same_state(fused, plain, (step, surplus, added, where))
        assert fused.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist(), (step, where)
        assert fused.sync_state()["n_removed"] - fused.sync_state()["n_added"] == surplus


@pytest.mark.parametrize("I,H,dtype,has_gate,frac", [
    (8192, 256, "float16", True, 0.35), (4096, 256, "bfloat16", False, 0.5), (16384, 256, "float16", True, 0.25),
    (1000, 128, "float16", True, 0.3), (14336, 256, "bfloat16", True, 0.25), (11008, 512, "float16", True, 0.1),
])
def test_fused_random_count_changes(I, H, dtype, has_gate, frac):
    """Random walks of the mask as a predictor's threshold produces them: the count drifts by a few percent per step
    (more removals than additions in about half the steps), jumps by up to 30 % now and then, stays put, or lands
    anywhere in 1 .. I; 0-40 % of the active set is swapped on top.  After every step the ordered list equals the
    oracle's, and every seventh step the output carries the same bits as update followed by forward."""
    for seed in (300, 301):
        rng = np.random.default_rng(seed)
        tdt = getattr(torch, dtype)
        m = syn.initial_mask(rng, I, max(1, int(frac * I)))
        fused, plain, (gate, up, down), g = _pair(I, H, dtype, has_gate, seed, torch.from_numpy(m))
        oc = oracle.OracleWeightCache(m, H, gate.float().numpy() if has_gate else None, up.float().numpy(),
                                      down.float().numpy(), has_gate)
        n0 = int(m.sum())
        for t in range(150):
            kind, cur = int(rng.integers(0, 10)), int(m.sum())
            if kind < 6:
                target = int(round(cur * (1.0 + rng.uniform(-0.08, 0.08))))
            elif kind < 8:
                target = int(round(n0 * (1.0 + rng.uniform(-0.3, 0.3))))
            elif kind == 8 or rng.random() >= 0.3:
                target = cur
            else:
                target = int(rng.integers(1, I + 1))
            m = syn.churn_step(rng, m, float(rng.choice([0.0, 0.02, 0.1, 0.15, 0.4])), max(1, min(I, target)))
            mt = torch.from_numpy(m).to(DEV)
            x = torch.randn(1, H, generator=g).to(tdt).to(DEV)
            yf = fused.update_and_forward(mt, x, "silu")
            oc.update_active_weights(m)
            assert fused.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist(), (seed, t, cur, target)
            plain.update_active_weights_async(mt)
            if t % 7 == 0:
                yp = plain.forward(x, "silu")
                torch.cuda.synchronize()
                assert torch.equal(yf, yp), (seed, t)
