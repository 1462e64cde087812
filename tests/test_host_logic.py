"""Host-side behaviour that needs no GPU: loud failure without the HIP path, synthetic generators."""
import numpy as np
import pytest
import torch

import sparse_transformers_amd as st
from sparse_transformers_amd import _lib, synthetic as syn


def test_cpu_tensors_are_refused():
    H, n = 16, 4
    x = torch.randn(1, H)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        st.sparse_mlp_forward(x, torch.randn(2 * n, H), torch.randn(n, H).t(), torch.zeros(1, H), torch.zeros(1, 2),
                              "silu")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        st.WeightCache(torch.ones(8, dtype=torch.bool), H, torch.randn(8, H), torch.randn(8, H), torch.randn(H, 8))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        st.predictor_mask(x, torch.randn(4, H), torch.randn(8, 4))


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libsparse_mlp_amd.so")
    with pytest.raises(_lib.NativeLibraryMissing, match="no CPU fallback"):
        _lib.lib()


def test_product_never_imports_the_oracle():
    import os
    root = os.path.dirname(os.path.abspath(st.__file__))
    for dirpath, _, files in os.walk(root):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text and "liboracle" not in text, f


def test_mask_trace_properties():
    tr = syn.mask_trace(1, 3, 512, 180, 40, 0.05, 0.15)
    assert tr.shape == (40, 3, 512) and tr.dtype == bool
    assert (tr.sum(-1) == 180).all()
    changed = (tr[1:] & ~tr[:-1]).sum(-1) / 180.0
    assert changed.min() >= 0.04 and changed.max() <= 0.16
    assert np.array_equal(tr, syn.mask_trace(1, 3, 512, 180, 40, 0.05, 0.15))  # seeded


def test_overlapping_token_masks():
    m = syn.overlapping_token_masks(2, 8192, 8, 2457, 0.6)
    assert (m.sum(1) == 2457).all()
    core = m.all(0).sum()
    assert core >= round(0.6 * 2457)
    assert 5500 < m.any(0).sum() < 7000   # union over 8 tokens, about 6300 expected


def test_threshold_guard_band():
    rng = np.random.default_rng(0)
    s = rng.standard_normal(8192)
    thr = syn.threshold_for_fraction(s, 0.35, guard=1e-7)
    frac = (s >= thr).mean()
    assert abs(frac - 0.35) < 0.002
    assert np.min(np.abs(s - thr)) >= 1e-7


def test_workloads_match_reference_shapes():
    w = syn.WORKLOADS["llama3b_stack_fp16"]
    assert (w.layers, w.hidden, w.intermediate, w.rank, w.n_active) == (28, 3072, 8192, 128, 2867)
    assert syn.WORKLOADS["mistral7b_stack_bf16"].n_active == 3584
    assert syn.WORKLOADS["relullama7b_stack_fp16"].rank == int(0.04 * 11008)


def test_predictor_checkpoints_round_trip(tmp_path):
    """Predictor files as the reference's trainer writes them (state dict with down.weight [r,H] and up.weight
    [I,r], src/trainer.py:570-585) load back, by the reference's file names, without executing anything."""
    import torch
    import sparse_transformers_amd as st

    H, I, r = 32, 96, 8
    want = []
    for layer in range(3):
        sd = {"down.weight": torch.randn(r, H), "up.weight": torch.randn(I, r)}
        name = st.FastLoRAProjection.checkpoint_name(layer, 4.0)
        assert name == f"final_predictor_layer_{layer}_lora_4.0pct.pt"
        torch.save(sd, tmp_path / name)
        want.append(sd)
    preds = st.load_predictors(str(tmp_path), 3, 4.0, device="cpu", dtype=torch.float16)
    for p, sd in zip(preds, want):
        assert p.lora_size == r and p.hidden_size == H and p.intermediate_size == I
        assert torch.equal(p.down_weight, sd["down.weight"].half()) and torch.equal(p.up_weight, sd["up.weight"].half())


def test_layer_constants_from_sparsity():
    """SkipDecoderLayer.__init__ (src/modeling_skip.py:134-143): the top-k count follows the *hidden* size and the
    statistical multiplier is the standard normal quantile at the sparsity (checked against scipy's ppf)."""
    from types import SimpleNamespace
    from scipy.stats import norm

    cache = SimpleNamespace(hidden_size=3072, intermediate_size=8192, device=torch.device("cpu"))
    pred = SimpleNamespace()
    layer = st.SparseDecodeLayer.from_sparsity(pred, cache, 0.65, "topk")
    assert (layer.method, layer.k) == ("topk", int(3072 * (1 - 0.65))) and layer.k == 1075
    layer = st.SparseDecodeLayer.from_sparsity(pred, cache, 0.9, "statistical_topk")
    assert layer.method == "statistical_topk" and abs(layer.std_multiplier - norm.ppf(0.9)) < 1e-6
    assert st.SparseDecodeLayer.from_sparsity(pred, cache, 0.5, "statistical_topk").std_multiplier == 0.0
    layer = st.SparseDecodeLayer.from_sparsity(pred, cache, 0.7)
    assert (layer.method, layer.k, layer.std_multiplier) == ("naive", 0, 0.0)
    with pytest.raises(ValueError):
        st.SparseDecodeLayer.from_sparsity(pred, cache, 0.7, "magnitude")


def test_bench_refuses_more_than_one_gpu():
    """bench.py --gpus N with N > 1 exits with a message before anything touches a GPU."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120, cwd=root)
    assert p.returncode != 0 and "ONE GPU" in p.stderr


def test_traffic_table_was_measured_on_these_sources():
    """profiles/hbm_traffic.md: the rows bench.py reads carry the hash of the HIP sources they were measured on; a
    change to the sources without a new measurement would silently drop `roofline.traffic` from the bench line."""
    import importlib.util
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_for_hash", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    for wl in ("llama3b_stack_fp16", "mistral7b_stack_bf16", "relullama7b_stack_fp16"):
        nbytes, source = bench.measured_traffic(wl, "cache_update_decode", 1)
        assert nbytes is not None and nbytes > 0, (wl, source)


def test_surplus_removal_closed_form():
    """The closed form the fused update + decode kernel uses when removals outnumber additions, against the
    reference's sequential rule (weight_cache.h:310-353: each surplus index, ascending, is replaced by the then-last
    entry of the list).  With S surplus indices the list ends as its first n - S positions; step k moves the entry
    of tail slot S-1-k to where the k-th surplus index sits at that time, which differs from its start position
    only when that start lies in the tail: then it sits where the step that took its slot's entry put it."""
    import oracle

    def closed_form(order, surplus_sorted):
        n, S = len(order), len(surplus_sorted)
        base = n - S
        rank = {e: k for k, e in enumerate(surplus_sorted)}
        place = [None] * S                       # place[k]: where step k puts the entry it moves (None: nothing moves)
        for p, e in enumerate(order):
            if e in rank:
                place[rank[e]] = p
        for k in range(S):                       # only indices that start in the tail need the chase
            pos = place[k]
            while pos >= base and S - 1 - (pos - base) < k:
                pos = place[S - 1 - (pos - base)]
            place[k] = None if pos >= base and S - 1 - (pos - base) == k else pos
        out = list(order)
        for s in range(S):                       # every surviving tail entry on its own
            if order[base + s] in rank:
                continue
            pos = place[S - 1 - s]
            while pos >= base:
                pos = place[S - 1 - (pos - base)]
            out[pos] = order[base + s]
        return out[:base]

    rng = np.random.default_rng(0)
    for trial in range(20000):
        n = int(rng.integers(2, 48))
        S = int(rng.integers(1, n))               # at least one index stays
        I = 64
        order = rng.permutation(I)[:n]
        mask = np.zeros(I, bool)
        mask[order] = True
        # (an arbitrary order cannot be put into the oracle's cache directly: the sequential rule is restated here,
        # and the closed form is checked against the oracle itself further down)
        surplus = np.sort(rng.choice(order, S, replace=False))
        lst, m = list(order), n
        pos = {e: i for i, e in enumerate(lst)}
        for e in surplus:
            p, last = pos[e], m - 1
            if p != last:
                lst[p] = lst[last]
                pos[lst[p]] = p
            m -= 1
        assert closed_form(list(order), list(surplus)) == lst[:m], (trial, order, surplus)
    # the sequential rule itself against the oracle: removals only, from the ascending initial order
    for trial in range(200):
        I = 40
        mask = rng.random(I) < 0.7
        if mask.sum() < 3:
            continue
        w = np.zeros((I, 8), np.float32)
        oc = oracle.OracleWeightCache(mask, 8, w, w, np.zeros((8, I), np.float32), True)
        order = oc.get_active_indices().tolist()
        drop = np.sort(rng.choice(order, int(rng.integers(1, len(order))), replace=False))
        m2 = mask.copy()
        m2[drop] = False
        oc.update_active_weights(m2)
        assert closed_form(order, list(drop)) == oc.get_active_indices().tolist(), trial


def test_surplus_removal_tail_only_form():
    """The form of the surplus removals that one wave of the fused update + decode kernel works out from the tail of
    the list alone (S surplus indices: the last S entries), against the reference's sequential rule
    (weight_cache.h:248-277 pairs in place, :310-353 each surplus index, ascending, replaced by the then-last entry).
    `kernel_form` follows the kernel step by step: the tail scan, the rounds that resolve the surplus indices which
    start in the tail (lanes of a round see the state before the round), the entries that travel until a step takes
    them below the tail, and the chain a position follows through `land`."""
    NONE, OUT, POP, UNRES = 0xffff, 0xfffe, 0xfffd, 0xfffc
    MARK = 0x8000

    def sequential(order, removed_sorted, added_sorted):
        """weight_cache.h:248-353 restated: pairs in place, then surplus removals by swap-with-last."""
        lst = list(order); na, nr = len(added_sorted), len(removed_sorted)
        pos = {e: i for i, e in enumerate(lst)}
        for i in range(min(na, nr)):
            p = pos.pop(removed_sorted[i]); lst[p] = added_sorted[i]; pos[added_sorted[i]] = p
        m = len(lst)
        for e in removed_sorted[na:]:
            p, last = pos[e], m - 1
            if p != last:
                lst[p] = lst[last]; pos[lst[p]] = p
            m -= 1
        return lst[:m]

    def kernel_form(order, removed_sorted, added_sorted, group=64):
        n, na, nr = len(order), len(added_sorted), len(removed_sorted)
        S = nr - na; base = n - S
        rank = {e: i for i, e in enumerate(removed_sorted)}
        T = [0] * S; loc = [NONE] * S
        for j in range(S):
            e = order[base + j]
            if e in rank:
                r = rank[e]
                if r < na: T[j] = added_sorted[r]
                else: T[j] = MARK | (r - na); loc[r - na] = j
            else: T[j] = e
        jlist = [k for k in range(S) if loc[k] != NONE]
        jres = [UNRES if loc[k] != NONE else NONE for k in range(S)]
        land = [NONE] * S
        rounds_max = 0
        for j0 in range(0, len(jlist), group):
            grp = jlist[j0:j0 + group]; open_ = set(grp); rounds = 0
            while open_:
                rounds += 1
                writes = []
                for kk in sorted(open_):
                    pos = loc[kk]; res = None
                    for _ in range(S + 1):
                        i = S - 1 - pos
                        if i > kk: res = pos; break
                        if i == kk: res = POP; break
                        if loc[i] == NONE or jres[i] == OUT: writes.append(('land', i, MARK | kk)); res = OUT; break
                        if jres[i] == UNRES: break
                        assert jres[i] < S
                        pos = jres[i]
                    if res is not None: writes.append(('jres', kk, res))
                for w, a, b in writes:      # lanes of a round see the state before the round
                    if w == 'land': land[a] = b
                    else: jres[a] = b; open_.discard(a)
                assert rounds <= group + 1
            rounds_max = max(rounds_max, rounds)
        for s in range(S):
            v = T[s]
            if v & MARK: continue
            k = S - 1 - s
            for _ in range(S + 1):
                if loc[k] == NONE or jres[k] == OUT: land[k] = v; break
                assert jres[k] < S, (jres[k], k)
                k = S - 1 - jres[k]
            else: raise AssertionError
        out = []
        for p in range(base):
            e = order[p]
            if e in rank:
                r = rank[e]
                if r < na: out.append(added_sorted[r])
                else:
                    v = land[r - na]
                    for _ in range(S + 1):
                        if not (v & MARK): break
                        assert v != NONE
                        v = land[v & (MARK - 1)]
                    assert not (v & MARK)
                    out.append(v)
            else: out.append(e)
        return out, rounds_max

    rng = np.random.default_rng(0)
    worst = 0
    for trial in range(12000):
        I = int(rng.choice([16, 64, 300]))
        n = int(rng.integers(2, min(I, 200)))
        order = rng.permutation(I)[:n].tolist()
        nr = int(rng.integers(1, n + 1))
        mode = rng.integers(0, 4)
        if mode == 0:
            removed = rng.choice(order, nr, replace=False)
        elif mode == 1:
            removed = np.array(order[n - nr:])               # the tail itself
        elif mode == 2:
            removed = np.array(sorted(order)[-nr:])          # the largest indices
        else:                                                # mostly the tail
            removed = np.array([e if rng.random() < 0.7 else order[int(rng.integers(0, n))] for e in order[n - nr:]])
        removed = np.sort(np.unique(removed)).tolist()
        nr = len(removed)
        free = sorted(set(range(I)) - set(order))
        na = int(rng.integers(0, min(nr, len(free) + 1)))    # na < nr: at least one surplus removal
        added = sorted(rng.choice(free, na, replace=False).tolist()) if na else []
        want = sequential(order, removed, added)
        got, rounds = kernel_form(order, removed, added, group=int(rng.choice([2, 4, 64])))
        worst = max(worst, rounds)
        assert got == want, (trial, order, removed, added)
    assert worst >= 3      # the cases did reach chains of dependent surplus indices
