"""Pins the CPU oracle (oracle/sparse_mlp_oracle.c): golden vectors written from the reference's own
compiled C++, the compiled reference itself when oracle/_ref is present, float64 closed forms with
numpy, and structural invariants.  Runs without a GPU."""
import numpy as np
import pytest

import oracle
from conftest import bits_to_mask, golden_weights


# ------------------------------------------------------------------ cache: golden traces
def _replay(trace, cache_factory):
    I, H, hg = trace["I"], trace["H"], trace["has_gate"]
    gate, up, down = golden_weights(I, H)
    c = cache_factory(bits_to_mask(trace["init_mask"]), H, gate if hg else None, up, down, hg)
    yield None, c, trace["init_order"]
    for step in trace["steps"]:
        yield step, c, step.get("order")


def test_cache_matches_reference_traces(golden_traces):
    n_err = n_noop = n_swap = 0
    for trace in golden_traces:
        I, H, hg = trace["I"], trace["H"], trace["has_gate"]
        gate, up, down = golden_weights(I, H)
        prev = None
        for step, c, order in _replay(trace, oracle.OracleWeightCache):
            if step is not None:
                m = bits_to_mask(step["mask"])
                if step["error"]:
                    with pytest.raises(RuntimeError, match="No active weights"):
                        c.update_active_weights(m)
                    n_err += 1
                    continue
                c.update_active_weights(m)
                n_noop += prev is not None and step["mask"] == prev
                prev = step["mask"]
            got = c.get_active_indices().tolist()
            assert got == order, (trace["seed"], got[:10], order[:10])
            n = len(order)
            n_swap += n > 0 and sorted(order) != order
            cw = c.get_concat_weight()
            if hg:
                assert np.array_equal(cw[:n], gate[order])
            assert np.array_equal(cw[-n:], up[order])
            dw = c.get_active_down_weight()
            assert dw.shape == (H, n) and dw.strides == (4, 4 * H)
            assert np.array_equal(dw, down[:, order])
    assert n_err >= 3 and n_noop >= 3 and n_swap > 50  # the fixtures really exercise those paths


def test_cache_worked_trace_from_reference():
    """Trace verified on the compiled reference (I=16): drop {1,3,5,7,9}, then add {1,3} / drop {0,2,4}."""
    I, H = 16, 2
    gate, up, down = golden_weights(I, H)
    c = oracle.OracleWeightCache(np.ones(I, bool), H, gate, up, down, True)
    assert c.get_active_indices().tolist() == list(range(16))
    m = np.ones(I, bool)
    m[[1, 3, 5, 7, 9]] = False
    c.update_active_weights(m)
    assert c.get_active_indices().tolist() == [0, 15, 2, 14, 4, 13, 6, 12, 8, 11, 10]
    m[[1, 3]] = True
    m[[0, 2, 4]] = False
    c.update_active_weights(m)
    assert c.get_active_indices().tolist() == [1, 15, 3, 14, 10, 13, 6, 12, 8, 11]


def test_cache_against_compiled_reference_random():
    ref = oracle.load_reference()
    if ref is None:
        pytest.skip("oracle/_ref not built (needs the reference checkout)")
    import torch
    WC = ref[0]
    rng = np.random.default_rng(3)
    for trial in range(12):
        I, H, hg = int(rng.integers(2, 90)), int(rng.integers(1, 7)), bool(trial % 3)
        g = rng.standard_normal((I, H)).astype(np.float32)
        u = rng.standard_normal((I, H)).astype(np.float32)
        d = rng.standard_normal((H, I)).astype(np.float32)
        init = rng.random(I) < 0.7
        init[0] = True
        oc = oracle.OracleWeightCache(init, H, g if hg else None, u, d, hg)
        rc = WC(torch.from_numpy(init), H, torch.from_numpy(g) if hg else None, torch.from_numpy(u),
                torch.from_numpy(d), hg)
        m = init.copy()
        cur, stale = init.copy(), False   # model of the reference's current_mask / "views are stale"
        for step in range(150):
            m = m ^ (rng.random(I) < rng.choice([0.02, 0.2, 0.6]))
            if step % 13 == 7:
                m = np.zeros(I, bool)
            if step % 13 == 9:
                m = cur.copy()
            e1 = e2 = None
            try:
                oc.update_active_weights(m)
            except RuntimeError as e:
                e1 = str(e)
            try:
                rc.update_active_weights(torch.from_numpy(m))
            except RuntimeError as e:
                e2 = "No active weights" if "No active weights" in str(e) else str(e)
            assert e1 == e2, (trial, step, e1, e2)
            noop = np.array_equal(m, cur)
            if e1 is not None:
                stale = True          # the reference now hands out the tensors of the last good update
            elif not noop:
                cur, stale = m.copy(), False
            if e1 is None and not stale:
                assert np.array_equal(rc.get_concat_weight().numpy(), oc.get_concat_weight()), (trial, step)
                assert np.array_equal(rc.get_active_down_weight().numpy(), oc.get_active_down_weight())


def test_cache_invariants_large():
    """Size-independent properties at a realistic intermediate size."""
    rng = np.random.default_rng(5)
    I, H = 8192, 8
    g = rng.standard_normal((I, H)).astype(np.float32)
    u = rng.standard_normal((I, H)).astype(np.float32)
    d = rng.standard_normal((H, I)).astype(np.float32)
    c = oracle.OracleWeightCache(np.ones(I, bool), H, g, u, d, True)
    m = np.ones(I, bool)
    for step in range(30):
        m = m ^ (rng.random(I) < 0.1)
        c.update_active_weights(m)
        idx = c.get_active_indices()
        assert len(idx) == int(m.sum()) and np.array_equal(np.sort(idx), np.flatnonzero(m))
        cw = c.get_concat_weight()
        assert np.array_equal(cw[:len(idx)], g[idx]) and np.array_equal(cw[len(idx):], u[idx])
        assert np.array_equal(c.get_active_down_weight(), d[:, idx])


# ------------------------------------------------------------------ forward
def _act64(v, act):
    if act == "relu":
        return np.maximum(v, 0.0)
    if act == "silu":
        return v / (1.0 + np.exp(-v))
    if act == "sigmoid":
        return 1.0 / (1.0 + np.exp(-v))
    if act == "gelu_pytorch_tanh":
        return 0.5 * v * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (v + 0.044715 * v ** 3)))
    return v


def test_forward_matches_reference_operator_vectors(golden_mlp):
    for case in golden_mlp:
        B, H, n, hg = case["B"], case["H"], case["n"], case["has_gate"]
        x = np.array(case["x"], dtype=np.float32).reshape(case["x_shape"])
        cw = np.array(case["concat"], dtype=np.float32).reshape(-1, H)
        dn = np.array(case["down_rows"], dtype=np.float32).reshape(n, H)
        out, comb = oracle.mlp_forward(x, cw, dn.T, "relu", hg)
        want = np.array(case["out"], dtype=np.float32).reshape(case["x_shape"])
        np.testing.assert_allclose(out, want, rtol=2e-5, atol=2e-5)
        wantc = np.array(case["combined"], dtype=np.float32).reshape(case["combined_shape"])
        np.testing.assert_allclose(comb, wantc, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("act", ["relu", "silu", "gelu_pytorch_tanh", "sigmoid", "identity"])
@pytest.mark.parametrize("has_gate", [True, False])
def test_forward_closed_form_float64(act, has_gate):
    import zlib
    rng = np.random.default_rng(zlib.crc32(f"{act}-{has_gate}".encode()) % 1000)   # (hash() of a str differs per process)
    B, H, n = 3, 40, 23
    x = rng.standard_normal((B, H)).astype(np.float32)
    cw = rng.standard_normal(((2 if has_gate else 1) * n, H)).astype(np.float32)
    dn = rng.standard_normal((n, H)).astype(np.float32)
    out, comb = oracle.mlp_forward(x, cw, dn.T, act, has_gate)
    x64, cw64, dn64 = x.astype(np.float64), cw.astype(np.float64), dn.astype(np.float64)
    if has_gate:
        g, u = x64 @ cw64[:n].T, x64 @ cw64[n:].T
        h = _act64(g, act) * u
    else:
        h = _act64(x64 @ cw64.T, act)
    # (fp32 outputs of sums in double: 1e-5 of the tensor's largest element, as for the GPU's fp32 results -- an
    # element that happens to cancel to almost nothing still carries the rounding of its terms)
    want = h @ dn64
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())
    np.testing.assert_allclose(comb[:, :n], h, rtol=1e-5, atol=1e-5 * np.abs(h).max())
    # a transposed down operand, a swapped gate/up or a dropped activation would all fail here
    if has_gate and act != "identity":
        swapped = _act64(x64 @ cw64[n:].T, act) * (x64 @ cw64[:n].T)
        assert not np.allclose(out, swapped @ dn64, rtol=1e-3, atol=1e-3)


def test_forward_special_cases():
    rng = np.random.default_rng(0)
    H, n = 16, 9
    cw = rng.standard_normal((2 * n, H)).astype(np.float32)
    dn = rng.standard_normal((n, H)).astype(np.float32)
    out, _ = oracle.mlp_forward(np.zeros((2, H), np.float32), cw, dn.T, "silu", True)
    assert not out.any()                                     # silu(0) * 0
    x = rng.standard_normal((1, H)).astype(np.float32)
    a, _ = oracle.mlp_forward(x, cw, dn.T, "identity", True)
    b, _ = oracle.mlp_forward(2 * x, cw, dn.T, "identity", True)
    np.testing.assert_allclose(b, 4 * a, rtol=1e-5)          # bilinear gate*up -> degree 2
    c, _ = oracle.mlp_forward(x, cw[n:], dn.T, "identity", False)
    np.testing.assert_allclose(c, (x @ cw[n:].T) @ dn, rtol=1e-4, atol=1e-5)   # plain two-matrix product


# ------------------------------------------------------------------ predictor and masks
def test_predictor_scores_closed_form():
    rng = np.random.default_rng(2)
    B, H, r, I = 4, 96, 12, 200
    x = rng.standard_normal((B, H)).astype(np.float32)
    A = rng.standard_normal((r, H)).astype(np.float32)
    Bm = rng.standard_normal((I, r)).astype(np.float32)
    s = oracle.predictor_scores(x, A, Bm)
    want = (x.astype(np.float64) @ A.T.astype(np.float64)) @ Bm.T.astype(np.float64)
    np.testing.assert_allclose(s, want, rtol=1e-5, atol=1e-4)
    assert s.shape == (B, I)


def test_masks_against_numpy():
    rng = np.random.default_rng(4)
    B, I = 5, 300
    s = rng.standard_normal((B, I)).astype(np.float32)
    assert np.array_equal(oracle.mask_threshold(s, 0.0, True), (s >= 0).any(0))
    s[2, 17] = 0.25
    assert oracle.mask_threshold(s[2:3], 0.25, True)[17] and not oracle.mask_threshold(s[2:3], 0.25, False)[17]
    k = 40
    want = np.zeros(I, bool)
    for b in range(B):
        want[np.argsort(-s[b], kind="stable")[:k]] = True
    assert np.array_equal(oracle.mask_topk(s, k), want)
    assert oracle.mask_topk(s[:1], k).sum() == k
    z = 0.7
    m, cut = oracle.mask_statistical(s, z)
    mean, std = s.astype(np.float64).mean(1), s.astype(np.float64).std(1)  # population std, like unbiased=False
    np.testing.assert_allclose(cut, mean + std * z, rtol=1e-6)
    assert np.array_equal(m, (s > cut[:, None]).any(0))


def test_mask_bruteforce_tiny():
    s = np.array([[0.1, -0.2, 0.0], [-1.0, -0.1, -0.5]], dtype=np.float32)
    assert oracle.mask_threshold(s, 0.0, True).tolist() == [True, False, True]
    assert oracle.mask_threshold(s, 0.0, False).tolist() == [True, False, False]
    assert oracle.mask_topk(s, 1).tolist() == [True, True, False]


# ------------------------------------------------------------------ sketch threshold (approx_topk.h)
def _b64_f32(s):
    import base64

    return np.frombuffer(base64.b64decode(s), dtype="<f4").copy()


def test_approx_topk_matches_reference_vectors():
    import json
    import os

    with open(os.path.join(os.path.dirname(__file__), "golden", "approx_topk.json")) as f:
        cases = json.load(f)["cases"]
    assert len(cases) >= 8
    for c in cases:
        sc = _b64_f32(c["scores_f32_b64"]).reshape(c["B"], c["F"])
        want = _b64_f32(c["threshold_f32_b64"])
        got = oracle.approx_topk_threshold(sc, c["k"])
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (c["B"], c["F"], c["k"])


def test_approx_topk_against_compiled_reference_random():
    if oracle.load_reference() is None:
        pytest.skip("oracle/_ref not built (needs the reference checkout)")
    import torch

    op = torch.ops.sparse_mlp.approx_topk_threshold
    rng = np.random.default_rng(21)
    for F in (4, 7, 63, 64, 1000, 4096, 4097, 8192, 11008, 14336):
        for B in (1, 3):
            sc = rng.standard_normal((B, F)).astype(np.float32)
            if F % 2:
                sc = np.round(sc * 8) / 8          # ties
            for k in sorted({1, max(1, F // 10), max(1, F // 2), F}):
                want = op(torch.from_numpy(sc), k).numpy().reshape(-1)
                got = oracle.approx_topk_threshold(sc, k)
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (F, B, k)


def test_approx_topk_f64_matches_reference_vectors_and_live_reference():
    """The reference dispatches approx_topk_threshold on the scores' floating type (approx_topk.h:33): double scores
    against the vectors written from the compiled reference, and against that build itself where it is present."""
    import base64
    import json
    import os

    with open(os.path.join(os.path.dirname(__file__), "golden", "approx_topk_f64.json")) as f:
        cases = json.load(f)["cases"]
    assert len(cases) >= 6
    for c in cases:
        sc = np.frombuffer(base64.b64decode(c["scores_f64_b64"]), dtype="<f8").copy().reshape(c["B"], c["F"])
        want = np.frombuffer(base64.b64decode(c["threshold_f64_b64"]), dtype="<f8")
        got = oracle.approx_topk_threshold(sc, c["k"])
        assert got.dtype == np.float64 and np.array_equal(got, want), (c["B"], c["F"], c["k"])
    if oracle.load_reference() is None:
        return
    import torch

    op = torch.ops.sparse_mlp.approx_topk_threshold
    rng = np.random.default_rng(22)
    for F in (4, 63, 1000, 4097, 11008):
        sc = rng.standard_normal((2, F))
        if F % 2:
            sc = 1.0 + sc * 1e-13              # equal upper halves of the bit patterns
        for k in sorted({1, max(1, F // 7), F}):
            want = op(torch.from_numpy(sc), k).numpy().reshape(-1)
            assert np.array_equal(oracle.approx_topk_threshold(sc, k), want), (F, k)


def test_approx_topk_special_cases():
    # F a multiple of the sketch width: all four sketches equal the per-residue maxima, so with k = F the
    # threshold is 0.9 * the smallest of those maxima
    F, W = 64, 16
    rng = np.random.default_rng(3)
    sc = rng.standard_normal((1, F)).astype(np.float32)
    maxima = sc[0].reshape(F // W, W).max(0)
    assert oracle.approx_topk_threshold(sc, F)[0] == np.float32(maxima.min()) * np.float32(0.9)
    # k = 1: sketch_k = 1, the largest cell, which is the global maximum
    assert oracle.approx_topk_threshold(sc, 1)[0] == np.float32(sc.max()) * np.float32(0.9)
    with pytest.raises(ValueError):
        oracle.approx_topk_threshold(sc, 0)
    with pytest.raises(ValueError):
        oracle.approx_topk_threshold(sc, F + 1)
