"""The whole per-layer chain at the full shapes of the benchmark configurations, as a SEQUENCE of decode
steps: predictor-driven masks -> differential cache update -> sparse MLP, through SparseMLPStack with the
fused update + decode kernel, against the oracle pipeline on the same seeded inputs.  Checked at every
step and layer: mask bits and ordered index list exact; stack output within the dtype's tolerance.
(Order of the reference: src/modeling_skip.py:234-261; the cache semantics: weight_cache.h:229-359.)

The predictor input of a layer follows an AR(1) process (correlation rho per step), so consecutive masks
share most of their indices, and the active fraction wobbles a little around its target, so that additions
outnumber removals in some steps and removals outnumber additions in others (both branches of the update)."""
import numpy as np
import pytest
import torch

import oracle
import sparse_transformers_amd as st
from sparse_transformers_amd import synthetic as syn
from conftest import assert_close, round_to

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _threshold_in_gap(s: np.ndarray, frac: float, guard_rel: float = 4e-6, per_row: bool = False) -> float:
    """A threshold with about `frac` of the columns of s [B,I] active (any row >= t) -- with `per_row`, about `frac`
    of every row's scores -- placed in the widest gap between ALL scores near that quantile; asserts that no score
    lies within guard_rel * max|s| of it (the GPU scores differ from the oracle's by less than half of that, see
    test_gpu_predictor)."""
    a = np.sort(s.astype(np.float64).ravel())
    t0 = np.quantile((s if per_row else s.max(0)).astype(np.float64), 1.0 - frac)
    j = int(np.searchsorted(a, t0))
    lo, hi = max(1, j - 16), min(a.size - 1, j + 16)
    gaps = a[lo:hi + 1] - a[lo - 1:hi]
    g = int(np.argmax(gaps)) + lo
    thr = 0.5 * (a[g - 1] + a[g])
    assert np.min(np.abs(a - thr)) >= guard_rel * np.abs(a).max(), "no guard band around the threshold"
    return float(thr)


def _build(dtype, L, H, I, r, has_gate, act, seed):
    rng = np.random.default_rng(seed)
    tdt = getattr(torch, dtype)
    layers, oracles = [], []
    init = np.ones(I, bool)
    for _ in range(L):
        w = syn.layer_weights(rng, H, I, r, std=0.02, has_gate=has_gate)
        w = {k: (None if v is None else round_to(v, dtype)) for k, v in w.items()}
        t = {k: (None if v is None else torch.from_numpy(v).to(DEV, tdt)) for k, v in w.items()}
        cache = st.WeightCache(torch.from_numpy(init).to(DEV), H, t["gate"], t["up"], t["down"], has_gate)
        layers.append(st.SparseDecodeLayer(st.FastLoRAProjection(t["A"], t["Bm"]), cache, act, 0.0, True))
        oracles.append((oracle.OracleWeightCache(init, H, w["gate"], w["up"], w["down"], has_gate), w))
        del t
    return st.SparseMLPStack(layers), oracles


# name, L, H, I, r, dtype, B, act, gate, active fraction, (rho_lo, rho_hi), steps, expected churn band, shared
# `shared` = 0: the rows of a step are independent and `frac` is the fraction of the UNION that is active;
# `shared` > 0: every row has `frac` of its own scores active and the rows share that part of their variance, so
# that the per-row masks overlap (0.6 for the batched bf16 configuration); the cache sees their union.
CASES = [
    ("llama1b_fp32_b1", 1, 2048, 8192, 64, "float32", 1, "silu", True, 0.30, (0.97, 0.97), 32, (0.05, 0.25), 0.0),
    ("llama3b_fp16_b1", 2, 3072, 8192, 128, "float16", 1, "silu", True, 0.35, (0.95, 0.995), 64, (0.03, 0.17), 0.0),
    ("llama3b_bf16_b16_union", 1, 3072, 8192, 128, "bfloat16", 16, "silu", True, 0.30, (0.9, 0.9), 8, (0.0, 0.2), 0.72),
    ("mistral7b_bf16_b2", 2, 4096, 14336, 256, "bfloat16", 2, "silu", True, 0.25, (0.98, 0.98), 16, (0.05, 0.2), 0.0),
    ("relullama7b_gated_fp16_b1", 2, 4096, 11008, 440, "float16", 1, "relu", True, 0.10, (0.95, 0.95), 16,
     (0.1, 0.35), 0.0),
    ("relullama7b_ungated_fp16_b1", 2, 4096, 11008, 440, "float16", 1, "relu", False, 0.10, (0.95, 0.95), 16,
     (0.1, 0.35), 0.0),
]


def _step_inputs(rng, state, rh, shared):
    """Predictor inputs [L,B,H] of the next step: AR(1) in time; with `shared` the rows of a step share that
    fraction of their variance."""
    common, own = state
    L, B, H = own.shape
    own = rh * own + np.sqrt(1.0 - rh * rh) * rng.standard_normal((L, B, H))
    if shared > 0.0:
        common = rh * common + np.sqrt(1.0 - rh * rh) * rng.standard_normal((L, 1, H))
        xp = np.sqrt(shared) * common + np.sqrt(1.0 - shared) * own
    else:
        xp = own
    return (common, own), xp.astype(np.float32)


@pytest.mark.parametrize("name,L,H,I,r,dtype,B,act,has_gate,frac,rho,steps,churn_band,shared", CASES,
                         ids=[c[0] for c in CASES])
def test_full_shape_decode_sequence(name, L, H, I, r, dtype, B, act, has_gate, frac, rho, steps, churn_band, shared):
    stack, oracles = _build(dtype, L, H, I, r, has_gate, act, seed=31)
    tdt = getattr(torch, dtype)
    rng = np.random.default_rng(7)
    stack.prepare(B)                 # fused update + decode kernel, the stack's own scratch
    stack.use_trace_masks = False    # the predictor's masks drive the caches
    assert stack.fused
    state = (rng.standard_normal((L, 1, H)), rng.standard_normal((L, B, H)))
    churns, overlaps, surplus_add, surplus_rem = [], [], 0, 0
    prev = [np.ones(I, bool) for _ in range(L)]
    for t in range(steps):
        rh = rng.uniform(*rho) if rho[1] > rho[0] else rho[0]
        state, xp = _step_inputs(rng, state, rh, shared)
        xph = round_to(xp, dtype)
        x = round_to(rng.standard_normal((B, H)).astype(np.float32), dtype)
        # thresholds: the step's target fraction (wobbling by a few percent of the set), placed in a score gap
        want_masks = []
        xo = x
        for l, (oc, w) in enumerate(oracles):
            s = oracle.predictor_scores(xph[l], w["A"], w["Bm"])
            f = frac * (1.0 + rng.uniform(-0.03, 0.03))
            thr = _threshold_in_gap(s, f, per_row=shared > 0.0)
            stack.layers[l].thr = thr
            m = oracle.mask_threshold(s, thr, True)
            if shared > 0.0:   # overlap of consecutive rows' own masks
                rows = s >= thr
                overlaps.append(float((rows[:-1] & rows[1:]).sum() / max(1, rows[:-1].sum())))
            want_masks.append(m)
            if t > 0:
                na, nr = int((m & ~prev[l]).sum()), int((prev[l] & ~m).sum())
                churns.append(max(na, nr) / max(1, int(prev[l].sum())))
                surplus_add += na > nr
                surplus_rem += nr > na
            prev[l] = m
            oc.update_active_weights(m)
            y, _ = oracle.mlp_forward(xo, oc.get_concat_weight(), oc.get_active_down_weight(), act, has_gate)
            xo = round_to(y, dtype)
        got = stack.step_staged(torch.from_numpy(x).to(DEV, tdt), torch.from_numpy(xph).to(DEV, tdt), None,
                                replay=False).clone()
        for l, (oc, _) in enumerate(oracles):
            assert np.array_equal(stack.layers[l].mask.cpu().numpy(), want_masks[l]), (name, t, l, "mask")
            stack.layers[l].cache._dirty = True
            assert stack.layers[l].cache.get_active_indices().cpu().tolist() == oc.get_active_indices().tolist(), \
                (name, t, l, "index order")
        assert_close(got.float().cpu().numpy(), xo, dtype, f"{name} step {t}")
    mean_churn = float(np.mean(churns))
    assert churn_band[0] <= mean_churn <= churn_band[1], f"mean churn {mean_churn:.3f} outside {churn_band}"
    assert surplus_add > 0 and surplus_rem > 0, "the sequence must exercise appends and surplus removals"
    if shared > 0.0:
        assert 0.5 <= float(np.mean(overlaps)) <= 0.7, f"mean overlap of the rows' masks {np.mean(overlaps):.3f}"
