"""Seeded synthetic workloads for the sparse-MLP decode path.

Everything is drawn with numpy generators on the host, so the same seed gives the same weights, inputs
and mask traces on every machine; tensors are then cast and moved by the caller.  Shapes follow the
Llama / Mistral / ReLU-Llama layer sizes the reference targets (its configs/*.json).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np


@dataclass(frozen=True)
class Workload:
    name: str
    layers: int
    hidden: int
    intermediate: int
    rank: int
    dtype: str            # "float32" | "float16" | "bfloat16"
    act: str
    has_gate: bool
    active_frac: float
    churn_lo: float
    churn_hi: float
    steps: int
    batch: int = 1

    @property
    def n_active(self) -> int:
        return int(self.active_frac * self.intermediate)


WORKLOADS = {
    # one Llama-3.2-1B-shaped layer, fp32, 30 % active, 10 % of the active set swapped per step
    "llama1b_layer_fp32": Workload("llama1b_layer_fp32", 1, 2048, 8192, 64, "float32", "silu", True, 0.30, 0.10, 0.10, 128),
    # Llama-3.2-3B-shaped stack, fp16, 35 % active, 5-15 % churn  (the headline workload)
    "llama3b_stack_fp16": Workload("llama3b_stack_fp16", 28, 3072, 8192, 128, "float16", "silu", True, 0.35, 0.05, 0.15, 512),
    # Llama-3.2-3B-shaped layer in bf16 with per-token masks of 30 % that overlap by 0.6 from one token to the next
    # (40 % of the active set swapped per step), stacked 28 deep so that the weights cannot sit in the Infinity Cache
    "llama3b_stack_bf16_overlap06": Workload("llama3b_stack_bf16_overlap06", 28, 3072, 8192, 128, "bfloat16", "silu", True,
                                             0.30, 0.40, 0.40, 64),
    # Mistral-7B-shaped stack, bf16, 25 % active, 10 % churn
    "mistral7b_stack_bf16": Workload("mistral7b_stack_bf16", 32, 4096, 14336, 256, "bfloat16", "silu", True, 0.25, 0.10, 0.10, 256),
    # ReLU-Llama-7B-shaped stack, fp16, 10 % active, 20 % churn, gated and ungated
    "relullama7b_stack_fp16": Workload("relullama7b_stack_fp16", 32, 4096, 11008, 440, "float16", "relu", True, 0.10, 0.20, 0.20, 256),
    "relullama7b_ungated_fp16": Workload("relullama7b_ungated_fp16", 32, 4096, 11008, 440, "float16", "relu", False, 0.10, 0.20, 0.20, 256),
}


def layer_weights(rng: np.random.Generator, hidden: int, intermediate: int, rank: int, std: float = 0.02,
                  has_gate: bool = True) -> dict:
    """gate/up [I,H], down [H,I], predictor A [r,H] and Bm [I,r], all ~ N(0, std^2), float32."""
    def nrm(*shape):
        return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std))
    w = {"up": nrm(intermediate, hidden), "down": nrm(hidden, intermediate),
         "A": nrm(rank, hidden), "Bm": nrm(intermediate, rank)}
    w["gate"] = nrm(intermediate, hidden) if has_gate else None
    return w


def initial_mask(rng: np.random.Generator, intermediate: int, n_active: int) -> np.ndarray:
    m = np.zeros(intermediate, dtype=bool)
    m[rng.choice(intermediate, size=n_active, replace=False)] = True
    return m


def churn_step(rng: np.random.Generator, mask: np.ndarray, frac: float, target: int = -1) -> np.ndarray:
    """Swap round(frac * n) active indices for as many inactive ones (n stays constant); with `target` >= 0 the
    count moves to `target` as well (more additions than removals, or the other way round)."""
    act = np.flatnonzero(mask)
    ina = np.flatnonzero(~mask)
    c = min(int(round(frac * act.size)), act.size, ina.size)
    delta = 0 if target < 0 else int(target) - act.size
    rem = min(act.size, c + max(0, -delta))
    add = min(ina.size, c + max(0, delta))
    out = mask.copy()
    if rem > 0:
        out[rng.choice(act, size=rem, replace=False)] = False
    if add > 0:
        out[rng.choice(ina, size=add, replace=False)] = True
    return out


def mask_trace(seed: int, layers: int, intermediate: int, n_active: int, steps: int, churn_lo: float,
               churn_hi: float, wobble: float = 0.0) -> np.ndarray:
    """bool [steps, layers, I]: per layer a correlated mask sequence; churn ~ U(lo, hi) per layer-step.  With
    `wobble` > 0 the count of every step is drawn from n_active * (1 + U(-wobble, wobble)) instead of staying at
    n_active, as it does when a predictor's threshold drives the mask: additions outnumber removals in some steps
    and removals outnumber additions in others."""
    rng = np.random.default_rng(seed)
    out = np.empty((steps, layers, intermediate), dtype=bool)
    for l in range(layers):
        m = initial_mask(rng, intermediate, n_active)
        out[0, l] = m
        for t in range(1, steps):
            frac = churn_lo if churn_hi <= churn_lo else rng.uniform(churn_lo, churn_hi)
            target = -1
            if wobble > 0.0:
                target = int(round(n_active * (1.0 + rng.uniform(-wobble, wobble))))
                target = max(1, min(intermediate, target))
            m = churn_step(rng, m, frac, target)
            out[t, l] = m
    return out


def ragged_mask_trace(seed: int, intermediate: int, steps: int, p_flip=(0.02, 0.1, 0.4),
                      keep_nonempty: bool = True) -> np.ndarray:
    """bool [steps, I] with independent flips, so the active count drifts and every phase of the
    update (pairing, append, swap-with-last) is exercised."""
    rng = np.random.default_rng(seed)
    m = rng.random(intermediate) < 0.5
    out = np.empty((steps, intermediate), dtype=bool)
    for t in range(steps):
        m = m ^ (rng.random(intermediate) < rng.choice(p_flip))
        if t % 11 == 5:
            m = m.copy()  # an unchanged mask now and then (no-op update)
        if keep_nonempty and not m.any():
            m[rng.integers(intermediate)] = True
        out[t] = m
    return out


def overlapping_token_masks(seed: int, intermediate: int, tokens: int, n_active: int, overlap: float) -> np.ndarray:
    """bool [tokens, I]: every token has n_active active indices, a shared core of round(overlap*n)
    plus private ones; the cache mask is their union over tokens."""
    rng = np.random.default_rng(seed)
    core_n = int(round(overlap * n_active))
    perm = rng.permutation(intermediate)
    core, rest = perm[:core_n], perm[core_n:]
    out = np.zeros((tokens, intermediate), dtype=bool)
    for t in range(tokens):
        out[t, core] = True
        out[t, rng.choice(rest, size=n_active - core_n, replace=False)] = True
    return out


def threshold_for_fraction(scores: np.ndarray, active_frac: float, guard: float = 0.0,
                           others: Optional[np.ndarray] = None) -> float:
    """A threshold t with about active_frac of scores >= t, placed in the widest nearby gap between
    consecutive sorted scores so that rounding differences between implementations cannot flip a
    mask bit (|score - t| >= guard is asserted when guard > 0)."""
    s = np.sort(np.asarray(scores, dtype=np.float64).ravel())
    k = int(round((1.0 - active_frac) * s.size))
    k = min(max(k, 1), s.size - 1)
    lo, hi = max(1, k - 8), min(s.size - 1, k + 8)
    gaps = s[lo:hi + 1] - s[lo - 1:hi]
    j = int(np.argmax(gaps)) + lo
    thr = 0.5 * (s[j - 1] + s[j])
    if guard > 0:
        allv = s if others is None else np.concatenate([s, np.asarray(others, dtype=np.float64).ravel()])
        assert np.min(np.abs(allv - thr)) >= guard, "no guard band around the threshold"
    return float(thr)
