#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ from the reference's own C++ operator.

The reference (NimbleEdge/sparse_transformers) ships no tests or known-answer vectors, so these are
produced by compiling its sources (sparse_transformers/csrc/sparse_mlp_op.cpp + weight_cache.h) with
`make -C oracle ref` and driving the resulting TorchScript class / operator on small seeded inputs:

  cache_traces.json   mask sequences and the ordered active list after every update
                      (weight_cache.h:229-359), incl. no-op updates, the all-false error and what the
                      cache does afterwards, gated and ungated
  mlp_forward.json    tiny fp32 inputs and outputs of torch.ops.sparse_mlp.forward
                      (sparse_mlp_op.cpp:79-192, the ReLU operator), gated and ungated
  approx_topk.json    fp32 score rows and the thresholds torch.ops.sparse_mlp.approx_topk_threshold
                      returns for them (approx_topk.h:10-88), incl. feature sizes that are not
                      multiples of the sketch width, repeated values and -inf scores
  approx_topk_f64.json the same operator on float64 scores (it dispatches on the scores' type), incl. values that
                      agree in the upper half of their bits

Run from the repository root in a container that has /root/reference:  python tests/golden/make_golden.py
"""
import base64
import json
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def weights(I, H):
    """Deterministic, exactly representable weights: row i of every matrix is recognisable."""
    gate = (np.arange(I * H, dtype=np.float32).reshape(I, H) + 0.25)
    up = -(np.arange(I * H, dtype=np.float32).reshape(I, H) + 0.5)
    down = (np.arange(H * I, dtype=np.float32).reshape(H, I) * 2.0 + 1.0)
    return gate, up, down


def bits(m):
    return "".join("1" if b else "0" for b in m)


def make_trace(WC, seed, I, H, steps, has_gate, p_flip, force_events):
    rng = np.random.default_rng(seed)
    gate, up, down = weights(I, H)
    init = rng.random(I) < 0.8
    init[0] = True
    rc = WC(torch.from_numpy(init), H, torch.from_numpy(gate) if has_gate else None, torch.from_numpy(up),
            torch.from_numpy(down), has_gate)
    def order():
        cw = rc.get_concat_weight().numpy()
        n = cw.shape[0] // (2 if has_gate else 1)
        # up rows are -(i*H + h + 0.5): recover the index of every active row from its first element
        first = cw[-n:, 0]
        return [int(round((-v - 0.5) / H)) for v in first]
    rec = {"I": I, "H": H, "has_gate": has_gate, "seed": seed, "init_mask": bits(init), "init_order": order(),
           "steps": []}
    m = init.copy()
    for t in range(steps):
        ev = force_events.get(t)
        if ev == "same":
            m = m.copy()
        elif ev == "empty":
            m = np.zeros(I, dtype=bool)
        elif ev == "full":
            m = np.ones(I, dtype=bool)
        elif ev == "shrink":
            m = m & (rng.random(I) < 0.4)
            if not m.any():
                m[3 % I] = True
        else:
            m = m ^ (rng.random(I) < rng.choice(p_flip))
            if not m.any():
                m[rng.integers(I)] = True
        err = None
        try:
            rc.update_active_weights(torch.from_numpy(m))
        except RuntimeError as e:
            err = "No active weights" if "No active weights" in str(e) else str(e)
        step = {"mask": bits(m), "error": err}
        if err is None:
            step["order"] = order()
        rec["steps"].append(step)
    return rec


def main():
    oracle.build(with_ref=True)
    ref = oracle.load_reference()
    if ref is None:
        raise SystemExit("reference operator not built (is /root/reference present?)")
    WC, fwd = ref
    traces = [
        make_trace(WC, 11, 16, 4, 60, True, [0.05, 0.2, 0.5], {7: "same", 20: "shrink", 30: "full"}),
        make_trace(WC, 12, 37, 4, 120, True, [0.03, 0.1, 0.3], {5: "same", 40: "shrink", 41: "same", 90: "full"}),
        make_trace(WC, 13, 64, 8, 200, False, [0.02, 0.1, 0.4], {10: "shrink", 100: "full", 101: "shrink"}),
        # the all-false error and the (odd but real) behaviour of the cache after it
        make_trace(WC, 14, 24, 4, 40, True, [0.1, 0.3], {6: "empty", 7: "empty", 15: "empty", 16: "full"}),
        make_trace(WC, 15, 64, 4, 300, True, [0.01, 0.02, 0.6], {}),
    ]
    with open(os.path.join(HERE, "cache_traces.json"), "w") as f:
        json.dump({"source": "reference WeightCache compiled from sparse_transformers/csrc", "traces": traces}, f,
                  separators=(",", ":"))

    cases = []
    g = torch.Generator().manual_seed(5)
    for (B, H, n, has_gate, shape3d) in [(1, 8, 5, True, False), (3, 16, 7, True, True), (2, 8, 6, False, False),
                                         (4, 12, 1, True, False)]:
        cw = torch.randn((2 if has_gate else 1) * n, H, generator=g)
        dn = torch.randn(n, H, generator=g)
        x = torch.randn(B, 1, H, generator=g) if shape3d else torch.randn(B, H, generator=g)
        db, cb = torch.zeros(1, H), torch.zeros(1, 2)
        out = fwd(x, cw, dn.t(), db, cb, "silu", has_gate)  # the activation string is ignored by the operator
        assert out.data_ptr() == db.data_ptr()
        cases.append({"B": B, "H": H, "n": n, "has_gate": has_gate, "x_shape": list(x.shape),
                      "x": x.flatten().tolist(), "concat": cw.flatten().tolist(), "down_rows": dn.flatten().tolist(),
                      "out": out.flatten().tolist(), "combined": cb.flatten().tolist(),
                      "combined_shape": list(cb.shape)})
    with open(os.path.join(HERE, "mlp_forward.json"), "w") as f:
        json.dump({"source": "torch.ops.sparse_mlp.forward compiled from sparse_transformers/csrc (ReLU operator)",
                   "cases": cases}, f, separators=(",", ":"))
    approx = torch.ops.sparse_mlp.approx_topk_threshold
    acases = []
    g = torch.Generator().manual_seed(9)
    for (B, F, k, kind) in [(1, 16, 4, "normal"), (3, 37, 5, "normal"), (2, 64, 64, "normal"), (2, 100, 1, "normal"),
                            (1, 257, 30, "coarse"), (2, 96, 20, "neginf"), (1, 5000, 700, "normal"),
                            (2, 4099, 1025, "coarse")]:
        sc = torch.randn(B, F, generator=g)
        if kind == "coarse":       # many equal values
            sc = (sc * 4).round() / 4
        elif kind == "neginf":     # whole residue classes at -inf: some sketch cells stay empty
            sc[:, ::2] = float("-inf")
            sc[1] = float("-inf")
        thr = approx(sc, k)
        # little-endian float32 bytes, base64 (keeps the fixture small and bit-exact)
        acases.append({"B": B, "F": F, "k": k,
                       "scores_f32_b64": base64.b64encode(sc.numpy().astype("<f4").tobytes()).decode("ascii"),
                       "threshold_f32_b64": base64.b64encode(thr.numpy().astype("<f4").tobytes()).decode("ascii")})
    with open(os.path.join(HERE, "approx_topk.json"), "w") as f:
        json.dump({"source": "torch.ops.sparse_mlp.approx_topk_threshold compiled from sparse_transformers/csrc",
                   "cases": acases}, f, separators=(",", ":"))
    # the same operator on double scores (it dispatches on the scores' type, approx_topk.h:33)
    dcases = []
    g = torch.Generator().manual_seed(10)
    for (B, F, k, kind) in [(2, 16, 4, "normal"), (3, 37, 5, "normal"), (1, 257, 30, "coarse"), (2, 96, 20, "neginf"),
                            (1, 1500, 200, "close"), (1, 2051, 513, "coarse")]:
        sc = torch.randn(B, F, generator=g, dtype=torch.float64)
        if kind == "coarse":
            sc = (sc * 4).round() / 4
        elif kind == "neginf":
            sc[:, ::2] = float("-inf")
            sc[1] = float("-inf")
        elif kind == "close":      # values that differ only far down the mantissa: equal upper key halves
            sc = 1.0 + sc * 1e-12
        thr = approx(sc, k)
        assert thr.dtype == torch.float64
        dcases.append({"B": B, "F": F, "k": k,
                       "scores_f64_b64": base64.b64encode(sc.numpy().astype("<f8").tobytes()).decode("ascii"),
                       "threshold_f64_b64": base64.b64encode(thr.numpy().astype("<f8").tobytes()).decode("ascii")})
    with open(os.path.join(HERE, "approx_topk_f64.json"), "w") as f:
        json.dump({"source": "torch.ops.sparse_mlp.approx_topk_threshold on float64 scores, compiled from "
                             "sparse_transformers/csrc", "cases": dcases}, f, separators=(",", ":"))
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()
