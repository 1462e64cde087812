#!/usr/bin/env python3
"""Benchmark of the sparse-MLP decode path on one MI355X.

A "step" is one decoded token through the whole stack of the chosen workload: per layer the LoRA
predictor + threshold mask, the differential weight-cache update (driven by a pre-generated mask trace
with the workload's active fraction and per-step churn) and the fused sparse MLP.  All inputs (weights,
predictor inputs, mask trace) are resident in HBM before the timed region starts.

Prints ONE JSON line.  `roofline` is for the dominant kernel (the decode MLP with the cache update fused
into it): algorithmic bytes per launch -- 3*n*H*s of active weights plus 2*3*k*H*s for the k changed rows
of the update -- over its mean duration, measured with HIP events stamped at the kernel's begin and end
in a second pass over the same workload.  `cpu_baseline` times the same path on the host cores on a
bounded sample.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic.md")


def csrc_hash() -> str:
    """sha256 over the HIP sources the library is built from (first 16 hex digits), or "" when they are not there."""
    import glob
    import hashlib
    files = sorted(glob.glob(os.path.join(ROOT, "sparse_transformers_amd", "csrc", "*")))
    if not files:
        return ""
    h = hashlib.sha256()
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def measured_traffic(workload: str, kernel_kind: str, batch: int):
    """HBM bytes per launch of a workload's dominant kernel as rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE counted them,
    from the table rows of profiles/hbm_traffic.md:
        | workload | batch | kernel kind | kernel | csrc hash | fetched bytes | written bytes |
    A row only counts while the sources it was measured on are the ones in this tree (same hash): otherwise the
    figure would silently describe another kernel.  Returns (bytes or None, where the figure comes from / why not)."""
    have = csrc_hash()
    if not os.path.exists(TRAFFIC_TABLE):
        return None, "profiles/hbm_traffic.md not found"
    stale = None
    with open(TRAFFIC_TABLE) as f:
        for line in f:
            cells = [c.strip().strip("`") for c in line.strip().strip("|").split("|")]
            if len(cells) != 7 or cells[0] != workload or cells[2] != kernel_kind:
                continue
            try:
                b, fetched, written = int(cells[1]), int(cells[5].replace(" ", "")), int(cells[6].replace(" ", ""))
            except ValueError:
                continue
            if b != batch:
                continue
            if cells[4] == have and have:
                return fetched + written, f"profiles/hbm_traffic.md ({cells[3]}, csrc {have}): FETCH_SIZE {fetched} + WRITE_SIZE {written}"
            stale = cells[4]
    if stale is not None:
        return None, f"profiles/hbm_traffic.md was measured on csrc {stale}, this tree is {have or 'without sources'}"
    return None, f"no row for {workload} batch {batch} {kernel_kind} in profiles/hbm_traffic.md"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="llama3b_stack_fp16")
    ap.add_argument("--layers", type=int, default=0, help="override the number of layers (debug)")
    ap.add_argument("--batch", type=int, default=0, help="override the decode batch (rows of x)")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--overlap", action="store_true",
                    help="run predictor/cache update on a side stream (measured slower inside a graph; off by default)")
    ap.add_argument("--no-fused", action="store_true",
                    help="cache update and MLP as two kernels per layer instead of the fused update+decode kernel")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-prefill-probe", action="store_true",
                    help="skip the short 512-row MFMA pass whose figures the decode line carries as `prefill_512`")
    ap.add_argument("--cpu-layers", type=int, default=4)
    ap.add_argument("--cpu-steps", type=int, default=300)
    ap.add_argument("--profile-steps", type=int, default=32)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a known-size reference for rocprofv3 --pmc)")
    ap.add_argument("--active-frac", type=float, default=0.0,
                    help="override the active fraction (e.g. the union of several rows' masks)")
    ap.add_argument("--churn", type=float, default=-1.0, help="override the fraction of the active set swapped per step")
    ap.add_argument("--count-wobble", type=float, default=0.0,
                    help="let the active count of every layer-step vary by this fraction around the workload's value "
                         "(as a predictor's threshold would: some updates add more than they remove, others remove "
                         "more); 0 keeps the count fixed, which is what the headline is quoted on")
    ap.add_argument("--mask-source", choices=("trace", "predictor"), default="trace",
                    help="what drives the caches: the pre-generated mask trace with exactly the configured count and churn "
                         "(the predictor's mask is computed and dropped), or the layer's own predictor mask (threshold "
                         "at the workload's active fraction; predictor inputs follow an AR(1) process whose correlation "
                         "gives about the configured churn; count and churn then wobble as they do in a model)")
    ap.add_argument("--prefill", type=int, default=0,
                    help="time the MFMA path instead: this many rows of x per step through the stack's sparse MLPs, "
                         "each cache at the union of the rows' masks (roofline against the dense MFMA peak)")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the short passes over the other workloads / batch sizes and the count-wobble pass that "
                         "the default line carries as `other_workloads` (they only run for the default workload, "
                         "depth and batch)")
    ap.add_argument("--seed", type=int, default=1236)
    return ap.parse_args()


MFMA_PEAK_TFLOPS = 2500.0   # dense fp16 / bf16


def prefill_measure(stack, wl, T, layers, K, W, profile_steps, seed, torch, _lib, syn):
    """`T` rows of x through the sparse MLP of the first `layers` layers of `stack`, each cache at the union of the
    rows' masks (per-row masks of the workload's active fraction that share 60 % of their indices): tok/s, the kernels'
    event times and the gate/up kernel against the dense MFMA peak."""
    import ctypes as C
    dev = torch.device("cuda:0")
    dt = getattr(torch, wl.dtype)
    H, I = wl.hidden, wl.intermediate
    g = torch.Generator(device=dev)
    g.manual_seed(seed + 101)
    sub = stack.layers[:layers]
    ns = []
    for l, layer in enumerate(sub):
        union = syn.overlapping_token_masks(seed + 11 + l, I, T, wl.n_active, 0.6).any(axis=0)
        layer.cache.update_active_weights(torch.from_numpy(union).to(dev))
        ns.append(int(union.sum()))
    x0 = torch.randn(T, H, generator=g, device=dev, dtype=torch.float32).to(dt)
    bufs = [torch.empty(T, H, device=dev, dtype=dt) for _ in range(2)]
    from sparse_transformers_amd.ops import mlp_workspace_bytes
    ws = torch.empty(mlp_workspace_bytes(T, H, I), dtype=torch.uint8, device=dev)

    def step():
        x = x0
        for l, layer in enumerate(sub):
            x = layer.cache.forward(x, wl.act, out=bufs[l & 1], workspace=ws)
        return x

    # the timed steps replay a HIP graph of the step, like the decode bench (launched one call at a time from
    # Python the GPU waits for the host between the three kernels of a layer)
    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for _ in range(W):
        graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(K):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    ms_per_step = e0.elapsed_time(e1) / K
    L = _lib.lib()
    cap = 8 * layers
    kinds, ms = (C.c_int * cap)(), (C.c_float * cap)()
    per = {}
    for _ in range(max(4, profile_steps // 4)):
        _lib.check(L.st_profile_enable(cap), "st_profile_enable")
        step()
        torch.cuda.synchronize()
        cnt = L.st_profile_collect(kinds, ms, cap)
        for i in range(cnt):
            per.setdefault(_lib.KERNEL_KINDS[kinds[i]], []).append(ms[i] * 1e3)
    L.st_profile_disable()
    kern = {k: {"launches": len(v), "mean_us": round(float(np.mean(v)), 3), "median_us": round(float(np.median(v)), 3)}
            for k, v in per.items()}
    n_mean = float(np.mean(ns))
    c = 3 if wl.has_gate else 2
    flops_layer = 2.0 * c * T * n_mean * H
    gu_flops = 2.0 * (c - 1) * T * n_mean * H
    gu_us = kern["mlp_prefill_gateup"]["mean_us"]
    achieved = gu_flops / (gu_us * 1e-6) / 1e12
    return {"ms_per_step": ms_per_step, "kernels_us": kern, "n_mean": n_mean, "flops_layer": flops_layer,
            "gu_flops": gu_flops, "gu_us": gu_us, "achieved_tflops": achieved, "layers": layers,
            "stack_tflops": layers * flops_layer / (ms_per_step * 1e-3) / 1e12}


def prefill_gateup_name(rows: int, n_active: float, cus: int = 256) -> str:
    """Which form of the gate/up kernel the library takes for this shape (mlp_prefill.hip: the wide form once 128-row
    tiles of 64 + 64 weight rows outnumber the CUs)."""
    tiles = ((int(n_active) + 127) // 128 * 2) * ((rows + 127) // 128)
    return "prefill_gateup_wide_kernel" if rows > 128 and tiles > cus else "prefill_gateup_kernel"


def prefill_bench(args, wl, torch, st, _lib, syn):
    """One step = `--prefill` rows of x through the sparse MLP of every layer (see prefill_measure)."""
    if wl.dtype == "float32":
        print("bench.py: --prefill needs an fp16 / bf16 workload (the MFMA kernels)", file=sys.stderr)
        sys.exit(2)
    T, H, I = args.prefill, wl.hidden, wl.intermediate
    layers = args.layers or min(wl.layers, 8)
    K, W = args.steps, args.warmup
    stack, _ = build_stack(wl, layers, 1, args.seed, torch, st)
    m = prefill_measure(stack, wl, T, layers, K, W, args.profile_steps, args.seed, torch, _lib, syn)
    out = {
        "metric": "sparse_mlp_prefill_tokens_per_s", "value": round(T / (m["ms_per_step"] * 1e-3), 1), "unit": "tok/s",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(m["ms_per_step"], 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": {"float16": "f16", "bfloat16": "bf16"}[wl.dtype],
        "data": "synthetic (seeded weights, inputs and per-row masks; caches at the union of the rows' masks)",
        "config": {"workload": wl.name + "_prefill", "layers": layers, "hidden": H, "intermediate": I, "rows": T,
                   "active_rows_mean": m["n_mean"], "act": wl.act, "has_gate": wl.has_gate},
        "roofline": {"bound": "mfma", "achieved": round(m["achieved_tflops"], 1), "peak": MFMA_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(m["achieved_tflops"] / MFMA_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": prefill_gateup_name(T, m["n_mean"]), "flops_per_launch": m["gu_flops"], "mean_us": m["gu_us"]},
        "stack_tflops": round(m["stack_tflops"], 1),
        "kernels_us": m["kernels_us"],
    }
    print(json.dumps(out))


def build_stack(wl, layers, batch, seed, torch, st):
    """Random-init weights of the workload's shape on the GPU, caches, predictors, thresholds."""
    dev = torch.device("cuda:0")
    dt = getattr(torch, wl.dtype)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)

    def nrm(*shape):
        return (torch.randn(*shape, generator=g, device=dev, dtype=torch.float32) * 0.02).to(dt)

    H, I, r = wl.hidden, wl.intermediate, wl.rank
    init_mask = torch.ones(I, dtype=torch.bool, device=dev)
    stack_layers = []
    for _ in range(layers):
        gate = nrm(I, H) if wl.has_gate else None
        up, down = nrm(I, H), nrm(H, I)
        A, Bm = nrm(r, H), nrm(I, r)
        cache = st.WeightCache(init_mask, H, gate, up, down, wl.has_gate)
        del gate, up, down
        pred = st.FastLoRAProjection(A, Bm)
        # threshold: the (1 - active_frac) quantile of this layer's scores on a probe input
        probe = torch.randn(1, H, generator=g, device=dev, dtype=torch.float32).to(dt)
        s = pred(probe).float().flatten()
        thr = float(torch.quantile(s, 1.0 - wl.active_frac))
        stack_layers.append(st.SparseDecodeLayer(pred, cache, wl.act, thr, True))
    return st.SparseMLPStack(stack_layers), g


def cpu_baseline(wl, stack, trace, x_in, x_pred, layers, steps, torch):
    """The same path on the host, on the GPU run's own inputs: the first `layers` layers' weights are read back from
    the GPU caches and predictors, the masks are the first steps of the GPU run's trace and x / the predictor inputs
    are the ones the GPU steps saw.  Cache = the reference's own C++ WeightCache (compiled into oracle/_ref) when it
    loads, else the C oracle; predictor and MLP as the torch-CPU calls of src/modeling_skip.py (fp32, as the
    reference cache is fp32 only).  Returns tok/s scaled to the full stack depth."""
    import oracle

    ref = oracle.load_reference()
    kind = "reference" if ref else "port"
    H = wl.hidden
    steps = min(steps, trace.shape[0] - 1)
    tr = trace[:steps + 1, :layers].cpu().numpy()
    xs = x_in[:steps + 1].float().cpu()
    xps = x_pred[:steps + 1, :layers].float().cpu()
    act = {"silu": torch.nn.functional.silu, "relu": torch.relu}[wl.act]
    built = []
    for l in range(layers):
        c, p = stack.layers[l].cache, stack.layers[l].predictor
        up, down = c.up_pool.float().cpu(), c.downT_pool.float().cpu().t().contiguous()
        gate = c.gate_pool.float().cpu() if wl.has_gate else None
        A, Bm = p.down_weight.float().cpu(), p.up_weight.float().cpu()
        if ref:
            cache = ref[0](torch.from_numpy(tr[0, l]), H, gate, up, down, wl.has_gate)
        else:
            cache = oracle.OracleWeightCache(tr[0, l], H, gate.numpy() if wl.has_gate else None, up.numpy(), down.numpy(),
                                             wl.has_gate)
        built.append((cache, A, Bm))
    times = []
    for t in range(1, steps + 1):
        x = xs[t]
        t0 = time.perf_counter()
        for l, (cache, A, Bm) in enumerate(built):
            scores = (xps[t, l] @ A.t()) @ Bm.t()
            _ = (scores >= 0).any(dim=0)                    # predictor + naive mask + union
            m = tr[t, l]
            if ref:
                cache.update_active_weights(torch.from_numpy(m))
                cw, dw = cache.get_concat_weight(), cache.get_active_down_weight()
            else:
                cache.update_active_weights(m)
                cw, dw = torch.from_numpy(cache.get_concat_weight()), torch.from_numpy(cache.get_active_down_weight())
            if wl.has_gate:
                gt, u = x.matmul(cw.t()).chunk(2, dim=-1)
                x = (act(gt) * u).matmul(dw.t())
            else:
                x = act(x.matmul(cw.t())).matmul(dw.t())
        times.append(time.perf_counter() - t0)
    per_layer_step = float(np.median(times[min(4, len(times) - 1):])) / layers
    tok_s = xs.shape[1] / (per_layer_step * wl.layers)
    return {
        "value": round(tok_s, 3), "unit": "tok/s", "cores": int(torch.get_num_threads()), "kind": kind,
        "sample": f"the first {layers} of {wl.layers} layers x the first {steps} steps of the GPU run's own weights, "
                  f"mask trace and inputs, fp32, median per-layer time scaled to {wl.layers} layers; cache update = "
                  + ("reference WeightCache compiled from its own sources" if ref else "C restatement")
                  + ", predictor/MLP = torch CPU matmul path",
        "ms_per_layer_step": round(per_layer_step * 1e3, 3),
    }


def ar1_inputs(torch, g, T, layers, B, H, churn_lo, churn_hi, dt, dev):
    """Predictor inputs [T, layers, B, H]: every (layer, row) follows x[t] = rho x[t-1] + sqrt(1 - rho^2) eps with
    N(0,1) marginals; rho is drawn per step so that a threshold mask changes by about churn_lo .. churn_hi of its
    set per step (measured for Gaussian scores at 35 % active: churn = 0.61 sqrt(1 - rho))."""
    x = torch.randn(layers, B, H, generator=g, device=dev, dtype=torch.float32)
    out = torch.empty(T, layers, B, H, device=dev, dtype=dt)
    out[0] = x.to(dt)
    for t in range(1, T):
        c = churn_lo if churn_hi <= churn_lo else float(torch.empty(1).uniform_(churn_lo, churn_hi, generator=None))
        rho = max(0.0, 1.0 - (c / 0.61) ** 2)
        x = rho * x + (1.0 - rho * rho) ** 0.5 * torch.randn(layers, B, H, generator=g, device=dev, dtype=torch.float32)
        out[t] = x.to(dt)
    return out


def decode_measure(args, wl, torch, st, _lib, syn, layers, B, K, W, P, count_wobble=0.0, wall=True,
                   mask_source="trace"):
    """One decode workload: W warm-up + K timed steps (one token through `layers` layers each, replayed from a HIP
    graph), then an eager pass over P of the same steps with per-kernel events.  Returns the result dict and what the
    CPU baseline needs (stack, trace, x_in, x_pred)."""
    dev = torch.device("cuda:0")
    dt = getattr(torch, wl.dtype)
    esz = 4 if wl.dtype == "float32" else 2
    H, I, n = wl.hidden, wl.intermediate, wl.n_active
    # the per-kernel pass walks the trace backwards from the last timed step and must stay inside it
    P = max(1, min(P, W + K - 1))

    stack, g = build_stack(wl, layers, B, args.seed, torch, st)
    T = W + K + 1
    trace = torch.from_numpy(syn.mask_trace(args.seed + 7, layers, I, n, T, wl.churn_lo, wl.churn_hi,
                                             count_wobble)).to(dev)
    # predictor inputs per layer and step, MLP input of the first layer per step
    from_predictor = mask_source == "predictor"
    if from_predictor:
        torch.manual_seed(args.seed + 3)
        x_pred = ar1_inputs(torch, g, T, layers, B, H, wl.churn_lo, wl.churn_hi, dt, dev)
    else:
        x_pred = torch.randn(T, layers, B, H, generator=g, device=dev, dtype=torch.float32).to(dt)
    x_in = torch.randn(T, B, H, generator=g, device=dev, dtype=torch.float32).to(dt)

    # bring every cache to the first mask of the trace (the big one-off shrink from all-ones)
    for l, layer in enumerate(stack.layers):
        layer.cache.update_active_weights(trace[0, l])
        assert layer.cache.get_num_active() == n

    use_graph = not args.no_graph
    stack.prepare(B, overlap=args.overlap, fused=not args.no_fused)
    if from_predictor:
        # the layers' own masks drive the caches; the first one brings each cache from the trace's first mask to
        # the predictor's (a larger change than the steps that follow: inside the warm-up)
        stack.use_trace_masks = False
        trace_arg = None
    if use_graph:
        stack.step_staged(x_in[0], x_pred[0], None if from_predictor else trace[0])     # first launches outside capture
        torch.cuda.synchronize()
        stack.capture()

    def masks_of(t):
        return None if from_predictor else trace[t]

    def run(t):
        stack.step_staged(x_in[t], x_pred[t], masks_of(t), replay=use_graph)

    for t in range(1, W + 1):
        run(t)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t_host0 = time.perf_counter()
    e0.record()
    for t in range(W + 1, W + K + 1):
        run(t)
    e1.record()
    torch.cuda.synchronize()
    host_s = time.perf_counter() - t_host0
    ms_per_step = e0.elapsed_time(e1) / K
    tok_s = B * 1000.0 / ms_per_step

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)          # 268435456 bytes read + as many written by one copy kernel
        torch.cuda.synchronize()
        del src, dst

    # ---- second pass over the same masks (backwards, so every transition has the same churn) with
    # ---- per-kernel HIP events recorded on the launch stream by the library.  With a graph the events
    L = _lib.lib()
    per_step = layers * 8
    kinds_all, ms_all = [], []
    kinds = (C.c_int * per_step)()
    ms = (C.c_float * per_step)()

    def collect():
        cnt = L.st_profile_collect(kinds, ms, per_step)
        if cnt < 0:
            _lib.check(cnt, "st_profile_collect")
        kinds_all.append(np.frombuffer(kinds, dtype=np.int32)[:cnt].copy())
        ms_all.append(np.frombuffer(ms, dtype=np.float32)[:cnt].copy())

    # (Events recorded inside a captured graph cannot be read back with hipEventElapsedTime on this ROCm, so
    # this pass launches eagerly.  The library launches with hipExtLaunchKernelGGL, whose start / stop events are
    # stamped at the kernel's own begin and end, so these are execution times, as rocprofv3 reports them.)
    def summarise():
        kinds_np, ms_np = np.concatenate(kinds_all), np.concatenate(ms_all)
        out = {}
        for k, name in enumerate(_lib.KERNEL_KINDS):
            sel = ms_np[kinds_np == k]
            if sel.size:
                out[name] = {"launches": int(sel.size), "mean_us": round(float(sel.mean()) * 1e3, 3),
                             "median_us": round(float(np.median(sel)) * 1e3, 3),
                             "p10_us": round(float(np.percentile(sel, 10)) * 1e3, 3),
                             "p90_us": round(float(np.percentile(sel, 90)) * 1e3, 3)}
        kinds_all.clear()
        ms_all.clear()
        return out

    # Launched one call at a time from Python, the GPU would wait for the host between the kernels of a step, which
    # is not how they run in the timed region (a graph keeps them back to back).  So every step of this pass is
    # enqueued behind a short spin kernel that holds the stream for as long as the host needs to enqueue the step:
    # the step's kernels then find each other in the queue, as in the replayed graph.
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    spin = getattr(torch.cuda, "_sleep", None) or (lambda cycles: None)   # (without it the pass runs as the host feeds it)
    ev0.record(); spin(1_000_000); ev1.record()
    torch.cuda.synchronize()
    cycles_per_ms = 1e6 / max(ev0.elapsed_time(ev1), 1e-3)
    h0 = time.perf_counter()
    stack.step_staged(x_in[W + K - 1], x_pred[W + K - 1], masks_of(W + K - 1), replay=False)   # (the masks the caches hold)
    host_ms = (time.perf_counter() - h0) * 1e3
    torch.cuda.synchronize()
    hold_cycles = int(min(3.0 * host_ms + 0.5, 20.0) * cycles_per_ms)

    t_lo = W + K - 1 - P
    seen_changed, seen_active = [], []
    for t in range(W + K - 1, t_lo, -1):
        _lib.check(L.st_profile_enable(per_step), "st_profile_enable")
        spin(hold_cycles)
        stack.step_staged(x_in[t], x_pred[t], masks_of(t), replay=False)
        torch.cuda.synchronize()
        collect()
        if from_predictor:      # what the updates of this step really did (read back from the caches' state words)
            for layer in stack.layers:
                layer.cache._dirty = True
                stt = layer.cache.sync_state()
                seen_changed.append(stt["n_changed"])
                seen_active.append(stt["n_active"])
    per_kernel = summarise()
    # the cache update on its own (it has no kernel of its own in the fused path): a few more steps, forwards again
    unfused = None
    if stack.fused:
        stack.fused = False
        for t in range(t_lo + 2, min(t_lo + 2 + max(4, P // 4), W + K)):
            _lib.check(L.st_profile_enable(per_step), "st_profile_enable")
            spin(hold_cycles)
            stack.step_staged(x_in[t], x_pred[t], masks_of(t), replay=False)
            torch.cuda.synchronize()
            collect()
        unfused = summarise()
        stack.fused = True
    L.st_profile_disable()

    # ---- wall time of the two halves of a layer's chain, each replayed from a graph of its own (a kernel's
    # ---- begin/end events cannot show what it costs inside the chain: an empty kernel already reads 4 us
    # ---- between its two events, while a dependent empty kernel adds only 1.6 us to a replayed chain)
    wall_parts = None
    if wall and use_graph and not args.overlap and not from_predictor:
        def part_predictor():
            for l, layer in enumerate(stack.layers):
                layer.predict_mask(stack.xp_stage[l], stack._t_ws)

        def part_update_mlp():
            x = stack.x_stage
            for l, layer in enumerate(stack.layers):
                out = stack._pingpong[l & 1]
                if stack.fused:
                    layer.cache.update_and_forward(stack.mask_stage[l], x, layer.act, out=out, workspace=stack._mlp_ws)
                else:
                    layer.cache.update_active_weights_async(stack.mask_stage[l])
                    layer.cache.forward(x, layer.act, out=out, workspace=stack._mlp_ws)
                x = out

        wall_parts = {}
        t_cur = min(t_lo + 2 + max(4, P // 4), W + K) - 1 if unfused is not None else t_lo + 1
        steps_w = max(4, min(32, K // 2))
        for name, fn in (("predictor", part_predictor), ("update_mlp", part_update_mlp)):
            # walk the trace one step at a time (up, then down again) so every update has the configured churn
            seq = list(range(t_cur + 1, min(t_cur + 1 + steps_w + 2, T)))
            if len(seq) < steps_w + 2:
                seq = list(range(t_cur - 1, t_cur - 3 - steps_w, -1))
            stack.x_stage.copy_(x_in[seq[0]]); stack.xp_stage.copy_(x_pred[seq[0]]); stack.mask_stage.copy_(trace[seq[0]])
            fn()
            torch.cuda.synchronize()
            gpart = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gpart):
                fn()
            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            for i, t in enumerate(seq[1:]):
                if i == 1:
                    ev0.record()
                stack.x_stage.copy_(x_in[t]); stack.xp_stage.copy_(x_pred[t]); stack.mask_stage.copy_(trace[t])
                gpart.replay()
            ev1.record()
            torch.cuda.synchronize()
            wall_parts[name] = round(ev0.elapsed_time(ev1) * 1e3 / (len(seq) - 2) / layers, 2)
            t_cur = seq[-1]
            for layer in stack.layers:
                layer.cache._dirty = True
        wall_parts["whole_layer"] = round(ms_per_step * 1e3 / layers, 2)
    mats = 3 if wl.has_gate else 2
    alg_bytes = mats * n * H * esz                      # active-weight bytes one launch streams
    dom = "cache_update_decode" if "cache_update_decode" in per_kernel else \
          ("mlp_decode" if "mlp_decode" in per_kernel else "mlp_batch_gateup")
    mlp_us = per_kernel[dom]["mean_us"]
    if dom == "mlp_batch_gateup":                        # the batch path streams the weights in two kernels
        mlp_us += per_kernel["mlp_batch_down"]["mean_us"]
    # changed rows per update over the timed steps (the trace swaps as many rows in as out)
    k_changed = float((trace[W + 1:W + K + 1] & ~trace[W:W + K]).sum(dim=-1).float().mean())
    if from_predictor:
        k_changed = float(np.mean(seen_changed))
        n = int(round(float(np.mean(seen_active))))
        alg_bytes = mats * n * H * esz
    upd_bytes = int(2 * mats * k_changed * H * esz)      # cache update: changed rows read + written
    launch_bytes = alg_bytes + (upd_bytes if dom == "cache_update_decode" else 0)
    achieved = launch_bytes / (mlp_us * 1e-6) / 1e9
    upd_us = (unfused or per_kernel).get("cache_update", {}).get("mean_us")

    traffic, traffic_src = measured_traffic(wl.name, dom, B)
    churn_mean = 0.5 * (wl.churn_lo + wl.churn_hi)
    result = {
        "metric": "sparse-MLP decode tok/s", "value": round(tok_s, 2), "unit": "tok/s",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"float32": "f32", "float16": "f16", "bfloat16": "bf16"}[wl.dtype], "data": "synthetic",
        "config": {"workload": wl.name, "layers": layers, "hidden": H, "intermediate": I, "predictor_rank": wl.rank,
                   "batch": B, "act": wl.act, "has_gate": wl.has_gate, "n_active": n,
                   "churn": [wl.churn_lo, wl.churn_hi], "count_wobble": count_wobble, "mask_source": mask_source,
                   "changed_rows_mean": round(k_changed, 1),
                   "launch": "hip_graph" if use_graph else "eager",
                   "streams": 2 if args.overlap else 1, "update_fused_into_decode": bool(stack.fused),
                   "kernel_timing": "hip events stamped at kernel begin/end (hipExtLaunchKernelGGL), second pass launched call by call, each step queued behind a spin kernel so that its kernels run back to back"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_source": traffic_src,
                     "kernel": {"cache_update_decode": "cache_sparse_decode_kernel", "mlp_decode": "mlp_decode_kernel",
                                "mlp_batch_gateup": "batch_gateup_kernel + batch_down_kernel"}[dom],
                     "bytes_per_launch": launch_bytes, "mean_us": mlp_us,
                     "bytes_mlp": alg_bytes, "bytes_cache_update": upd_bytes if dom == "cache_update_decode" else 0,
                     "frac_mlp_bytes_only": round(alg_bytes / (mlp_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)},
        "cache_update_us_per_layer": upd_us,
        "cache_update_note": ("standalone cache_update_kernel, measured in a short unfused pass; the timed path "
                              "runs it fused into the decode kernel") if unfused else "standalone kernel",
        "stack_hbm_gbps": round(layers * alg_bytes / (ms_per_step * 1e-3) / 1e9, 1),
        "host_wall_ms_per_step": round(host_s * 1e3 / K, 5),
        "wall_us_per_layer": wall_parts,
        "wall_note": "graph replays of the predictor kernels alone, of update + MLP (+ reduce) alone, and of the whole step",
        "kernels_us": per_kernel,
        "kernels_us_unfused": unfused,
        "churn_mean": churn_mean,
        "profile_pass": {"steps": P, "trace_steps": [t_lo + 1, W + K - 1],
                         "note": "eager pass with per-kernel events, backwards over the last steps of the timed range"},
    }
    return result, (stack, trace, x_in, x_pred)


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (every box has one); --gpus {args.gpus} is not supported. "
              "The path would shard along the intermediate dimension, but no multi-GPU code exists.",
              file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    import sparse_transformers_amd as st
    from sparse_transformers_amd import _lib, synthetic as syn

    wl = syn.WORKLOADS[args.workload]
    if args.active_frac > 0.0 or args.churn >= 0.0:
        import dataclasses
        wl = dataclasses.replace(wl, active_frac=args.active_frac if args.active_frac > 0.0 else wl.active_frac,
                                 churn_lo=args.churn if args.churn >= 0.0 else wl.churn_lo,
                                 churn_hi=args.churn if args.churn >= 0.0 else wl.churn_hi)
    if args.prefill > 0:
        prefill_bench(args, wl, torch, st, _lib, syn)
        return
    layers = args.layers or wl.layers
    B = args.batch or wl.batch
    result, (stack, trace, x_in, x_pred) = decode_measure(args, wl, torch, st, _lib, syn, layers, B, args.steps, args.warmup,
                                                          args.profile_steps, args.count_wobble,
                                                          mask_source=args.mask_source)
    if not args.no_prefill_probe and wl.dtype != "float32" and B == 1:
        # the MFMA path in the same line: 512 rows of x through the first layers' sparse MLPs (caches at the union of
        # the rows' masks).  Runs last: it moves those caches away from the decode trace.
        try:
            pl = max(1, min(8, layers))
            m = prefill_measure(stack, wl, 512, pl, 6, 2, 8, args.seed, torch, _lib, syn)
            result["prefill_512"] = {
                "layers": pl, "rows": 512, "active_rows_mean": m["n_mean"], "tok_s": round(512 / (m["ms_per_step"] * 1e-3), 1),
                "us_per_layer": round(m["ms_per_step"] * 1e3 / pl, 2), "stack_tflops": round(m["stack_tflops"], 1),
                "roofline": {"bound": "mfma", "kernel": prefill_gateup_name(512, m["n_mean"]), "achieved": round(m["achieved_tflops"], 1),
                             "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                             "frac": round(m["achieved_tflops"] / MFMA_PEAK_TFLOPS, 4), "mean_us": m["gu_us"]},
                "kernels_us": m["kernels_us"]}
        except Exception as exc:
            result["prefill_512"] = {"error": repr(exc)}
    if not args.no_cpu_baseline:
        try:
            result["cpu_baseline"] = cpu_baseline(wl, stack, trace, x_in, x_pred, max(1, min(args.cpu_layers, layers)),
                                                  args.cpu_steps, torch)
        except Exception as exc:  # the baseline is reported, never required for the GPU numbers
            result["cpu_baseline"] = {"value": None, "unit": "tok/s", "cores": 0, "kind": "port",
                                      "sample": f"failed: {exc!r}"}
    default_run = (args.workload == "llama3b_stack_fp16" and not args.layers and not args.batch and args.churn < 0.0
                   and args.active_frac <= 0.0 and args.count_wobble == 0.0 and not args.no_graph and not args.overlap
                   and not args.no_fused and args.mask_source == "trace")
    if default_run and not args.no_other_workloads:
        del stack, trace, x_in, x_pred
        result["other_workloads"] = other_workloads(args, torch, st, _lib, syn)
    print(json.dumps(result))


# (workload, rows of x): the configurations of the other benchmark shapes, each as a short pass
OTHER_WORKLOADS = [("llama1b_layer_fp32", 1), ("llama3b_stack_fp16", 4), ("llama3b_stack_fp16", 16),
                   ("mistral7b_stack_bf16", 1), ("mistral7b_stack_bf16", 8), ("relullama7b_stack_fp16", 1),
                   ("relullama7b_ungated_fp16", 1)]


def other_workloads(args, torch, st, _lib, syn, steps=12, warmup=4, profile_steps=6):
    """Short passes (no CPU baseline, no prefill probe) over the other workloads and batch sizes, and one over the
    headline workload with the active count wobbling by 3 % per layer-step, as a predictor's threshold makes it."""
    import dataclasses
    import gc

    def brief(r):
        rf = r["roofline"]
        return {"tok_s": r["value"], "ms_per_step": r["ms_per_step"], "layers": r["config"]["layers"],
                "us_per_layer": round(r["ms_per_step"] * 1e3 / r["config"]["layers"], 2), "kernel": rf["kernel"],
                "kernel_mean_us": rf["mean_us"], "frac": rf["frac"], "frac_mlp_bytes_only": rf["frac_mlp_bytes_only"],
                "stack_hbm_gbps": r["stack_hbm_gbps"], "kernels_us": {k: v["median_us"] for k, v in r["kernels_us"].items()}}

    out = {"steps": steps, "warmup": warmup}
    runs = [(name, b, 0.0, "trace") for name, b in OTHER_WORKLOADS] + [("llama3b_stack_fp16", 1, 0.03, "trace"),
                                                                       ("llama3b_stack_fp16", 1, 0.0, "predictor")]
    for name, b, wobble, source in runs:
        wl = syn.WORKLOADS[name]
        layers = wl.layers if wl.layers > 1 else 16     # a single layer's weights would sit in the Infinity Cache
        key = f"{name}_b{b}" if wobble == 0.0 else f"{name}_b{b}_count_wobble_{wobble}"
        if source == "predictor":
            key += "_mask_source_predictor"
        short = wobble == 0.0 and source == "trace"
        try:
            r, keep = decode_measure(args, wl, torch, st, _lib, syn, layers, b, steps if short else 20, warmup,
                                     profile_steps, wobble, wall=False, mask_source=source)
            out[key] = brief(r)
            if source == "predictor":
                out[key]["n_active_mean"] = r["config"]["n_active"]
                out[key]["changed_rows_mean"] = r["config"]["changed_rows_mean"]
            del keep
        except Exception as exc:
            out[key] = {"error": repr(exc)}
        gc.collect()
        torch.cuda.empty_cache()
    return out


if __name__ == "__main__":
    main()
