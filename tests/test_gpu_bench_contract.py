"""bench.py prints one JSON line with the fields its callers rely on (short runs in a child process)."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                       timeout=280, cwd=ROOT)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1, p.stdout[-2000:]
    return json.loads(lines[0])


def test_decode_line():
    # (more profile steps than the run has: the per-kernel pass must clamp itself to the trace, not wrap around it)
    d = _run("--layers", "2", "--steps", "6", "--warmup", "2", "--profile-steps", "32", "--cpu-layers", "1",
             "--cpu-steps", "4")
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 6 and d["warmup"] == 2 and d["vs_baseline"] is None
    assert d["unit"] == "tok/s" and d["value"] > 0 and d["higher_is_better"] is True
    assert d["config"]["workload"] == "llama3b_stack_fp16" and d["dtype"] == "f16"
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["unit"] == "GB/s"
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3 and 0 < r["frac"] < 1
    pp = d["profile_pass"]
    assert pp["steps"] == 7 and pp["trace_steps"] == [1, 7], pp
    # every update of the pass has the configured churn: no launch moves many times the usual number of rows
    ku = d["kernels_us"]["cache_update_decode"]
    assert ku["launches"] == 2 * 7 and ku["p90_us"] < 1.5 * ku["median_us"], ku
    assert "other_workloads" not in d      # only the default workload, depth and batch carry them
    c = d["cpu_baseline"]
    assert c["value"] > 0 and c["cores"] >= 1 and c["kind"] in ("reference", "port") and c["sample"]


def test_prefill_line():
    d = _run("--workload", "llama3b_stack_bf16_overlap06", "--prefill", "128", "--layers", "1", "--steps", "3",
             "--warmup", "1", "--profile-steps", "4")
    r = d["roofline"]
    assert d["dtype"] == "bf16" and r["bound"] == "mfma" and r["unit"] == "TFLOP/s" and r["peak"] == 2500.0
    assert 0 < r["frac"] < 1 and d["value"] > 0 and d["config"]["rows"] == 128


def test_default_line_carries_the_other_workloads():
    """The line a bare `bench.py --steps K --warmup W` prints: the other workloads, a wobbling count and predictor-driven
    masks ride along as short passes, and the measured traffic belongs to the sources in the tree."""
    d = _run("--steps", "6", "--warmup", "2", "--no-cpu-baseline")
    ow = d["other_workloads"]
    for key in ("llama1b_layer_fp32_b1", "llama3b_stack_fp16_b4", "llama3b_stack_fp16_b16", "mistral7b_stack_bf16_b1",
                "mistral7b_stack_bf16_b8", "relullama7b_stack_fp16_b1", "relullama7b_ungated_fp16_b1",
                "llama3b_stack_fp16_b1_count_wobble_0.03", "llama3b_stack_fp16_b1_mask_source_predictor"):
        assert ow[key]["tok_s"] > 0 and 0 < ow[key]["frac"] < 1, key
    assert d["config"]["mask_source"] == "trace" and d["config"]["count_wobble"] == 0.0
    assert d["roofline"]["traffic"] is not None, d["roofline"]["traffic_source"]
    assert 0.9 < d["roofline"]["traffic"] / d["roofline"]["bytes_per_launch"] < 1.3
    assert d["prefill_512"]["roofline"]["bound"] == "mfma"
