"""bench.py prints one JSON line with the fields its readers rely on (a short run on the GPU)."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args):
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    return json.loads(lines[0])


def test_bench_line_has_the_contract_fields():
    d = run_bench("--steps", "5", "--warmup", "1", "--extras")
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 1 and d["vs_baseline"] is None
    assert d["config"]["workload"].startswith("C3") and "model" not in d["config"]
    rf = d["roofline"]
    assert rf["bound"] == "hbm" and rf["unit"] == "GB/s" and rf["peak"] == 8000.0
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-9 and 0.3 < rf["frac"] < 1.0
    assert rf["kernel"] == "decode_attention_quad_kernel"
    assert abs(d["value"] - d["config"]["algorithmic_bytes"] / (d["ms_per_step"] * 1e-3) / 1e9) < 1e-6 * d["value"]
    cb = d["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] >= 1 and cb["value"] > 0 and cb["unit"] == "GB/s" and cb["sample"]
    assert set(d["extras"]) >= {"rope_us", "append_us", "rope_append_fused_us", "kv_cache_reorder_us"}


def test_bench_custom_shape():
    d = run_bench("--custom", "hq=8,hkv=2,d=64,batch=8,kvmin=200,kvmax=400", "--steps", "3", "--warmup", "1", "--no-cpu-baseline")
    assert d["config"]["workload"].startswith("custom(") and d["roofline"]["traffic"] is None and d["value"] > 0


def test_bench_short_chunks():
    d = run_bench("--chunks", "hq=8,hkv=2,d=128,seqs=8,qmin=2,qmax=4,prior=700", "--steps", "3")
    assert d["config"]["columns_per_kv_head"] == 16 and d["workspace_bytes"] > 0
    assert d["tile_kernel_us"] > 0 and d["decode_kernel_path_us"] > 0 and d["max_abs_difference_between_the_two"] < 0.05
