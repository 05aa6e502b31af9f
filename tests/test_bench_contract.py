"""bench.py against the driver's contract: the refusal of more than one GPU (no GPU needed)
and, on a GPU, the shape of the one JSON line."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True, timeout=120)
    assert res.returncode != 0
    assert "one GPU" in res.stdout + res.stderr


@pytest.mark.gpu
def test_bench_prints_one_json_line_with_the_contract_keys():
    print("[case] bench.py line", flush=True)
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "1", "--steps", "4",
                          "--warmup", "1", "--no-swap", "--no-fragmented", "--no-prefill", "--no-graph",
                          "--no-rope-step", "--no-mixed", "--no-page8"], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    lines = [l for l in res.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 4 and d["warmup"] == 1 and d["vs_baseline"] is None
    assert d["unit"] == "GB/s" and d["higher_is_better"] is True and d["data"] == "synthetic"
    assert "workload" in d["config"] and "model" not in d["config"]
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["unit"] == "GB/s"
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3 and 0.3 < r["frac"] < 1.0
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["config"] == "configs[0]"
    assert c["cores"] >= 1 and c["value"] > 0 and c["sample"]
    h = c["hip_same_config"]
    assert h["pages_bit_equal"] is True and h["max_rel_err_vs_cpu_per_request"] <= 1e-4 and h["us_per_step"] > 0
    assert c["scalar_port_on_benched_config"]["kind"] == "port"
    assert r["traffic"] is None or "not measured in this run" in r["traffic_source"]
    assert d["value"] > 100 * c["value"]            # the GPU path is not the CPU path in disguise
