"""bench.py's one line: the keys the driver reads, on a short run of the smallest layer workload."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu


def test_bench_prints_one_json_line_with_the_contract_keys(dev):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    print("bench line", flush=True)
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--workload", "qwen3_30b_t64_zipf",
                        "--steps", "5", "--warmup", "2"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, r.stdout[-2000:]
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 2 and d["higher_is_better"] is True
    assert d["vs_baseline"] is None and d["data"] == "synthetic" and d["config"]["workload"] == "qwen3_30b_t64_zipf"
    assert abs(d["value"] - d["config"]["T"] / (d["ms_per_step"] * 1e-3)) / d["value"] < 1e-3
    roof = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert 0.0 < roof["frac"] < 1.0
    cpu = d["cpu_baseline"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in cpu, key
    assert cpu["kind"] == "port" and cpu["value"] > 0
