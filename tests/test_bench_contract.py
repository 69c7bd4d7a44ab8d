"""bench.py's contract: one JSON line with the agreed keys, and a clear refusal
of more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused():
    out = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=60)
    assert out.returncode != 0
    assert "ONE GPU" in out.stderr


@pytest.mark.gpu
def test_bench_prints_one_json_line_with_the_contract_keys(gpu):
    out = subprocess.run([sys.executable, BENCH, "--workload", "c2", "--steps", "200", "--warmup", "20",
                          "--no-also"], capture_output=True, text=True, timeout=110)
    assert out.returncode == 0, out.stderr
    lines = [l for l in out.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
              "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert k in d, k
    assert d["n_gpus"] == 1 and d["steps"] == 200 and d["warmup"] == 20 and d["vs_baseline"] is None
    assert d["unit"] == "env-steps/s" and d["dtype"] == "f32" and d["higher_is_better"] is True
    assert "workload" in d["config"] and "model" not in d["config"]
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-12
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] >= 1 and c["value"] > 0 and c["unit"] == "env-steps/s"
    assert d["value"] > c["value"]
