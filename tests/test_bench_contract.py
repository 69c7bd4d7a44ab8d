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
    out = subprocess.run([sys.executable, BENCH, "--workload", "c2", "--steps", "4", "--warmup", "1",
                          "--no-also"], capture_output=True, text=True, timeout=110)
    assert out.returncode == 0, out.stderr
    lines = [l for l in out.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
              "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert k in d, k
    assert d["n_gpus"] == 1 and d["steps"] == 4 and d["warmup"] == 1 and d["vs_baseline"] is None
    assert d["unit"] == "env-steps/s" and d["dtype"] == "f32" and d["higher_is_better"] is True
    c = d["config"]
    assert "workload" in c and "model" not in c
    # the launch length belongs to the workload, not to --steps: one bench step = one launch
    assert c["steps_per_launch"] == 10000 and c["launches_timed"] == 4
    assert c["env_steps_timed"] == c["n_envs"] * 10000 * 4
    assert c["launch_ms_min"] <= c["launch_ms_median"] <= c["launch_ms_max"]
    assert abs(d["value"] - c["env_steps_timed"] / (d["ms_per_step"] * 1e-3 * 4)) <= 1e-6 * d["value"]
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-12
    assert r["algorithmic_bytes_per_launch"] == 42.5 * c["n_envs"] * 10000
    want = r["algorithmic_bytes_per_launch"] / (r["kernel_ms_per_launch"] * 1e-3) / 1e9
    assert abs(r["achieved"] - want) <= 1e-9 * want
    b = d["cpu_baseline"]
    assert b["kind"] == "port" and b["cores"] >= 1 and b["value"] > 0 and b["unit"] == "env-steps/s"
    assert b["single_thread"]["cores"] == 1 and b["single_thread"]["value"] > 0
    assert b["nproc"] >= b["cores"] and isinstance(b["cpu_model"], str) and b["cpu_model"]
    assert d["value"] > b["value"]
    # one launch on a fresh engine against what the CPU leg computed from the same seeds
    par = b["parity"]
    assert d["parity_checked"] is True and par["parity_checked"] is True and par["mismatches"] == {}
    assert par["envs"] >= 64 and par["env_steps_each"] == 10000 and par["tables"] == par["envs"]
    # measured traffic (profiles/) beside the algorithmic figure
    assert r["traffic"] == 8.2 * c["n_envs"] * 10000
    want = r["traffic"] / (r["kernel_ms_per_launch"] * 1e-3) / 1e9 / 8000.0
    assert abs(r["hbm_measured_frac"] - want) <= 1e-9 * want


@pytest.mark.gpu
def test_bench_names_the_target_config_and_checks_it(gpu):
    """The shared-table configuration the contract's target is quoted on: reported in a
    `north_star` block with the target, whether it is met, and its own parity check."""
    out = subprocess.run([sys.executable, BENCH, "--workload", "c2", "--steps", "2", "--warmup", "1",
                          "--also-only", "c3"], capture_output=True, text=True, timeout=110)
    assert out.returncode == 0, out.stderr
    d = json.loads([l for l in out.stdout.splitlines() if l.strip()][-1])
    ns = d["north_star"]
    assert ns["target"] == 1e10 and ns["unit"] == "env-steps/s" and ns["config"].startswith("c3")
    assert ns["met"] == (ns["value"] >= 1e10) and ns["value"] > 1e9
    assert ns["parity"]["parity_checked"] is True and ns["parity"]["envs"] == 65536
    c3 = d["also"]["c3"]
    assert c3["launches_timed"] >= 5 and c3["kernel"].startswith("k_shared")
    assert abs(ns["value"] - c3["value_at_median_launch"]) <= 1e-9 * ns["value"]


@pytest.mark.gpu
def test_launch_plan_reported_is_the_plan_that_runs(gpu):
    """A 1000-step and a 20-step launch of the same engine use different plans; the
    report names the one asked about."""
    cfg = gpu.make_config(1 << 18, 16, 16, episode_len=128, gamma=0.95, seed=3)
    cls, start = gpu.gen_maps_bernoulli(3, cfg.n_envs, cfg.n_envs, 16, 16, 0.1, 0.02)
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        long_plan, short_plan = eng.fused_kernel_info(1000), eng.fused_kernel_info(20)
        assert eng.fused_kernel_info(0) == eng.fused_kernel_info(1 << 20)
        assert "hbm+lds" in long_plan["name"] and "hbm+lds" not in short_plan["name"]
        eng.run_fused(20)
        assert eng.fused_split()[1] == 0
        eng.run_fused(1000)
        hbm, lds = eng.fused_split()
        assert lds > 0 and hbm + lds == cfg.n_envs
