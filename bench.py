#!/usr/bin/env python3
"""Benchmark of the fused env-step + epsilon-greedy select + TD-update hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c2|c3|c5]

One "step" advances every env of the workload by one select -> step -> update.
W warm-up steps run first, then exactly K steps are timed with the inputs (maps,
tables, state) already resident in HBM.  Prints ONE JSON line.

Workloads (the benchmark configurations, numbered from 1):
  c2  4096 envs, 32x32, per-env tables (64 MB; cache resident)
  c3  65536 envs sharing one 64x64 map and ONE table (ordered reduction per step)
  c4  1,048,576 envs, 16x16, per-env tables (4 GB; the HBM-bound config)  [default]
  c5  8192 envs, 256x256, 8 actions, per-env tables (16 GB)
"""
import argparse
import ctypes as C
import json
import os
import sys
import threading
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "cudarl-arena_amd"))
import pycrl  # noqa: E402

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E

WORKLOADS = {
    # algorithmic bytes per env-step: 22 B of state/outputs + (4A+4) B of table
    # traffic (one new row, one write) + S/(8T) B of map per episode (+4 B/cell reward)
    "c2": dict(n=4096, w=32, h=32, a=4, t=256, steps=10000, warmup=256, bytes=42.5,
               name="c2: 4096 envs 32x32, per-env tables 1024x4, eps 0.1, T=256"),
    "c3": dict(n=65536, w=64, h=64, a=4, t=0, steps=1000, warmup=50, bytes=24.0,
               name="c3: 65536 envs, shared 64x64 map, one shared table 4096x4, ordered reduction"),
    # traffic: HBM bytes per env-step from rocprofv3 FETCH_SIZE x2.000 + WRITE_SIZE x1.000
    # (profiles/k_fused_tickets_c4.md), valid for the default launch only
    "c4": dict(n=1 << 20, w=16, h=16, a=4, t=128, steps=1000, warmup=128, bytes=42.25, traffic=30.8,
               name="c4: 1048576 envs 16x16, per-env tables 256x4 (4 GB), traps, eps 0.1, T=128"),
    "c5": dict(n=8192, w=256, h=256, a=8, t=1024, steps=1024, warmup=64, bytes=70.0,
               name="c5: 8192 envs 256x256, 8 actions, per-env tables 65536x8 (16 GB), cell rewards"),
}


def build_workload(key, n_override=None):
    wl = WORKLOADS[key]
    n = n_override or wl["n"]
    if key == "c2":
        cfg = pycrl.make_config(n, 32, 32, episode_len=256, lr=0.1, gamma=0.99, eps0=0.1, seed=0)
        cls, start = pycrl.gen_maps_bernoulli(0, n, n, 32, 32, 0.2)
        return cfg, cls, start, None
    if key == "c3":
        cfg = pycrl.make_config(n, 64, 64, table_mode=pycrl.TABLE_SHARED, map_mode=pycrl.MAP_SHARED,
                                lr=0.05, gamma=0.99, eps0=0.2, seed=0)
        cls, start = pycrl.gen_maps_bernoulli(0, 1, n, 64, 64, 0.15)
        return cfg, cls, start, None
    if key == "c4":
        cfg = pycrl.make_config(n, 16, 16, episode_len=128, lr=0.1, gamma=0.95, eps0=0.1, seed=0,
                                trap_reward=-1.0)
        cls, start = pycrl.gen_maps_bernoulli(0, n, n, 16, 16, 0.1, 0.02)
        return cfg, cls, start, None
    if key == "c5":
        cfg = pycrl.make_config(n, 256, 256, n_actions=8, episode_len=1024, lr=0.1, gamma=0.99,
                                eps_mode=pycrl.EPS_EPISODE_LINEAR, eps0=1.0, eps_end=0.05, eps_span=100,
                                seed=0, reward_flags=pycrl.REWARD_CELLS | pycrl.REWARD_BASE_CELLS)
        cls, start, cr = pycrl.gen_maps_noise(0, n, 256, 256, 16, 0.25, 0.05, 10.0)
        return cfg, cls, start, cr
    raise SystemExit("unknown workload %r" % key)


class HipEvents:
    """hipEvent timing on the stream the engine launches on (the null stream)."""

    def __init__(self):
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [C.c_void_p]
        self.hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.hip.hipEventDestroy.argtypes = [C.c_void_p]

    def pair(self):
        a, b = C.c_void_p(), C.c_void_p()
        assert self.hip.hipEventCreate(C.byref(a)) == 0 and self.hip.hipEventCreate(C.byref(b)) == 0
        return a, b

    def record(self, ev):
        assert self.hip.hipEventRecord(ev, None) == 0

    def elapsed_ms(self, a, b):
        assert self.hip.hipEventSynchronize(b) == 0
        ms = C.c_float()
        assert self.hip.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return float(ms.value)


def time_gpu(key, steps, warmup, launches=1, n_override=None, resident=0, variant=0):
    """-> dict(steps_per_s, ms_per_step, kernel_ms, wall_s, info)"""
    wl = WORKLOADS[key]
    cfg, cls, start, cr = build_workload(key, n_override)
    n = cfg.n_envs
    ev = HipEvents()
    with pycrl.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start, cr)
        del cls, cr
        if resident:
            eng.set_resident_envs(resident)
        if variant:
            eng.set_fused_variant(variant)
        info = eng.fused_kernel_info()
        if warmup:
            eng.run_fused(warmup)
        eng.sync()
        a, b = ev.pair()
        per_launch = steps // launches
        counts = [per_launch] * launches
        counts[-1] += steps - per_launch * launches
        t0 = time.perf_counter()
        ev.record(a)
        for c in counts:
            eng.run_fused(c)
        ev.record(b)
        eng.sync()
        wall = time.perf_counter() - t0
        dev_ms = ev.elapsed_ms(a, b)
        st = eng.get_state()
        split = eng.fused_split()
    secs = max(wall, dev_ms * 1e-3)
    return dict(n=n, steps_per_s=n * steps / secs, ms_per_step=secs * 1e3 / steps, device_ms=dev_ms,
                wall_s=wall, launches=launches, info=info, split=split, episodes_min=int(st["episode"].min()),
                bytes_per_step=wl["bytes"])


def time_cpu(key, n_sample, steps, threads):
    """The oracle (a scalar C port of the reference's kernels) on `threads` host
    threads over the first n_sample envs of the same workload."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from conftest import ORACLE_SO, Oracle
    if not os.path.exists(ORACLE_SO):
        import subprocess
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "-s"])
    orc = Oracle(C.CDLL(ORACLE_SO))
    cfg, cls, start, cr = build_workload(key, n_sample)
    S, A = cfg.width * cfg.height, cfg.n_actions
    st = orc.new_state(cfg, start)
    if cfg.table_mode == pycrl.TABLE_SHARED:
        Q = np.zeros((1, S, A), np.float32)
        t0 = time.perf_counter()
        orc.run(cfg, cls, cr, start, Q, st, 0, steps)
        dt = time.perf_counter() - t0
        return n_sample * steps / dt, 1, dt
    Q = np.zeros((n_sample, S, A), np.float32)
    p = Oracle._p
    bounds = [n_sample * i // threads for i in range(threads + 1)]

    def work(lo, hi):
        rc = orc.lib.orc_run_range(C.byref(cfg), lo, hi, p(cls), p(cr), p(start), p(Q), p(st["s"]),
                                   p(st["ep_step"]), p(st["episode"]), p(st["reward"]), p(st["done"]),
                                   p(st["action"]), 0, steps)
        assert rc == 0

    ths = [threading.Thread(target=work, args=(bounds[i], bounds[i + 1])) for i in range(threads)]
    t0 = time.perf_counter()
    for t in ths:
        t.start()
    for t in ths:
        t.join()
    dt = time.perf_counter() - t0
    return n_sample * steps / dt, threads, dt


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS))
    ap.add_argument("--launches", type=int, default=1, help="split the K timed steps over this many launches")
    ap.add_argument("--envs", type=int, default=None, help="override the env count (not a headline figure)")
    ap.add_argument("--resident", type=int, default=0, help="envs in flight at once (0 = automatic)")
    ap.add_argument("--variant", type=int, default=0, help="fused kernel: 0 automatic, 1 plain, 2 hybrid")
    ap.add_argument("--probe-copy", type=int, default=0, metavar="MIB",
                    help="only run one plain copy kernel of this many MiB (calibrates rocprofv3 counters)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-also", action="store_true", help="skip the short c2/c3/c5 side measurements")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on ONE GPU (envs shard trivially, but no second "
                         "GPU is used in this run); got --gpus %d" % args.gpus)
    lib = pycrl.load()
    if lib.crl_device_count() < 1:
        raise SystemExit("bench.py: no HIP device: %s" % lib.crl_last_error().decode())

    if args.probe_copy:
        pycrl._check(lib.crl_probe_copy(args.probe_copy << 20, 3))
        print(json.dumps({"probe_copy_bytes_per_launch": args.probe_copy << 20, "launches": 3}))
        return
    key = args.workload
    wl = WORKLOADS[key]
    steps = args.steps if args.steps is not None else wl["steps"]
    warmup = args.warmup if args.warmup is not None else wl["warmup"]
    g = time_gpu(key, steps, warmup, args.launches, args.envs, args.resident, args.variant)

    achieved = g["steps_per_s"] * wl["bytes"] / 1e9
    # the dominant kernel's own duration (device events around its launches)
    kern_achieved = g["n"] * steps * wl["bytes"] / (g["device_ms"] * 1e-3) / 1e9
    out = {
        "metric": "env-steps/sec (step+select+TD update) at 1 MI355X",
        "value": g["steps_per_s"],
        "unit": "env-steps/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": g["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic (Philox-seeded maps, zero-initialised tables)",
        "config": {"workload": wl["name"], "n_envs": g["n"], "steps_per_launch": steps // args.launches,
                   "kernel": g["info"]["name"], "grid": g["info"]["grid"], "block": g["info"]["block"],
                   "lds_bytes": g["info"]["lds_bytes"],
                   "envs_stepped_from_hbm_tables": g["split"][0], "envs_stepped_from_lds_tables": g["split"][1]},
        "roofline": {"bound": "hbm", "achieved": kern_achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": kern_achieved / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes_per_env_step": wl["bytes"],
                     "kernel_ms_per_launch": g["device_ms"] / args.launches,
                     "whole_job_GBps": achieved},
    }
    if ("traffic" in wl and steps == wl["steps"] and args.launches == 1 and not args.envs
            and not args.resident):
        # measured in separate rocprofv3 --pmc runs of this same command, not in this run
        out["roofline"]["traffic"] = wl["traffic"] * g["n"] * steps

    if not args.no_cpu:
        threads = min(16, os.cpu_count() or 1)
        # about 10-30 s of CPU work each (the wall time is that divided by the threads)
        n_sample = {"c2": 4096, "c3": 65536, "c4": 1 << 18, "c5": 2048}[key]
        cpu_steps = {"c2": 50000, "c3": 1500, "c4": 1000, "c5": 16384}[key]
        v, cores, dt = time_cpu(key, min(n_sample, g["n"]), cpu_steps, threads)
        out["cpu_baseline"] = {"value": v, "unit": "env-steps/s", "cores": cores, "kind": "port",
                               "sample": "%d envs x %d steps of the same workload, %.1f s wall on %d threads"
                                         % (min(n_sample, g["n"]), cpu_steps, dt, cores)}
    if not args.no_also and not args.envs:
        also = {}
        for k2, s2, w2 in (("c3", 300, 20), ("c2", 4000, 256), ("c5", 1024, 64)):
            if k2 == key:
                continue
            r = time_gpu(k2, s2, w2)
            also[k2] = {"workload": WORKLOADS[k2]["name"], "value": r["steps_per_s"], "unit": "env-steps/s",
                        "steps": s2, "ms_per_step": r["ms_per_step"], "kernel": r["info"]["name"]}
        out["also"] = also
    print(json.dumps(out))


if __name__ == "__main__":
    main()
