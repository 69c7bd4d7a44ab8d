"""crl_run_fused_noalloc, the entry point for callers that cannot allocate: through
the C ABI, against crl_run_fused on the same inputs, bit for bit - two calls in a
row on one GPU, the second with a smaller input, for per-env tables (scratch: the
ticket counters) and for a shared table (scratch: the hand-off cells of the ordered
reduction) - and no device memory taken or returned while it runs."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def free_device_bytes():
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def run_pair(gpu, cfg, cls, start, chunks, n_tables, variant=0):
    """-> (state, tables) after the launches in `chunks`, once per entry point"""
    out = []
    for noalloc in (False, True):
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, start)
            if variant:
                eng.set_fused_variant(variant)
            eng.sync()
            before = free_device_bytes()
            for c in chunks:
                (eng.run_fused_noalloc if noalloc else eng.run_fused)(c)
            eng.sync()
            if noalloc:
                assert free_device_bytes() == before  # nothing allocated, nothing freed
            out.append((eng.get_state(), eng.q_get(0, n_tables), eng.fused_split(), eng.step_count))
    (st_a, q_a, split_a, t_a), (st_b, q_b, split_b, t_b) = out
    assert t_a == t_b == sum(chunks)
    assert np.array_equal(q_a, q_b, equal_nan=True)
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(st_a[k], st_b[k]), k
    assert sum(split_a) == sum(split_b)
    return st_b, q_b


def test_noalloc_per_env_tables_two_calls_second_smaller(gpu):
    big = None
    for N, W, H, chunks in ((70000, 16, 16, (150, 37)), (3000, 12, 9, (90,))):  # hybrid and plain ticket kernels
        cls, start = gpu.gen_maps_bernoulli(3, N, N, W, H, 0.1, 0.02)
        cfg = gpu.make_config(N, W, H, episode_len=64, gamma=0.95, eps0=0.15, seed=11)
        st, q = run_pair(gpu, cfg, cls, start, chunks, N)
        assert np.count_nonzero(q) > N and st["episode"].min() >= 1
        big = big or N
    assert big == 70000


def test_noalloc_shared_table_two_calls_second_smaller(gpu):
    for N, W, H, steps in ((65536, 64, 64, 40), (5000, 16, 16, 60)):
        cls, start = gpu.gen_maps_bernoulli(2, 1, N, W, H, 0.15)
        cfg = gpu.make_config(N, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.002,
                              eps0=0.2, episode_len=50, seed=13)
        for variant in (0, 2):  # two launches per step; all steps in one launch (its flags, too, come from the scratch)
            st, q = run_pair(gpu, cfg, cls, start, (steps,), 1, variant)
            assert np.isfinite(q).all() and np.count_nonzero(q) > 100


def test_noalloc_rejects_a_reduction_larger_than_the_scratch(gpu):
    # 262,144 envs on a 64x64x4 table: 256 owners x 1024 blocks x 64 B = 16 MB of hand-off cells
    N, W, H = 1 << 18, 64, 64
    cls, start = gpu.gen_maps_bernoulli(2, 1, N, W, H, 0.15)
    cfg = gpu.make_config(N, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.001, seed=1)
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        with pytest.raises(gpu.CrlError) as err:
            eng.run_fused_noalloc(1)
        assert err.value.code == -5 and "static scratch" in str(err.value)
        assert eng.step_count == 0
        eng.run_fused(2)  # the allocating entry point still takes it
        assert eng.step_count == 2
