"""GPU parity on randomly drawn configurations: every switch of the configuration
(actions, grid shape, table and map sharing, reward source, goal rule, restart,
time limit, epsilon schedule, TD max, episode budget, trace, kernel variant, envs
in flight, launch splits) in combinations no hand-written case lists.  Final
state and tables - and the whole trajectory when traced - must be the oracle's,
bit for bit.  Seeds are fixed: a failure names its case."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

STATE = ("s", "ep_step", "episode", "reward", "done", "action")


def same(gpu_q, gpu_state, Q, ost):
    return (np.array_equal(gpu_q.reshape(Q.shape), Q, equal_nan=True) and
            all(np.array_equal(gpu_state[k], ost[k]) for k in STATE))


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_configs_folded_loop(gpu, oracle, seed):
    """The common configuration (fixed epsilon, class rewards, goal on the target
    cell, restart) on per-env tables: the folded loop of both kinds of workers."""
    rng = np.random.default_rng(seed)
    for case in range(40):
        A = int(rng.choice([4, 8]))
        small = rng.random() < 0.5  # small grids: 32 whole tables fit LDS
        W, H = (int(rng.integers(2, 17 if small else 40)) for _ in range(2))
        N = int(rng.choice([1, 31, 33, 64, 65, 500, 2049, 4100, 9000]))
        T = int(rng.choice([0, 1, 2, 7, 50, 300]))
        steps, t0 = int(rng.integers(1, 200)), int(rng.integers(0, 5))
        eps = float(rng.choice([0.0, 0.05, 0.3, 1.0]))
        variant, resident = int(rng.choice([0, 1, 2])), int(rng.choice([0, 64, 200, 1000, 5000]))
        p_wall, p_trap = float(rng.choice([0.0, 0.1, 0.3])), float(rng.choice([0.0, 0.05]))
        map_seed = int(rng.integers(0, 1 << 30))
        cls, start = gpu.gen_maps_bernoulli(map_seed, N, N, W, H, p_wall, p_trap)
        cfg = gpu.make_config(N, W, H, n_actions=A, episode_len=T, eps0=eps, gamma=0.93, lr=0.2, seed=map_seed,
                              trap_reward=-0.7)
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, start)
            eng.set_fused_variant(variant)
            eng.set_resident_envs(resident)
            eng.step_count = t0
            name = eng.fused_kernel_info()["name"]
            third = steps // 3
            for c in (third, steps - 2 * third, third):
                eng.run_fused(c)
            q, st = eng.q_get(0, N), eng.get_state()
        Q = np.zeros((N, W * H, A), np.float32)
        ost = oracle.new_state(cfg, start)
        oracle.run(cfg, cls, None, start, Q, ost, t0, steps)
        assert "fast" in name
        assert same(q, st, Q, ost), (seed, case, name, A, W, H, N, T, steps, t0, eps, variant, resident)


@pytest.mark.parametrize("seed", [8, 9])
def test_random_configs_folded_loop_cell_rewards_and_schedules(gpu, oracle, seed):
    """Per-env maps small enough for LDS with per-cell rewards and / or an epsilon
    that follows the episode count: the ticket kernel runs the folded loop's variant
    for them (plain workers only; staged or derived move codes, two lanes per env
    on small batches)."""
    rng = np.random.default_rng(seed)
    for case in range(40):
        A = int(rng.choice([4, 8]))
        W, H = (int(rng.integers(2, 40)) for _ in range(2))
        N = int(rng.choice([1, 31, 33, 64, 65, 500, 2049, 4100, 17000]))
        T = int(rng.choice([0, 1, 2, 7, 50, 300]))
        steps, t0 = int(rng.integers(1, 450)), int(rng.integers(0, 5))
        eps_mode, span = int(rng.choice([0, 2, 3])), int(rng.integers(1, 30))
        flags = int(rng.choice([0, gpu.REWARD_CELLS, gpu.REWARD_CELLS | gpu.REWARD_BASE_CELLS]))
        if eps_mode == 0 and flags == 0:
            flags = gpu.REWARD_CELLS
        resident = int(rng.choice([0, 64, 200, 1000, 5000]))
        map_seed = int(rng.integers(0, 1 << 30))
        if flags:
            cls, start, cr = gpu.gen_maps_noise(map_seed, N, W, H, 8, 0.2, 0.3, 5.0)
        else:
            cls, start = gpu.gen_maps_bernoulli(map_seed, N, N, W, H, 0.15, 0.05)
            cr = None
        cfg = gpu.make_config(N, W, H, n_actions=A, episode_len=T, lr=0.2, gamma=0.9, reward_flags=flags,
                              eps_mode=eps_mode, eps0=float(rng.choice([0.0, 0.3, 0.6, 1.0])), eps_decay=0.9,
                              eps_end=0.05, eps_span=span, seed=map_seed, trap_reward=-0.5)
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, start, cr)
            eng.set_resident_envs(resident)
            eng.step_count = t0
            name = eng.fused_kernel_info()["name"]
            third = steps // 3
            for c in (third, steps - 2 * third, third):
                eng.run_fused(c)
            q, st = eng.q_get(0, N), eng.get_state()
        Q = np.zeros((N, W * H, A), np.float32)
        ost = oracle.new_state(cfg, start)
        oracle.run(cfg, cls, cr, start, Q, ost, t0, steps)
        assert name.startswith("k_fused_tickets") and "fast+" in name, name
        assert same(q, st, Q, ost), (seed, case, name, A, W, H, N, T, steps, t0, eps_mode, flags, resident)


@pytest.mark.parametrize("seed", [4, 5])
def test_random_configs_folded_loop_large_or_shared_maps(gpu, oracle, seed):
    """The folded loop's variant for maps that are shared or too large for LDS:
    per-cell rewards (all three reward sources), epsilon fixed or following the
    env's episode count, 4 and 8 actions, short and long episodes."""
    rng = np.random.default_rng(seed)
    for case in range(40):
        A = int(rng.choice([4, 8]))
        shared_map = rng.random() < 0.5
        big = rng.random() < (0.3 if shared_map else 1.0)  # per-env maps reach this kernel only when large
        W, H = (int(rng.integers(65, 100)) if big else int(rng.integers(2, 40)) for _ in range(2))
        # (up to 16,384 envs the kernel gives every env two lanes)
        N = int(rng.choice([1, 63, 64, 65, 300, 1000] if big else [1, 33, 257, 700, 3000, 17000]))
        T = int(rng.choice([0, 1, 2, 9, 40, 400]))
        steps, t0 = int(rng.integers(1, 160)), int(rng.integers(0, 5))
        eps_mode, span = int(rng.choice([0, 2, 3])), int(rng.integers(1, 30))
        flags = int(rng.choice([0, gpu.REWARD_CELLS, gpu.REWARD_CELLS | gpu.REWARD_BASE_CELLS]))
        map_seed = int(rng.integers(0, 1 << 30))
        n_maps = 1 if shared_map else N
        if flags:
            cls, start, cr = gpu.gen_maps_noise(map_seed, n_maps, W, H, 8, 0.2, 0.3, 5.0)
            start = np.resize(start, N).astype(np.int32)
        else:
            cls, start = gpu.gen_maps_bernoulli(map_seed, n_maps, N, W, H, 0.15, 0.05)
            cr = None
        cfg = gpu.make_config(N, W, H, n_actions=A, map_mode=gpu.MAP_SHARED if shared_map else gpu.MAP_PER_ENV,
                              episode_len=T, lr=0.2, gamma=0.9, reward_flags=flags, eps_mode=eps_mode,
                              eps0=float(rng.choice([0.0, 0.3, 0.6, 1.0])), eps_decay=0.9, eps_end=0.05,
                              eps_span=span, seed=map_seed, trap_reward=-0.5)
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, start, cr)
            eng.step_count = t0
            name = eng.fused_kernel_info()["name"]
            third = steps // 3
            for c in (third, steps - 2 * third, third):
                eng.run_fused(c)
            q, st = eng.q_get(0, N), eng.get_state()
        Q = np.zeros((N, W * H, A), np.float32)
        ost = oracle.new_state(cfg, start)
        oracle.run(cfg, cls, cr, start, Q, ost, t0, steps)
        assert name.startswith("k_fused_per_env") and "fast" in name, name
        assert same(q, st, Q, ost), (seed, case, name, A, W, H, N, T, steps, t0, eps_mode, flags, shared_map)


@pytest.mark.parametrize("seed", [1, 7])
def test_random_configs_general(gpu, oracle, seed):
    """Everything else: shared tables and maps, maps too large for LDS, per-cell
    rewards, goal test on the resulting cell, sticky done, epsilon schedules, the
    zero-floored max, episode budgets, traces."""
    rng = np.random.default_rng(seed)
    for case in range(60):
        A = int(rng.choice([4, 8]))
        big = rng.random() < 0.25  # more than 4096 cells: the map stays in global memory
        W, H = (int(rng.integers(65, 90)) if big else int(rng.integers(2, 30)) for _ in range(2))
        shared_table = rng.random() < 0.35
        shared_map = shared_table or rng.random() < 0.3
        N = int(rng.choice([5, 70, 300] if big else [1, 33, 257, 700, 3000]))
        T = int(rng.choice([0, 1, 3, 20, 100]))
        steps = int(rng.integers(1, 90 if shared_table else 200))
        eps_mode, span = int(rng.choice([0, 1, 2, 3])), int(rng.integers(1, 50))
        flags = int(rng.choice([0, gpu.REWARD_CELLS, gpu.REWARD_CELLS | gpu.REWARD_BASE_CELLS]))
        goal_mode, max_mode = int(rng.choice([0, 1])), int(rng.choice([0, 1]))
        auto_reset = int(rng.choice([0, 1, 1]))
        max_episodes = int(rng.choice([0, 0, 2])) if auto_reset else 0
        map_seed = int(rng.integers(0, 1 << 30))
        n_maps = 1 if shared_map else N
        if flags:
            cls, start, cr = gpu.gen_maps_noise(map_seed, n_maps, W, H, 8, 0.2, 0.3, 5.0)
            start = np.resize(start, N).astype(np.int32)
        else:
            cls, start = gpu.gen_maps_bernoulli(map_seed, n_maps, N, W, H, 0.15, 0.05)
            cr = None
        cfg = gpu.make_config(N, W, H, n_actions=A,
                              table_mode=gpu.TABLE_SHARED if shared_table else gpu.TABLE_PER_ENV,
                              map_mode=gpu.MAP_SHARED if shared_map else gpu.MAP_PER_ENV, max_mode=max_mode,
                              goal_mode=goal_mode, auto_reset=auto_reset, episode_len=T,
                              lr=0.002 if shared_table else 0.2, gamma=0.9, reward_flags=flags, eps_mode=eps_mode,
                              eps0=0.6, eps_decay=0.97, eps_end=0.05, eps_span=span, seed=map_seed,
                              max_episodes=max_episodes, trap_reward=-0.5)
        n_tables = 1 if shared_table else N
        trace_n = N if rng.random() < 0.5 else 0
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, start, cr)
            if trace_n:
                eng.set_trace(trace_n, steps)
            name = eng.fused_kernel_info()["name"]
            eng.run_fused(steps // 2)
            eng.run_fused(steps - steps // 2)
            tr = eng.get_trace(steps) if trace_n else None
            q, st = eng.q_get(0, n_tables), eng.get_state()
        Q = np.zeros((n_tables, W * H, A), np.float32)
        ost = oracle.new_state(cfg, start)
        want = oracle.run(cfg, cls, cr, start, Q, ost, 0, steps, trace_n=trace_n)
        what = (seed, case, name, A, W, H, N, T, steps, eps_mode, flags, goal_mode, auto_reset, max_mode,
                max_episodes, shared_table, shared_map, trace_n)
        assert same(q, st, Q, ost), what
        if trace_n:
            assert all(np.array_equal(tr[k], want[k]) for k in ("s_next", "action", "reward", "done")), what


@pytest.mark.parametrize("seed", [7, 8])
def test_random_configs_shared_table(gpu, oracle, seed):
    """One shared table under the ordered reduction at every size of table and batch the
    one-launch kernel takes (3x3 to 64x64 cells, 300 to 65,536 envs, learning rates from
    tame to diverging, episodes of one step to none), through one launch per call and
    through two launches per step, calls split at a random step."""
    rng = np.random.default_rng(seed)
    for case in range(12):
        A = int(rng.choice([4, 4, 8]))
        W, H = int(rng.integers(3, 65)), int(rng.integers(3, 65))
        while W * H * A > 16384:
            H = max(3, H // 2)
        N = int(rng.choice([300, 1000, 5000, 20000, 65536]))
        lr = float(rng.choice([0.0005, 0.01, 0.05, 0.3]))
        steps = int(rng.integers(20, 120)) if N > 20000 else int(rng.integers(50, 300))
        cls, start = gpu.gen_maps_bernoulli(int(rng.integers(1, 99)), 1, N, W, H, float(rng.uniform(0, 0.25)),
                                            float(rng.uniform(0, 0.05)))
        cfg = gpu.make_config(N, W, H, n_actions=A, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=lr,
                              eps0=float(rng.uniform(0.05, 1.0)), episode_len=int(rng.choice([0, 1, 7, 40])),
                              seed=int(rng.integers(1, 1000)), trap_reward=-0.5)
        first = int(rng.integers(1, steps))
        variant = 1 if case % 4 == 3 else 2
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, start)
            eng.set_fused_variant(variant)
            name = eng.fused_kernel_info(first)["name"]
            eng.run_fused(first)
            eng.run_fused(steps - first)
            q, st = eng.q_get(0, 1), eng.get_state()
        Q = np.zeros((1, W * H, A), np.float32)
        ost = oracle.new_state(cfg, start)
        oracle.run(cfg, cls, None, start, Q, ost, 0, steps)
        assert same(q, st, Q, ost), (seed, case, name, A, W, H, N, lr, steps, first)
