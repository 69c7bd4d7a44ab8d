"""GPU parity: the HIP engine, called through its C ABI, against the CPU oracle on
the same seeded inputs.  Bar: trajectories (s', action, reward, done) bit-exact;
fp32 Q-tables within 1e-5 relative (the tests assert the stronger bit equality
first and report the relative error if that fails)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REL_TOL = 1e-5  # the stated bar: fp32 Q-tables within 1e-5 relative


def assert_q_close(got, want):
    # summed deltas can overflow a shared table (the effective step size is lr
    # times the number of envs on one (s,a)); NaNs must then sit in the same places
    if np.array_equal(got, want, equal_nan=True):
        return
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    got, want = np.nan_to_num(got, posinf=0, neginf=0), np.nan_to_num(want, posinf=0, neginf=0)
    denom = np.maximum(np.maximum(np.abs(got), np.abs(want)), 1e-30)
    rel = np.abs(got - want) / denom
    assert rel.max() <= REL_TOL, "Q tables differ: max rel %.3g at %s" % (rel.max(), np.argmax(rel))
    pytest.fail("Q tables within 1e-5 but not bit-identical (max rel %.3g)" % rel.max())


def assert_trace_equal(got, want):
    for k in ("s_next", "action", "reward", "done"):
        if not np.array_equal(got[k], want[k]):
            bad = np.argwhere(got[k] != want[k])[0]
            pytest.fail("trace %s differs first at step %d env %d: %r vs %r"
                        % (k, bad[0], bad[1], got[k][tuple(bad)], want[k][tuple(bad)]))


def run_both(gpu, oracle, cfg, cls, start, n_steps, cr=None, chunks=None, trace_n=None, stream=None, variant=0):
    N = cfg.n_envs
    trace_n = N if trace_n is None else trace_n
    A, S = cfg.n_actions, cfg.width * cfg.height
    n_tables = 1 if cfg.table_mode == gpu.TABLE_SHARED else N
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start, cr)
        eng.set_trace(trace_n, n_steps)
        if variant:
            eng.set_fused_variant(variant)
        if stream is not None:
            eng.set_exploration_stream(*stream)
        for c in (chunks or [n_steps]):
            eng.run_fused(c)
        tr = eng.get_trace(n_steps)
        q = eng.q_get(0, n_tables).reshape(n_tables, S, A)
        st = eng.get_state()
        assert eng.step_count == n_steps
    Q = np.zeros((n_tables, S, A), np.float32)
    ost = oracle.new_state(cfg, start)
    want = oracle.run(cfg, cls, cr, start, Q, ost, 0, n_steps, trace_n=trace_n,
                      u=None if stream is None else stream[0], a_rand=None if stream is None else stream[1])
    assert_trace_equal(tr, want)
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(st[k], ost[k]), k
    assert_q_close(q, Q)
    return tr, q


# ---- per-env tables, fused ------------------------------------------------------

@pytest.mark.parametrize("N,W,H,T,steps", [
    (1, 10, 10, 0, 300),       # one env, no time limit
    (65, 7, 5, 11, 200),       # ragged: not a multiple of the wave or of 16 cells
    (512, 32, 32, 256, 1000),  # config 2 shape, reduced N
    (4096, 16, 16, 128, 300),  # config 4 shape, reduced N
])
def test_fused_per_env_matches_oracle(gpu, oracle, N, W, H, T, steps):
    cls, start = gpu.gen_maps_bernoulli(7, N, N, W, H, 0.15, 0.03)
    cfg = gpu.make_config(N, W, H, episode_len=T, eps0=0.1, gamma=0.95, seed=11, trap_reward=-1.0)
    tr, _ = run_both(gpu, oracle, cfg, cls, start, steps)
    if N >= 512:
        assert tr["done"].sum() > 0  # goals reached: the restart path ran


def test_fused_chunked_equals_one_launch(gpu, oracle):
    """K steps in one launch == the same steps split over launches (odd splits
    exercise the two-steps-per-Philox-block bookkeeping)."""
    N, W, H = 300, 12, 9
    cls, start = gpu.gen_maps_bernoulli(3, N, N, W, H, 0.2)
    cfg = gpu.make_config(N, W, H, episode_len=20, eps0=0.3, seed=5)
    run_both(gpu, oracle, cfg, cls, start, 101, chunks=[1, 1, 3, 7, 30, 59])


def test_fused_result_independent_of_resident_envs(gpu, oracle):
    """Few envs in flight (blocks loop over chunks, re-staging maps) == all at once,
    for the plain kernel and for the hybrid one (the last wave of each workgroup steps
    envs whose tables it holds in LDS; N is not a multiple of the 32-env ticket)."""
    N, W, H, T = 3001, 16, 16, 150
    cls, start = gpu.gen_maps_bernoulli(31, N, N, W, H, 0.1, 0.02)
    cfg = gpu.make_config(N, W, H, episode_len=40, eps0=0.2, gamma=0.95, seed=17)
    outs = []
    for resident, variant in ((0, 1), (64, 1), (640, 1), (1000, 1), (0, 2), (256, 2), (1024, 2), (1500, 2), (2200, 2),
                              (3000, 2)):
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, start)
            eng.set_resident_envs(resident)
            eng.set_fused_variant(variant)
            info = eng.fused_kernel_info()
            assert ("hbm+lds" in info["name"]) == (variant == 2), info
            eng.set_trace(N, T)
            eng.run_fused(T)
            outs.append((eng.get_trace(T), eng.q_get(0, N), eng.get_state()))
    Q = np.zeros((N, W * H, 4), np.float32)
    st = oracle.new_state(cfg, start)
    want = oracle.run(cfg, cls, None, start, Q, st, 0, T, trace_n=N)
    for tr, q, got in outs:
        assert_trace_equal(tr, want)
        assert_q_close(q, Q)
        assert np.array_equal(got["s"], st["s"]) and np.array_equal(got["episode"], st["episode"])


@pytest.mark.parametrize("variant", [1, 2])
@pytest.mark.parametrize("N,W,H,T,steps,t_odd", [(4097, 16, 16, 128, 300, 0), (700, 32, 32, 50, 401, 1),
                                                 (33, 5, 7, 9, 77, 1)])
def test_fused_fast_loop_matches_oracle(gpu, oracle, variant, N, W, H, T, steps, t_odd):
    """Without a trace the common configuration runs the folded loop; final state
    and tables must still be the oracle's, for waves on HBM tables and (variant 2)
    the wave that steps envs from LDS-resident tables, from even and odd start steps."""
    cls, start = gpu.gen_maps_bernoulli(41, N, N, W, H, 0.12, 0.03)
    cfg = gpu.make_config(N, W, H, episode_len=T, eps0=0.15, gamma=0.95, seed=19, trap_reward=-1.0)
    S = W * H
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        eng.set_fused_variant(variant)
        eng.step_count = t_odd
        info = eng.fused_kernel_info()
        assert "fast" in info["name"], info
        if variant == 2 and S * 4 * 4 <= 4096:
            assert "hbm+lds" in info["name"], info
        eng.run_fused(steps // 2)
        eng.run_fused(steps - steps // 2)
        q, st = eng.q_get(0, N), eng.get_state()
        hbm, lds = eng.fused_split()
    assert hbm + lds == N
    Q = np.zeros((N, S, 4), np.float32)
    ost = oracle.new_state(cfg, start)
    oracle.run(cfg, cls, None, start, Q, ost, t_odd, steps)
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(st[k], ost[k]), k
    assert_q_close(q.reshape(N, S, 4), Q)
    assert st["episode"].max() >= 1


@pytest.mark.parametrize("variant", [1, 2])
def test_fused_fast_loop_short_launches_no_time_limit(gpu, oracle, variant):
    """The folded loop in launches of 0, 1, 2 and 3 steps (tables staged in and out
    of LDS around a single step; odd and even first steps) and without a time limit
    (episodes end on the goal only)."""
    N, W, H = 2300, 12, 12
    cls, start = gpu.gen_maps_bernoulli(53, N, N, W, H, 0.1, 0.02)
    cfg = gpu.make_config(N, W, H, episode_len=0, eps0=0.25, gamma=0.9, seed=31)
    chunks = [1, 0, 1, 2, 3, 1, 40, 1]
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        eng.set_fused_variant(variant)
        assert "fast" in eng.fused_kernel_info()["name"]
        for c in chunks:
            eng.run_fused(c)
        q, st = eng.q_get(0, N), eng.get_state()
        assert eng.step_count == sum(chunks)
    Q = np.zeros((N, W * H, 4), np.float32)
    ost = oracle.new_state(cfg, start)
    oracle.run(cfg, cls, None, start, Q, ost, 0, sum(chunks))
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(st[k], ost[k]), k
    assert_q_close(q.reshape(Q.shape), Q)


@pytest.mark.parametrize("variant,resident", [(1, 0), (1, 192), (2, 0)])
@pytest.mark.parametrize("N,W,H,A", [(2500, 16, 16, 8), (300, 9, 6, 8), (2100, 7, 5, 4), (130, 33, 31, 4),
                                     (17000, 9, 6, 4)])
def test_fused_fast_loop_move_codes(gpu, oracle, variant, resident, N, W, H, A):
    """The folded loop works on per-cell move codes (what each action does from a
    cell) instead of map lookups and bounds tests: pre-built codes staged in LDS
    (plain kernel - with two lanes per env up to 16,384 envs, one beyond - and the
    LDS wave of the hybrid one) or derived from the class map (table waves of the
    hybrid one), with 4 and 8 actions, on grids whose width is
    no multiple of the 16 cells of a map word, with walls, traps and goals on the
    edges."""
    cls, start = gpu.gen_maps_bernoulli(43, N, N, W, H, 0.2, 0.05)
    cfg = gpu.make_config(N, W, H, n_actions=A, episode_len=37, eps0=0.3, gamma=0.9, seed=23, trap_reward=-0.5)
    S, steps = W * H, 150
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        eng.set_fused_variant(variant)
        eng.set_resident_envs(resident)
        info = eng.fused_kernel_info()
        assert "fast" in info["name"], info
        eng.run_fused(steps)
        q, st = eng.q_get(0, N), eng.get_state()
    Q = np.zeros((N, S, A), np.float32)
    ost = oracle.new_state(cfg, start)
    oracle.run(cfg, cls, None, start, Q, ost, 0, steps)
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(st[k], ost[k]), k
    assert_q_close(q.reshape(N, S, A), Q)
    assert st["episode"].max() >= 1


@pytest.mark.parametrize("variant", [1, 2])
def test_fused_fast_loop_after_set_cell(gpu, oracle, variant):
    """crl_set_cell changes one cell of one map: the move codes of its neighbours
    follow, and the folded loop then agrees with the oracle on the edited maps."""
    N, W, H, steps = 2200, 16, 16, 120
    cls, start = gpu.gen_maps_bernoulli(47, N, N, W, H, 0.1, 0.02)
    cfg = gpu.make_config(N, W, H, episode_len=50, eps0=0.2, gamma=0.95, seed=29)
    cls = cls.reshape(N, W * H).copy()
    edits = [(0, 17, gpu.CELL_WALL), (5, 200, gpu.CELL_GOAL), (2199, 34, gpu.CELL_TRAP), (77, 255, gpu.CELL_FREE),
             (77, 0, gpu.CELL_WALL)]
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        eng.set_fused_variant(variant)
        eng.run_fused(steps)
        for m, c, k in edits:
            if c == start[m]:
                continue
            eng.set_cell(m, c, k)
        eng.run_fused(steps)
        assert "fast" in eng.fused_kernel_info()["name"]
        q, st = eng.q_get(0, N), eng.get_state()
    Q = np.zeros((N, W * H, 4), np.float32)
    ost = oracle.new_state(cfg, start)
    oracle.run(cfg, cls, None, start, Q, ost, 0, steps)
    for m, c, k in edits:
        if c != start[m]:
            cls[m, c] = k
    oracle.run(cfg, cls, None, start, Q, ost, steps, steps)
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(st[k], ost[k]), k
    assert_q_close(q.reshape(N, W * H, 4), Q)


def test_fused_large_map_global_path(gpu, oracle):
    """Maps too large for LDS are read from global memory (config 5 shape: 8
    actions, value-noise walls, per-cell rewards, linear epsilon)."""
    N, W, H = 6, 256, 256
    cls, start, cr = gpu.gen_maps_noise(21, N, W, H, 16, 0.25, 0.05, 10.0)
    cfg = gpu.make_config(N, W, H, n_actions=8, episode_len=64, eps_mode=gpu.EPS_EPISODE_LINEAR, eps0=1.0,
                          eps_end=0.05, eps_span=10, seed=2,
                          reward_flags=gpu.REWARD_CELLS | gpu.REWARD_BASE_CELLS)
    assert (cls == 3).sum(axis=1).tolist() == [W * H // 4] * N
    tr, _ = run_both(gpu, oracle, cfg, cls, start, 1500, cr=cr)
    assert len(np.unique(tr["action"])) == 8


def test_fused_shared_map_per_env_tables(gpu, oracle):
    N, W, H = 200, 20, 20
    cls, start = gpu.gen_maps_bernoulli(4, 1, N, W, H, 0.15)
    cfg = gpu.make_config(N, W, H, map_mode=gpu.MAP_SHARED, episode_len=50, eps0=0.2, seed=8)
    run_both(gpu, oracle, cfg, cls, start, 400)


def test_fused_supplied_exploration_stream(gpu, oracle):
    """'The same supplied exploration random stream': numpy draws replace Philox."""
    N, W, H, T = 128, 8, 8, 150
    cls, start = gpu.gen_maps_bernoulli(9, N, N, W, H, 0.1)
    cfg = gpu.make_config(N, W, H, episode_len=30, eps0=0.25, seed=1)
    rng = np.random.default_rng(0)
    u = rng.random((T, N), dtype=np.float32)
    a = rng.integers(0, 4, (T, N)).astype(np.int32)
    run_both(gpu, oracle, cfg, cls, start, T, stream=(u, a))


@pytest.mark.parametrize("eps_mode", ["step", "episode"])
def test_fused_eps_schedules_and_zero_floor(gpu, oracle, eps_mode):
    N, W, H = 100, 10, 10
    cls, start = gpu.gen_maps_bernoulli(5, N, N, W, H, 0.1)
    kw = (dict(eps_mode=gpu.EPS_STEP_MULT, eps_span=400) if eps_mode == "step"
          else dict(eps_mode=gpu.EPS_EPISODE_MULT, eps_span=50))
    cfg = gpu.make_config(N, W, H, episode_len=25, eps0=1.0, eps_decay=0.99, seed=4,
                          max_mode=gpu.MAX_ZERO_FLOOR, **kw)
    run_both(gpu, oracle, cfg, cls, start, 500)


def test_fused_sticky_done_without_auto_reset(gpu, oracle):
    """auto_reset = 0: done stays set and stepping goes on (src/environment.cu:44-46)."""
    N, W, H = 64, 5, 5
    cls = np.zeros((N, W * H), np.uint8)
    cls[:, W - 1] = 1
    start = np.full(N, (H // 2) * W + W // 2, np.int32)
    cfg = gpu.make_config(N, W, H, auto_reset=0, goal_mode=gpu.GOAL_ON_RESULT, eps0=1.0, seed=6)
    tr, _ = run_both(gpu, oracle, cfg, cls, start, 200)
    d = tr["done"]
    assert d[-1].sum() > 0 and (np.diff(d.astype(int), axis=0) >= 0).all()


@pytest.mark.parametrize("shared", [False, True])
def test_episode_budget_and_return_tracking(gpu, oracle, shared):
    """max_episodes + track_returns (the episode loop and reward lists of
    src/train.py:186-226 kept on the device): fused, decomposed and oracle agree."""
    N, W, H, T, E = 700, 8, 8, 260, 4
    n_maps = 1 if shared else N
    cls, start = gpu.gen_maps_bernoulli(15, n_maps, N, W, H, 0.1, 0.04)
    cfg = gpu.make_config(N, W, H, episode_len=19, eps0=0.35, seed=12, lr=0.002 if shared else 0.1,
                          table_mode=gpu.TABLE_SHARED if shared else gpu.TABLE_PER_ENV,
                          map_mode=gpu.MAP_SHARED if shared else gpu.MAP_PER_ENV, max_episodes=E,
                          track_returns=1)
    n_tables = 1 if shared else N
    Q = np.zeros((n_tables, W * H, 4), np.float32)
    ost, ostats = oracle.new_state(cfg, start), oracle.new_stats(N)
    want = oracle.run(cfg, cls, None, start, Q, ost, 0, T, trace_n=N, stats=ostats)
    assert (ost["episode"] == E).all()
    for mode in ("fused", "chunks", "calls"):
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, start)
            eng.set_trace(N, T)
            if mode == "fused":
                eng.run_fused(T)
            elif mode == "chunks":
                for c in (1, 30, 99, T - 130):
                    eng.run_fused(c)
            else:
                for _ in range(T):
                    eng.select(fetch=False)
                    eng.step()
                    eng.update()
            assert_trace_equal(eng.get_trace(T), want)
            st, stats = eng.get_state(), eng.episode_stats()
            assert_q_close(eng.q_get(0, n_tables).reshape(Q.shape), Q)
        for k in ("s", "ep_step", "episode", "reward", "done", "action"):
            assert np.array_equal(st[k], ost[k]), (mode, k)
        for k in ("last_return", "last_length", "return_sum", "length_sum"):
            assert np.array_equal(stats[k], ostats[k]), (mode, k)
    with gpu.Engine(gpu.make_config(4, 4, 4), 0) as eng:
        with pytest.raises(gpu.CrlError):
            eng.episode_stats()  # not tracked


# ---- the decomposed calls equal the fused kernel --------------------------------

@pytest.mark.parametrize("shared", [False, True])
def test_select_step_update_equals_fused(gpu, oracle, shared):
    N, W, H, T = 333, 9, 9, 60
    n_maps = 1 if shared else N
    cls, start = gpu.gen_maps_bernoulli(12, n_maps, N, W, H, 0.15, 0.05)
    cfg = gpu.make_config(N, W, H, episode_len=13, eps0=0.3, seed=3,
                          table_mode=gpu.TABLE_SHARED if shared else gpu.TABLE_PER_ENV,
                          map_mode=gpu.MAP_SHARED if shared else gpu.MAP_PER_ENV)
    n_tables = 1 if shared else N
    with gpu.Engine(cfg, 0) as a, gpu.Engine(cfg, 0) as b:
        for e in (a, b):
            e.set_maps(cls, start)
            e.set_trace(N, T)
        a.run_fused(T)
        acts = []
        for _ in range(T):
            acts.append(b.select())
            b.step()
            b.update()
        ta, tb = a.get_trace(T), b.get_trace(T)
        assert_trace_equal(tb, ta)
        assert np.array_equal(np.array(acts, np.uint8), ta["action"])
        assert np.array_equal(a.q_get(0, n_tables), b.q_get(0, n_tables))
        sa, sb = a.get_state(), b.get_state()
        for k in sa:
            assert np.array_equal(sa[k], sb[k]), k
        assert a.step_count == b.step_count == T


# ---- shared table: ordered reduction ----------------------------------------------

# variant 1: two launches per step; 2: every step of a call in one launch
@pytest.mark.parametrize("variant", [1, 2])
@pytest.mark.parametrize("N,W,H,steps,lr", [(64, 4, 4, 50, 0.05), (5000, 16, 16, 120, 0.002),
                                            (5000, 16, 16, 120, 0.05),  # overflows: inf/nan parity
                                            (65536, 64, 64, 12, 0.05)])
def test_shared_table_matches_oracle(gpu, oracle, variant, N, W, H, steps, lr):
    cls, start = gpu.gen_maps_bernoulli(2, 1, N, W, H, 0.15)
    cfg = gpu.make_config(N, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=lr,
                          eps0=0.2, episode_len=0, seed=13)
    _, q = run_both(gpu, oracle, cfg, cls, start, steps, trace_n=min(N, 4096), variant=variant)
    if lr < 0.01:
        assert np.isfinite(q).all() and np.count_nonzero(q) > 50


def test_shared_table_one_launch_kernel_shapes(gpu, oracle):
    """The one-launch kernel where its roles do not line up: more owners than blocks
    of envs (workgroups without envs), a last block that is not full, 8 actions
    with per-cell rewards and per-env maps read from global memory, calls that
    alternate (chunked launches)."""
    # 300 envs = 2 of 256 blocks with envs, 1024 keys = 4 to an owner
    cls, start = gpu.gen_maps_bernoulli(5, 1, 300, 16, 16, 0.1, 0.03)
    cfg = gpu.make_config(300, 16, 16, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.01, eps0=0.3,
                          episode_len=25, seed=3, trap_reward=-0.5)
    with gpu.Engine(cfg, 0) as eng:
        assert eng.fused_kernel_info(10)["name"] == "k_shared_persist<4,1,folded>"  # (automatic; the common rules)
        eng.set_fused_variant(1)
        assert eng.fused_kernel_info(10)["name"] == "k_shared_act+k_reduce_owners"
        eng.set_fused_variant(2)
        assert eng.fused_kernel_info(1)["name"] == "k_shared_persist<4,1,folded>" and eng.fused_kernel_info(1)["grid"] == 256
    run_both(gpu, oracle, cfg, cls, start, 90, chunks=[1, 30, 1, 1, 50, 7], variant=2)
    # 8 actions, cell rewards, per-env maps (global memory), linear epsilon, 1000 envs: last block 232 envs
    N, W, H = 1000, 24, 20
    cls, start, cr = gpu.gen_maps_noise(6, N, W, H, 8, 0.2, 0.05, 2.0)
    cfg = gpu.make_config(N, W, H, n_actions=8, table_mode=gpu.TABLE_SHARED, lr=0.004, eps_mode=gpu.EPS_EPISODE_LINEAR,
                          eps0=0.9, eps_end=0.1, eps_span=4, episode_len=40, seed=8,
                          reward_flags=gpu.REWARD_CELLS | gpu.REWARD_BASE_CELLS)
    with gpu.Engine(cfg, 0) as eng:
        eng.set_fused_variant(2)
        assert eng.fused_kernel_info(10)["name"] == "k_shared_persist<8,2>"
    tr, q = run_both(gpu, oracle, cfg, cls, start, 130, cr=cr, chunks=[64, 66], variant=2)
    assert len(np.unique(tr["action"])) == 8 and np.isfinite(q).all()
    # goal test on the resulting cell, sticky done, zero-floored max, supplied stream
    N, W, H = 700, 9, 7
    cls, start = gpu.gen_maps_bernoulli(7, 1, N, W, H, 0.1)
    cfg = gpu.make_config(N, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.01, eps0=0.25,
                          auto_reset=0, goal_mode=gpu.GOAL_ON_RESULT, max_mode=gpu.MAX_ZERO_FLOOR, seed=5)
    rng = np.random.default_rng(1)
    u = rng.random((45, N), dtype=np.float32)  # (the oracle takes a stream that covers the whole run)
    a = rng.integers(0, 4, (45, N)).astype(np.int32)
    run_both(gpu, oracle, cfg, cls, start, 45, stream=(u, a), chunks=[20, 25], variant=2)
    # episode budget and return accumulators
    N, W, H, T, E = 600, 8, 8, 200, 3
    cls, start = gpu.gen_maps_bernoulli(15, 1, N, W, H, 0.1, 0.04)
    cfg = gpu.make_config(N, W, H, episode_len=19, eps0=0.35, seed=12, lr=0.002, table_mode=gpu.TABLE_SHARED,
                          map_mode=gpu.MAP_SHARED, max_episodes=E, track_returns=1)
    Q = np.zeros((1, W * H, 4), np.float32)
    ost, ostats = oracle.new_state(cfg, start), oracle.new_stats(N)
    want = oracle.run(cfg, cls, None, start, Q, ost, 0, T, trace_n=N, stats=ostats)
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        eng.set_trace(N, T)
        eng.set_fused_variant(2)
        eng.run_fused(120)
        eng.run_fused(T - 120)
        assert_trace_equal(eng.get_trace(T), want)
        st, stats = eng.get_state(), eng.episode_stats()
        assert_q_close(eng.q_get(0, 1).reshape(Q.shape), Q)
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(st[k], ost[k]), k
    for k in ("last_return", "last_length", "return_sum", "length_sum"):
        assert np.array_equal(stats[k], ostats[k]), k
    assert (ost["episode"] == E).all()


def test_shared_table_one_launch_kernel_gives_up_cleanly(gpu):
    """Failure handling of the one-launch kernel, forced from the host: with a wait of
    one poll the threads do not find their peers' data, give up, and every workgroup
    leaves the kernel.  A second call before anybody has looked must not hide the first
    one's report (its launch sees the give-up word and returns at once); the next
    synchronising call reports it once, calls that work on state or table are refused
    until they are set again, and the device is fine afterwards."""
    N, W, H = 20000, 32, 32
    cls, start = gpu.gen_maps_bernoulli(6, 1, N, W, H, 0.15)
    cfg = gpu.make_config(N, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.004, eps0=0.2, seed=21)
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        eng.set_fused_variant(2)
        eng.set_persist_spin_limit(1)
        eng.run_fused(50)  # asynchronous: the launch itself succeeds
        eng.run_fused(5)   # and so does this one, on top of what the first left
        with pytest.raises(gpu.CrlError) as err:
            eng.sync()
        assert err.value.code == -2 and "gave up" in str(err.value)
        eng.sync()  # reported once
        for call in (lambda: eng.run_fused(3), eng.get_state, lambda: eng.q_get(0), eng.select):
            with pytest.raises(gpu.CrlError) as err:
                call()
            assert err.value.code == gpu.E_STATE and "gave up earlier" in str(err.value)
        # state and table set again: the engine works, on the default wait
        eng.set_persist_spin_limit(1 << 20)
        eng.reset()
        eng.q_set(0, np.zeros((W * H, 4), np.float32))
        eng.set_state(s=start.copy(), ep_step=np.zeros(N, np.int32), episode=np.zeros(N, np.int32))
        eng.step_count = 0
        eng.run_fused(50)
        q_again = eng.q_get(0)
    with gpu.Engine(cfg, 0) as eng:  # same device, default limit: all is well
        eng.set_maps(cls, start)
        eng.set_fused_variant(2)
        eng.run_fused(50)
        q_one = eng.q_get(0)
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        eng.set_fused_variant(1)
        eng.run_fused(50)
        assert np.array_equal(eng.q_get(0), q_one) and np.isfinite(q_one).all()
    assert np.array_equal(q_again, q_one)


def test_shared_table_automatic_plan_and_cell_sizes(gpu, oracle):
    """What crl_run_fused picks by itself, and tables of every size: through the one-launch
    kernel (always 256 owners: 64 keys each down to none) and through two launches per
    step (hand-off cells of 8 records for 256 owners, 16 for 64, 32 for 32, 64 for 16 and
    fewer)."""
    for N, W, H, auto in ((3000, 64, 64, "persist"), (3000, 32, 32, "persist"), (3000, 32, 16, "persist"),
                          (3000, 16, 16, "persist"), (700, 5, 5, "persist")):
        cls, start = gpu.gen_maps_bernoulli(9, 1, N, W, H, 0.12, 0.03)
        cfg = gpu.make_config(N, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.003, eps0=0.3,
                              episode_len=30, seed=4, trap_reward=-0.5)
        with gpu.Engine(cfg, 0) as eng:
            name = eng.fused_kernel_info(50)["name"]
            assert name == ("k_shared_persist<4,1,folded>" if auto == "persist" else "k_shared_act+k_reduce_owners"), (W, H, name)
            assert eng.fused_kernel_info(1)["name"] == "k_shared_act+k_reduce_owners"  # too short to repay the set-up
        for variant in (1, 2):
            _, q = run_both(gpu, oracle, cfg, cls, start, 40, variant=variant)
            assert np.isfinite(q).all() and np.count_nonzero(q) > 20


@pytest.mark.parametrize("variant", [1, 2])
def test_shared_table_cells_that_overflow(gpu, oracle, variant):
    """More distinct keys for one owner than a hand-off cell has records: every env starts
    (and, with episodes of one step, always acts) on one of the 16 cells that one owner of
    a 32x32x4 table holds, with random actions - 64 keys for cells of 16 records, in every
    block and step - so the owners go back to the blocks' raw samples."""
    N, W, H = 2000, 32, 32
    cells = np.arange(W * H)
    hi = cells >> 6                      # 64 owners of 16 cells each
    owner = (cells + 37 * hi) & 63
    mine = cells[owner == 5]
    assert len(mine) == 16
    rng = np.random.default_rng(3)
    start = rng.choice(mine, N).astype(np.int32)
    cls = np.zeros((1, W * H), np.uint8)
    cfg = gpu.make_config(N, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.01, eps0=1.0,
                          episode_len=1, seed=6)
    _, q = run_both(gpu, oracle, cfg, cls, start, 30, variant=variant)
    touched = np.count_nonzero(q.reshape(W * H, 4)[mine])
    assert touched == 64 and np.count_nonzero(q) == 64


def test_shared_table_all_envs_on_one_cell(gpu, oracle):
    """Degenerate segment: every env hits the same (s,a) keys."""
    N, W, H = 3000, 3, 3
    cls = np.zeros((1, W * H), np.uint8)
    cls[0, 8] = 1
    start = np.zeros(N, np.int32)
    cfg = gpu.make_config(N, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.05,
                          eps0=0.5, episode_len=6, seed=1)
    run_both(gpu, oracle, cfg, cls, start, 40)


def test_shared_table_run_to_run_identity(gpu):
    N, W, H = 20000, 32, 32
    cls, start = gpu.gen_maps_bernoulli(6, 1, N, W, H, 0.15)
    cfg = gpu.make_config(N, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.004,
                          eps0=0.2, seed=21)
    qs = []
    for _ in range(2):
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, start)
            eng.run_fused(100)
            qs.append(eng.q_get(0))
    assert np.isfinite(qs[0]).all() and np.array_equal(qs[0], qs[1])
    assert np.count_nonzero(qs[0]) > 100


# ---- checkpoint / resume -------------------------------------------------------------

@pytest.mark.parametrize("shared", [False, True])
def test_resume_from_saved_state_equals_uninterrupted_run(gpu, shared):
    """(tables, s, ep_step, episode, step count) is a complete resume state (the
    exploration stream is counter-based): a fresh engine loaded with what a first
    one held mid-run (src/q_learning.cu:176-189 get/set_q_table; src/train.py:150-168
    save/load) ends bit-identical to a run that was never interrupted."""
    N, W, H, first, rest = 1500, 12, 12, 333, 412  # an odd split: the Philox block of a step pair is cut
    cls, start = gpu.gen_maps_bernoulli(9, 1 if shared else N, N, W, H, 0.15, 0.0 if shared else 0.03)
    kw = dict(table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.002, eps0=0.2) if shared else \
        dict(eps_mode=gpu.EPS_EPISODE_LINEAR, eps0=0.9, eps_end=0.05, eps_span=6, lr=0.1)
    cfg = gpu.make_config(N, W, H, episode_len=40, seed=17, **kw)
    n_tables = 1 if shared else N
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        eng.run_fused(first + rest)
        want_st, want_q = eng.get_state(), eng.q_get(0, n_tables)
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        eng.run_fused(first)
        saved_st, saved_q, saved_t = eng.get_state(), eng.q_get(0, n_tables).copy(), eng.step_count
    assert saved_t == first
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        for i in range(n_tables):
            eng.q_set(i, saved_q.reshape(n_tables, -1)[i])
        eng.set_state(saved_st["s"], saved_st["ep_step"], saved_st["episode"])
        eng.step_count = saved_t
        eng.run_fused(rest)
        got_st, got_q = eng.get_state(), eng.q_get(0, n_tables)
        assert eng.step_count == first + rest
    assert np.array_equal(got_q, want_q, equal_nan=True) and np.isfinite(want_q).all()
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(got_st[k], want_st[k]), k
    assert np.count_nonzero(want_q) > 100 and want_st["episode"].min() >= 5


# ---- explicit batches (CudaQLearning::update_batch) --------------------------------

@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("n", [1, 10, 1024, 5000])
def test_td_update_batch_matches_oracle(gpu, oracle, mode, n):
    W, H, A = 10, 10, 4
    S = W * H
    cfg = gpu.make_config(1, W, H, max_mode=mode, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED)
    rng = np.random.default_rng(n + mode)
    Q0 = rng.normal(0, 1, (S, A)).astype(np.float32)
    s, a, s2 = rng.integers(0, S, n), rng.integers(0, A, n), rng.integers(0, S, n)
    r = rng.normal(0, 1, n).astype(np.float32)
    done = (rng.random(n) < 0.2).astype(np.uint8)
    with gpu.Engine(cfg, 0) as eng:
        eng.q_set(0, Q0)
        eng.td_update(0, s, a, r, s2, done)
        got = eng.q_get(0)
    want = Q0.copy().reshape(-1)
    oracle.td_update_batch(want, S, A, s, a, r, s2, done, 0.1, 0.99, mode)
    assert_q_close(got.reshape(-1), want)


def _td_case(gpu, oracle, W, H, A, s, a, r, s2, done, mode=0):
    S = W * H
    cfg = gpu.make_config(1, W, H, n_actions=A, max_mode=mode, table_mode=gpu.TABLE_SHARED,
                          map_mode=gpu.MAP_SHARED)
    rng = np.random.default_rng(S)
    Q0 = rng.normal(0, 1, (S, A)).astype(np.float32)
    with gpu.Engine(cfg, 0) as eng:
        eng.q_set(0, Q0)
        eng.td_update(0, s, a, r, s2, done)
        got = eng.q_get(0)
    want = Q0.copy().reshape(-1)
    oracle.td_update_batch(want, S, A, s, a, r, s2, done, 0.1, 0.99, mode)
    assert_q_close(got.reshape(-1), want)


def test_td_update_skips_samples_with_an_action_outside_the_table(gpu, oracle):
    """An action that is no action moves nothing in a step (src/kernels.cu:15-23) and
    has no table entry: such a sample changes nothing, the samples around it keep
    their place in the order of the sums (one block of 256 samples: plain left to
    right, so leaving the skipped samples out altogether gives the same bits)."""
    W, H, A, n = 6, 5, 4, 250
    rng = np.random.default_rng(42)
    s, s2 = rng.integers(0, W * H, n), rng.integers(0, W * H, n)
    a = rng.integers(0, A, n)
    bad = rng.random(n) < 0.3
    a[bad] = rng.choice([-1, A, A + 3, 100, -7], bad.sum())
    r = rng.normal(0, 1, n).astype(np.float32)
    done = (rng.random(n) < 0.2).astype(np.uint8)
    _td_case(gpu, oracle, W, H, A, s, a, r, s2, done)
    # the same table from the valid samples alone
    cfg = gpu.make_config(1, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED)
    Q0 = np.random.default_rng(W * H).normal(0, 1, (W * H, A)).astype(np.float32)
    got = []
    for keep in (np.ones(n, bool), ~bad):
        with gpu.Engine(cfg, 0) as eng:
            eng.q_set(0, Q0)
            eng.td_update(0, s[keep], a[keep], r[keep], s2[keep], done[keep])
            got.append(eng.q_get(0))
    assert np.array_equal(got[0], got[1])


def test_td_update_many_blocks_and_tiles(gpu, oracle):
    """70 000 samples = 274 blocks: more than one 256-block tile and 18 groups;
    deltas of mixed magnitude make a wrong association visible."""
    W, H, A, n = 8, 8, 4, 70000
    rng = np.random.default_rng(5)
    S = W * H
    s, a, s2 = rng.integers(0, S, n), rng.integers(0, A, n), rng.integers(0, S, n)
    r = (rng.normal(0, 1, n) * 10.0 ** rng.integers(-3, 3, n)).astype(np.float32)
    _td_case(gpu, oracle, W, H, A, s, a, r, s2, (rng.random(n) < 0.2).astype(np.uint8))


def test_td_update_slot_overflow_path(gpu, oracle):
    """One block holds 40 distinct keys of the same owner workgroup (more than a
    block can hand over): the owner re-reads that block's samples in order."""
    W, H, A = 64, 64, 4
    owner, mix = 5, 37
    keys = [(h << 8) | ((owner - mix * h) & 255) for h in range(40)]
    rng = np.random.default_rng(9)
    n = 3 * 256
    key = rng.integers(0, W * H * A, n)
    key[256:256 + 200] = rng.choice(keys, 200)  # block 1 overflows owner 5
    s, a = key // A, key % A
    s2 = rng.integers(0, W * H, n)
    r = rng.normal(0, 1, n).astype(np.float32)
    _td_case(gpu, oracle, W, H, A, s, a, r, s2, np.zeros(n, np.uint8))


def test_td_update_large_table_scan_path(gpu, oracle):
    """More than 16384 keys: the scanning fallback, same tree order."""
    W, H, A, n = 80, 80, 8, 9000
    rng = np.random.default_rng(3)
    S = W * H
    hot = rng.integers(0, S, 30)  # few cells: long runs per key across blocks and groups
    s, a, s2 = rng.choice(hot, n), rng.integers(0, A, n), rng.integers(0, S, n)
    r = (rng.normal(0, 1, n) * 10.0 ** rng.integers(-3, 3, n)).astype(np.float32)
    _td_case(gpu, oracle, W, H, A, s, a, r, s2, (rng.random(n) < 0.1).astype(np.uint8), mode=1)


def test_shared_table_large_table_scan_path(gpu, oracle):
    N, W, H = 6000, 72, 72  # 20736 keys > 16384
    cls, start = gpu.gen_maps_bernoulli(8, 1, N, W, H, 0.15)
    cfg = gpu.make_config(N, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.01,
                          eps0=0.2, seed=2)
    run_both(gpu, oracle, cfg, cls, start, 40, trace_n=N)


# ---- step rule, exhaustively, through the engine ------------------------------------

def test_step_rule_brute_force_against_float_grid(gpu, oracle):
    """Every (cell, action) on float grids holding every class and threshold
    edge value: engine step on the classified grid == src/kernels.cu:13-66."""
    from test_oracle_pins import EDGE_VALUES
    W, H = 5, 4
    S = W * H
    vals = np.array(EDGE_VALUES, np.float32)
    rng = np.random.default_rng(3)
    actions = list(range(-1, 6))
    for trial in range(4):
        grid = vals[rng.integers(0, len(vals), S)].astype(np.float32)
        cls, cr = gpu.classify_grid(grid)
        N = S * len(actions)
        cfg = gpu.make_config(N, W, H, map_mode=gpu.MAP_SHARED, auto_reset=0, reward_flags=gpu.REWARD_CELLS)
        start = np.repeat(np.arange(S, dtype=np.int32), len(actions))
        act = np.tile(np.array(actions, np.int32), S)
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, start, cr)
            eng.step(act)
            st = eng.get_state()
        for i in range(N):
            x, y, r, d = oracle.step_e2(grid, W, H, int(start[i]) % W, int(start[i]) // W, 0, int(act[i]))
            assert (st["s"][i], st["reward"][i], st["done"][i]) == (y * W + x, np.float32(r), d), (trial, i)


def test_step_rule_hand_worked_cell_rewards(gpu):
    """The hand-worked cases of tests/test_oracle_pins.py (per-cell base rewards, diagonals
    with cell rewards, both goal modes) through crl_step: literal expectations, no oracle."""
    from test_oracle_pins import HAND_CASES, HAND_MAP
    m = HAND_MAP
    cls, cr = np.array(m["cls"], np.uint8), np.array(m["cr"], np.float32)
    groups = {}
    for flags, goal_mode, s, a, want in HAND_CASES:
        groups.setdefault((flags, goal_mode), []).append((s, a, want))
    for (flags, goal_mode), cases in groups.items():
        cfg = gpu.make_config(len(cases), m["W"], m["H"], n_actions=8, map_mode=gpu.MAP_SHARED,
                              reward_flags=flags, goal_mode=goal_mode, auto_reset=0, trap_reward=-0.75)
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, np.array([c[0] for c in cases], np.int32), cr if flags else None)
            eng.step(np.array([c[1] for c in cases], np.int32))
            st = eng.get_state()
        for i, (s, a, want) in enumerate(cases):
            got = (int(st["s"][i]), st["reward"][i], int(st["done"][i]))
            assert got == (want[0], np.float32(want[1]), want[2]), (flags, goal_mode, s, a, got)


def test_full_size_config4(gpu, oracle):
    """The whole 1,048,576-env / 4 GB configuration for its 1000 steps: EVERY env's
    state and EVERY table bit-exact against the oracle (which of the two kinds of
    workers steps an env is settled at run time, so slices would not pin both), the
    tables fetched and compared in chunks to keep host memory bounded; plus properties
    that do not need the oracle."""
    from conftest import oracle_run_threads
    N, W, H, steps = 1 << 20, 16, 16, 1000
    cls, start = gpu.gen_maps_bernoulli(0, N, N, W, H, 0.1, 0.02)
    cfg = gpu.make_config(N, W, H, episode_len=128, eps0=0.1, gamma=0.95, seed=0, trap_reward=-1.0)
    Q, ost = oracle_run_threads(oracle, cfg, cls, start, 0, steps)
    chunk, bad_tables = 1 << 16, 0
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        eng.run_fused(steps)
        st = eng.get_state()
        hbm, lds = eng.fused_split()
        info = eng.fused_kernel_info()
        for lo in range(0, N, chunk):
            q = eng.q_get(lo, chunk).reshape(chunk, W * H, 4)
            same = (q == Q[lo:lo + chunk]).all(axis=(1, 2))
            bad_tables += int(chunk - np.count_nonzero(same))
    assert "fast,hbm+lds" in info["name"] and hbm + lds == N and hbm > 0 and lds > 0
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(st[k], ost[k]), (k, int(np.count_nonzero(st[k] != ost[k])))
    assert bad_tables == 0
    assert np.count_nonzero(Q) > N * 50
    here = cls[np.arange(N), st["s"]]
    assert (here < 2).all()
    assert set(np.unique(st["reward"]).tolist()) <= {np.float32(-0.01), np.float32(1.0), np.float32(-1.0)}
    assert (st["ep_step"] < 128).all() and st["episode"].min() >= steps // 128


def config5(gpu, n, seed=0):
    return gpu.make_config(n, 256, 256, n_actions=8, episode_len=1024, lr=0.1, gamma=0.99,
                           eps_mode=gpu.EPS_EPISODE_LINEAR, eps0=1.0, eps_end=0.05, eps_span=100, seed=seed,
                           reward_flags=gpu.REWARD_CELLS | gpu.REWARD_BASE_CELLS)


def test_config5_shape_untraced_pairs_kernel(gpu, oracle):
    """Config 5 at its own shape - 256x256 value-noise maps, 8 actions, per-cell
    rewards, T = 1024, epsilon 1.0 -> 0.05 over 100 episodes - for a few hundred
    envs and more than two episodes, untraced, so that the kernel the benchmark
    times runs (folded loop, two lanes per env, move codes from global memory):
    every table and all state bit-exact against the oracle."""
    N, steps = 320, 2 * 1024 + 77
    cls, start, cr = gpu.gen_maps_noise(0, N, 256, 256, 16, 0.25, 0.05, 10.0)
    cfg = config5(gpu, N)
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start, cr)
        assert eng.fused_kernel_info(steps)["name"] == "k_fused_per_env<8,2,fast,pairs>"
        eng.run_fused(1024)  # in two launches: the second starts mid-way with trained tables
        eng.run_fused(steps - 1024)
        st, q = eng.get_state(), eng.q_get(0, N)
    Q = np.zeros((N, 256 * 256, 8), np.float32)
    ost = oracle.new_state(cfg, start)
    oracle.run(cfg, cls, cr, start, Q, ost, 0, steps)
    assert_q_close(q.reshape(Q.shape), Q)
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(st[k], ost[k]), k
    assert st["episode"].min() >= 2 and np.count_nonzero(Q) > N * 1000


def test_full_size_config5(gpu, oracle):
    """The whole 8192-env / 16 GB configuration for two episodes and a bit: EVERY
    env's state bit-exact against the oracle, every table of sixteen 128-env chunks
    spread over the batch (4 GB of the 16), and size-independent properties over all envs."""
    from conftest import oracle_run_threads
    N, W, H, steps = 8192, 256, 256, 2 * 1024 + 100
    S = W * H
    cls, start, cr = gpu.gen_maps_noise(0, N, W, H, 16, 0.25, 0.05, 10.0)
    cfg = config5(gpu, N)
    Q, ost = oracle_run_threads(oracle, cfg, cls, start, 0, steps, cr=cr)
    chunk, bad_tables = 128, 0
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start, cr)
        info = eng.fused_kernel_info(steps)
        eng.run_fused(steps)
        st = eng.get_state()
        for lo in list(range(0, N, 4 * chunk)) + [N - chunk]:
            q = eng.q_get(lo, chunk).reshape(chunk, S, 8)
            same = (q == Q[lo:lo + chunk]).all(axis=(1, 2))
            bad_tables += int(chunk - np.count_nonzero(same))
    assert info["name"] == "k_fused_per_env<8,2,fast,pairs>"
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(st[k], ost[k]), (k, int(np.count_nonzero(st[k] != ost[k])))
    assert bad_tables == 0
    del Q
    env = np.arange(N)
    assert (cls[env, st["s"]] < 2).all()                      # nobody stands in a wall
    assert (st["ep_step"] < 1024).all() and (st["episode"] >= 2).all() and (st["action"] < 8).all()
    assert np.isfinite(st["reward"]).all() and np.abs(st["reward"]).max() < 10.5
    # an env that has not just restarted got the reward of the cell it stands on
    # (per-cell base rewards; there are no traps in these maps)
    moved_on = st["ep_step"] > 0
    assert np.array_equal(st["reward"][moved_on], cr[env, st["s"]][moved_on])
    assert ((st["done"] == 1) <= (st["ep_step"] == 0)).all()  # reaching the goal restarts the env


def test_large_batches_of_large_per_env_maps(gpu, oracle):
    """Per-env maps so large that only one or two 64-env waves' worth fit the LDS of
    a workgroup (the planner has to give up waves, and the plain ticket kernels
    need more than the default 64 KB): 65,536+ envs, two slices against the oracle."""
    from conftest import oracle_run_slice
    for N, W, H, steps in ((65536, 64, 64, 8), (66000, 40, 40, 150), (65536, 48, 48, 70)):
        cls, start = gpu.gen_maps_bernoulli(4, N, N, W, H, 0.15, 0.02)
        cfg = gpu.make_config(N, W, H, episode_len=64, eps0=0.15, seed=4)
        with gpu.Engine(cfg, 0) as eng:
            eng.set_maps(cls, start)
            info = eng.fused_kernel_info(steps)
            assert info["lds_bytes"] <= 160 * 1024
            eng.run_fused(steps)
            st = eng.get_state()
            slices = [(0, 256), (N - 300, N)]
            qs = [eng.q_get(lo, hi - lo) for lo, hi in slices]
        for (lo, hi), q in zip(slices, qs):
            Q, ost = oracle_run_slice(oracle, cfg, lo, hi, cls[lo:hi], start[lo:hi], 0, steps)
            assert_q_close(q.reshape(Q.shape), Q)
            for k in ("s", "ep_step", "episode", "reward", "done", "action"):
                assert np.array_equal(st[k][lo:hi], ost[k]), (N, W, lo, k, info)
        assert (cls[np.arange(N), st["s"]] < 2).all()


def test_full_size_config3_into_the_overflow_regime(gpu, oracle):
    """65,536 envs on the shared 64x64 table with the configuration's own lr = 0.05
    for 150 steps: the table overflows on the way (inf / NaN), and every
    trajectory of the first 4096 envs, the final state of all envs and the table -
    NaN placement included - equal the oracle's."""
    N, W, H, steps = 65536, 64, 64, 150
    cls, start = gpu.gen_maps_bernoulli(0, 1, N, W, H, 0.15)
    cfg = gpu.make_config(N, W, H, table_mode=gpu.TABLE_SHARED, map_mode=gpu.MAP_SHARED, lr=0.05,
                          gamma=0.99, eps0=0.2, seed=0)
    _, q = run_both(gpu, oracle, cfg, cls, start, steps, trace_n=4096)
    assert not np.isfinite(q).all()


@pytest.mark.parametrize("fixture", ["baseline", "reference"])
def test_full_size_config1(gpu, oracle, fixture):
    """Config 1, whole program: one 10x10 grid without walls, 1000 episodes of at
    most 500 steps, eps 1.0 decaying x0.995.  Two fixtures: the benchmark's wording
    (start (0,0), goal (9,9), decay per episode) and the reference's default world
    (start (5,5), goal (9,0): src/environment.cu:9-10,146; decay per update:
    src/train.py:140-141).  Every step of every episode is compared."""
    W = H = 10
    E, T = 1000, 500
    cls = np.zeros(W * H, np.uint8)
    if fixture == "baseline":
        start, goal = [0], 9 * W + 9
        sched = dict(eps_mode=gpu.EPS_EPISODE_MULT, eps_span=E + 1)
    else:
        start, goal = [(H // 2) * W + W // 2], W - 1
        sched = dict(eps_mode=gpu.EPS_STEP_MULT, eps_span=E * T + 1)
    cls[goal] = gpu.CELL_GOAL
    cfg = gpu.make_config(1, W, H, map_mode=gpu.MAP_SHARED, episode_len=T, lr=0.1, gamma=0.99, eps0=1.0,
                          eps_decay=0.995, max_episodes=E, seed=0, **sched)
    tr, q = run_both(gpu, oracle, cfg, cls, start, E * T)
    ends = int(tr["done"].sum())
    assert ends > E // 2  # most episodes reach the goal once the table has learnt the way
    assert float(q.max()) > 0.9


def test_full_size_config2(gpu, oracle):
    """4096 envs, 32x32, 256-step episodes, all 10,000 steps: final tables and
    state bit-exact against the oracle."""
    N, W, H, steps = 4096, 32, 32, 10000
    cls, start = gpu.gen_maps_bernoulli(0, N, N, W, H, 0.2)
    cfg = gpu.make_config(N, W, H, episode_len=256, lr=0.1, gamma=0.99, eps0=0.1, seed=0)
    with gpu.Engine(cfg, 0) as eng:
        eng.set_maps(cls, start)
        eng.run_fused(steps)
        st, q = eng.get_state(), eng.q_get(0, N)
    Q = np.zeros((N, W * H, 4), np.float32)
    ost = oracle.new_state(cfg, start)
    import ctypes as C
    import threading
    p = oracle._p
    def work(lo, hi):
        assert oracle.lib.orc_run_range(C.byref(cfg), lo, hi, p(cls), None, p(start), p(Q), p(ost["s"]),
                                        p(ost["ep_step"]), p(ost["episode"]), p(ost["reward"]),
                                        p(ost["done"]), p(ost["action"]), 0, steps) == 0
    ths = [threading.Thread(target=work, args=(N * i // 8, N * (i + 1) // 8)) for i in range(8)]
    [t.start() for t in ths]
    [t.join() for t in ths]
    assert_q_close(q.reshape(Q.shape), Q)
    for k in ("s", "ep_step", "episode", "reward", "done", "action"):
        assert np.array_equal(st[k], ost[k]), k
    assert st["episode"].min() >= steps // 256
