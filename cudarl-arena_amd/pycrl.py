"""ctypes view of the engine's C ABI (include/crl.h).

Thin plumbing for tests, the benchmark and Python callers: every method maps to
one C entry point and raises `CrlError` on a non-zero status.  Nothing here
computes; if the HIP library is not built, `load()` raises."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libcrl.so")

CELL_FREE, CELL_GOAL, CELL_TRAP, CELL_WALL = 0, 1, 2, 3
TABLE_PER_ENV, TABLE_SHARED = 0, 1
MAP_PER_ENV, MAP_SHARED = 0, 1
MAX_TRUE, MAX_ZERO_FLOOR = 0, 1
GOAL_ON_TARGET, GOAL_ON_RESULT = 0, 1
EPS_FIXED, EPS_STEP_MULT, EPS_EPISODE_MULT, EPS_EPISODE_LINEAR = 0, 1, 2, 3
REWARD_CELLS, REWARD_BASE_CELLS = 1, 2


class Config(C.Structure):
    """crl_config (and, field for field, the oracle's orc_config)."""

    _fields_ = [
        ("struct_size", C.c_uint32),
        ("n_envs", C.c_int32),
        ("width", C.c_int32),
        ("height", C.c_int32),
        ("n_actions", C.c_int32),
        ("table_mode", C.c_int32),
        ("map_mode", C.c_int32),
        ("max_mode", C.c_int32),
        ("goal_mode", C.c_int32),
        ("auto_reset", C.c_int32),
        ("episode_len", C.c_int32),
        ("lr", C.c_float),
        ("gamma", C.c_float),
        ("step_reward", C.c_float),
        ("goal_reward", C.c_float),
        ("trap_reward", C.c_float),
        ("reward_flags", C.c_int32),
        ("eps_mode", C.c_int32),
        ("eps0", C.c_float),
        ("eps_decay", C.c_float),
        ("eps_end", C.c_float),
        ("eps_span", C.c_int32),
        ("max_episodes", C.c_int32),
        ("track_returns", C.c_int32),
        ("seed", C.c_uint64),
    ]


def make_config(n_envs, width, height, n_actions=4, table_mode=TABLE_PER_ENV, map_mode=MAP_PER_ENV,
                max_mode=MAX_TRUE, goal_mode=GOAL_ON_TARGET, auto_reset=1, episode_len=0, lr=0.1,
                gamma=0.99, step_reward=-0.01, goal_reward=1.0, trap_reward=-1.0, reward_flags=0,
                eps_mode=EPS_FIXED, eps0=0.1, eps_decay=1.0, eps_end=0.0, eps_span=1, seed=0,
                max_episodes=0, track_returns=0):
    c = Config()
    c.struct_size = C.sizeof(Config)
    c.n_envs, c.width, c.height, c.n_actions = n_envs, width, height, n_actions
    c.table_mode, c.map_mode, c.max_mode, c.goal_mode = table_mode, map_mode, max_mode, goal_mode
    c.auto_reset, c.episode_len = auto_reset, episode_len
    c.lr, c.gamma = lr, gamma
    c.step_reward, c.goal_reward, c.trap_reward = step_reward, goal_reward, trap_reward
    c.reward_flags, c.eps_mode = reward_flags, eps_mode
    c.eps0, c.eps_decay, c.eps_end, c.eps_span = eps0, eps_decay, eps_end, eps_span
    c.max_episodes, c.track_returns = max_episodes, track_returns
    c.seed = seed
    return c


E_ARG, E_DEVICE, E_ALLOC, E_STATE, E_RANGE = -1, -2, -3, -4, -5  # include/crl.h


class CrlError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("crl status %d: %s" % (code, text))
        self.code = code


_lib = None

# every symbol include/crl.h declares
EXPORTS = [
    "crl_last_error", "crl_version", "crl_device_count", "crl_create", "crl_destroy",
    "crl_set_stream", "crl_sync", "crl_set_resident_envs", "crl_set_fused_variant", "crl_get_fused_split", "crl_set_maps", "crl_set_cell", "crl_classify_grid", "crl_reset",
    "crl_step", "crl_select", "crl_update", "crl_td_update", "crl_run_fused", "crl_run_fused_noalloc", "crl_get_state",
    "crl_set_state", "crl_get_episode_stats", "crl_get_step_count", "crl_set_step_count", "crl_q_get", "crl_q_set",
    "crl_q_get_range", "crl_set_trace", "crl_get_trace", "crl_set_exploration_stream", "crl_set_persist_spin_limit",
    "crl_device_ptr", "crl_fused_kernel_info", "crl_fused_plan_for_config", "crl_philox4x32_10", "crl_explore_draw",
    "crl_eps_table", "crl_gen_maps_bernoulli", "crl_gen_maps_noise", "crl_probe_copy", "crl_probe_barrier", "crl_get_persist_clocks", "crl_set_persist_clocks",
]


def load():
    """Load libcrl.so; raises OSError with a build hint if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise OSError("%s not found: build it with `python -c 'import __graft_entry__ as g; g.build()'`"
                      % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    lib.crl_last_error.restype = C.c_char_p
    lib.crl_version.restype = C.c_char_p
    vp, i32, u64, f32 = C.c_void_p, C.c_int32, C.c_uint64, C.c_float
    lib.crl_create.argtypes = [C.POINTER(Config), C.c_int, C.POINTER(vp)]
    lib.crl_destroy.argtypes = [vp]
    lib.crl_set_stream.argtypes = [vp, vp]
    lib.crl_sync.argtypes = [vp]
    lib.crl_set_resident_envs.argtypes = [vp, i32]
    lib.crl_set_fused_variant.argtypes = [vp, i32]
    lib.crl_get_fused_split.argtypes = [vp, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
    lib.crl_set_maps.argtypes = [vp, vp, vp, vp]
    lib.crl_set_cell.argtypes = [vp, i32, i32, i32, f32]
    lib.crl_classify_grid.argtypes = [vp, C.c_size_t, f32, vp, vp]
    lib.crl_reset.argtypes = [vp, i32, i32]
    lib.crl_step.argtypes = [vp, vp]
    lib.crl_select.argtypes = [vp, vp]
    lib.crl_update.argtypes = [vp]
    lib.crl_td_update.argtypes = [vp, i32, i32, vp, vp, vp, vp, vp]
    lib.crl_run_fused.argtypes = [vp, i32]
    lib.crl_run_fused_noalloc.argtypes = [vp, i32]
    lib.crl_get_state.argtypes = [vp, vp, vp, vp, vp, vp, vp]
    lib.crl_set_state.argtypes = [vp, vp, vp, vp]
    lib.crl_get_episode_stats.argtypes = [vp, vp, vp, vp, vp]
    lib.crl_get_step_count.argtypes = [vp, C.POINTER(u64)]
    lib.crl_set_step_count.argtypes = [vp, u64]
    lib.crl_q_get.argtypes = [vp, i32, vp]
    lib.crl_q_set.argtypes = [vp, i32, vp]
    lib.crl_q_get_range.argtypes = [vp, i32, i32, vp]
    lib.crl_set_trace.argtypes = [vp, i32, i32]
    lib.crl_get_trace.argtypes = [vp, i32, vp, vp, vp, vp]
    lib.crl_set_exploration_stream.argtypes = [vp, i32, vp, vp]
    lib.crl_set_persist_spin_limit.argtypes = [vp, i32]
    lib.crl_device_ptr.argtypes = [vp, i32, C.POINTER(vp)]
    lib.crl_fused_kernel_info.argtypes = [vp, i32, C.c_char_p, C.c_size_t, C.POINTER(i32), C.POINTER(i32),
                                          C.POINTER(i32)]
    lib.crl_fused_plan_for_config.argtypes = [C.POINTER(Config), i32, C.c_char_p, C.c_size_t, C.POINTER(i32),
                                              C.POINTER(i32), C.POINTER(i32)]
    lib.crl_philox4x32_10.argtypes = [vp, vp, vp]
    lib.crl_philox4x32_10.restype = None
    lib.crl_explore_draw.argtypes = [u64, C.c_uint32, u64, i32, C.POINTER(f32), C.POINTER(i32)]
    lib.crl_explore_draw.restype = None
    lib.crl_eps_table.argtypes = [C.POINTER(Config), vp, i32, C.POINTER(i32)]
    lib.crl_gen_maps_bernoulli.argtypes = [u64, i32, i32, i32, i32, f32, f32, vp, vp]
    lib.crl_gen_maps_noise.argtypes = [u64, i32, i32, i32, i32, f32, f32, f32, vp, vp, vp]
    lib.crl_probe_copy.argtypes = [C.c_size_t, C.c_int]
    lib.crl_probe_barrier.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double)]
    lib.crl_get_persist_clocks.argtypes = [vp, vp, C.c_size_t]
    lib.crl_set_persist_clocks.argtypes = [vp, C.c_int32]
    _lib = lib
    return lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _check(rc):
    if rc != 0:
        raise CrlError(rc, load().crl_last_error().decode())


def _arr(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def gen_maps_bernoulli(seed, n_maps, n_envs, width, height, p_wall, p_trap=0.0):
    cls = np.empty((n_maps, width * height), np.uint8)
    start = np.empty(n_envs, np.int32)
    _check(load().crl_gen_maps_bernoulli(seed, n_maps, n_envs, width, height, p_wall, p_trap,
                                         _ptr(cls), _ptr(start)))
    return cls, start


def gen_maps_noise(seed, n_maps, width, height, pitch=16, wall_frac=0.25, sigma=0.05, goal_bonus=10.0):
    cls = np.empty((n_maps, width * height), np.uint8)
    start = np.empty(n_maps, np.int32)
    cr = np.empty((n_maps, width * height), np.float32)
    _check(load().crl_gen_maps_noise(seed, n_maps, width, height, pitch, wall_frac, sigma, goal_bonus,
                                     _ptr(cls), _ptr(start), _ptr(cr)))
    return cls, start, cr


def eps_table(cfg):
    n = C.c_int32(0)
    _check(load().crl_eps_table(C.byref(cfg), None, 0, C.byref(n)))
    out = np.empty(n.value, np.float32)
    _check(load().crl_eps_table(C.byref(cfg), _ptr(out), n.value, C.byref(n)))
    return out


def fused_plan_for_config(cfg, n_steps=0):
    """Launch plan of crl_run_fused(n_steps) for an engine made from cfg (host only)."""
    name = C.create_string_buffer(128)
    g, b, l = C.c_int32(), C.c_int32(), C.c_int32()
    _check(load().crl_fused_plan_for_config(C.byref(cfg), n_steps, name, 128, C.byref(g), C.byref(b), C.byref(l)))
    return dict(name=name.value.decode(), grid=g.value, block=b.value, lds_bytes=l.value)


def probe_barrier(pattern, n_groups=256, rounds=2000):
    ns = C.c_double()
    _check(load().crl_probe_barrier(pattern, n_groups, rounds, C.byref(ns)))
    return ns.value


def classify_grid(grid, step_reward=-0.01):
    g = _arr(grid, np.float32).ravel()
    cls = np.empty(g.size, np.uint8)
    rew = np.empty(g.size, np.float32)
    _check(load().crl_classify_grid(_ptr(g), g.size, step_reward, _ptr(cls), _ptr(rew)))
    return cls, rew


class Engine:
    """One crl_engine on one device."""

    def __init__(self, cfg, device=0):
        self.lib = load()
        self.cfg = cfg
        self.N, self.A = cfg.n_envs, cfg.n_actions
        self.S = cfg.width * cfg.height
        self.n_tables = 1 if cfg.table_mode == TABLE_SHARED else cfg.n_envs
        h = C.c_void_p()
        _check(self.lib.crl_create(C.byref(cfg), device, C.byref(h)))
        self.h = h

    def close(self):
        if self.h:
            self.lib.crl_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def set_maps(self, cell_class, start=None, cell_reward=None):
        cls = _arr(cell_class, np.uint8)
        st = _arr(start, np.int32)
        cr = _arr(cell_reward, np.float32)
        n_maps = 1 if self.cfg.map_mode == MAP_SHARED else self.N
        if cls.size != n_maps * self.S:
            raise ValueError("cell_class has %d entries, expected %d" % (cls.size, n_maps * self.S))
        if st is not None and st.size != self.N:
            raise ValueError("start has %d entries, expected %d" % (st.size, self.N))
        if cr is not None and cr.size != cls.size:
            raise ValueError("cell_reward size mismatch")
        _check(self.lib.crl_set_maps(self.h, _ptr(cls), _ptr(st), _ptr(cr)))

    def set_cell(self, map_index, cell, cell_class, cell_reward=0.0):
        _check(self.lib.crl_set_cell(self.h, map_index, cell, cell_class, cell_reward))

    def reset(self, first=0, count=None):
        _check(self.lib.crl_reset(self.h, first, self.N - first if count is None else count))

    def step(self, actions=None):
        a = _arr(actions, np.int32)
        if a is not None and a.size != self.N:
            raise ValueError("actions has %d entries, expected %d" % (a.size, self.N))
        _check(self.lib.crl_step(self.h, _ptr(a)))

    def select(self, fetch=True):
        out = np.empty(self.N, np.int32) if fetch else None
        _check(self.lib.crl_select(self.h, _ptr(out)))
        return out

    def update(self):
        _check(self.lib.crl_update(self.h))

    def td_update(self, table, s, a, r, s_next, done):
        s, a = _arr(s, np.int32), _arr(a, np.int32)
        r, s2, d = _arr(r, np.float32), _arr(s_next, np.int32), _arr(done, np.uint8)
        n = s.size
        if not (a.size == r.size == s2.size == d.size == n):
            raise ValueError("Inconsistent batch sizes")
        _check(self.lib.crl_td_update(self.h, table, n, _ptr(s), _ptr(a), _ptr(r), _ptr(s2), _ptr(d)))

    def run_fused(self, n_steps):
        _check(self.lib.crl_run_fused(self.h, n_steps))

    def run_fused_noalloc(self, n_steps):
        _check(self.lib.crl_run_fused_noalloc(self.h, n_steps))

    def set_resident_envs(self, n):
        _check(self.lib.crl_set_resident_envs(self.h, n))

    def set_fused_variant(self, v):
        _check(self.lib.crl_set_fused_variant(self.h, v))

    def fused_split(self):
        a, b = C.c_uint32(), C.c_uint32()
        _check(self.lib.crl_get_fused_split(self.h, C.byref(a), C.byref(b)))
        return a.value, b.value

    def sync(self):
        _check(self.lib.crl_sync(self.h))

    def get_state(self):
        N = self.N
        out = dict(s=np.empty(N, np.int32), reward=np.empty(N, np.float32), done=np.empty(N, np.uint8),
                   action=np.empty(N, np.uint8), ep_step=np.empty(N, np.int32),
                   episode=np.empty(N, np.int32))
        _check(self.lib.crl_get_state(self.h, _ptr(out["s"]), _ptr(out["reward"]), _ptr(out["done"]),
                                      _ptr(out["action"]), _ptr(out["ep_step"]), _ptr(out["episode"])))
        return out

    def episode_stats(self):
        N = self.N
        out = dict(last_return=np.empty(N, np.float32), last_length=np.empty(N, np.int32),
                   return_sum=np.empty(N, np.float32), length_sum=np.empty(N, np.int32))
        _check(self.lib.crl_get_episode_stats(self.h, _ptr(out["last_return"]), _ptr(out["last_length"]),
                                              _ptr(out["return_sum"]), _ptr(out["length_sum"])))
        return out

    def set_state(self, s=None, ep_step=None, episode=None):
        _check(self.lib.crl_set_state(self.h, _ptr(_arr(s, np.int32)), _ptr(_arr(ep_step, np.int32)),
                                      _ptr(_arr(episode, np.int32))))

    @property
    def step_count(self):
        t = C.c_uint64(0)
        _check(self.lib.crl_get_step_count(self.h, C.byref(t)))
        return t.value

    @step_count.setter
    def step_count(self, t):
        _check(self.lib.crl_set_step_count(self.h, t))

    def q_get(self, table=0, count=1):
        out = np.empty((count, self.S, self.A), np.float32)
        _check(self.lib.crl_q_get_range(self.h, table, count, _ptr(out)))
        return out[0] if count == 1 else out

    def q_set(self, table, q):
        q = _arr(q, np.float32)
        if q.size != self.S * self.A:
            raise ValueError("Invalid Q-table size")
        _check(self.lib.crl_q_set(self.h, table, _ptr(q)))

    def set_trace(self, n_envs, max_steps):
        self._trace_n = n_envs
        _check(self.lib.crl_set_trace(self.h, n_envs, max_steps))

    def get_trace(self, n_steps):
        n = self._trace_n
        out = dict(s_next=np.empty((n_steps, n), np.int32), action=np.empty((n_steps, n), np.uint8),
                   reward=np.empty((n_steps, n), np.float32), done=np.empty((n_steps, n), np.uint8))
        _check(self.lib.crl_get_trace(self.h, n_steps, _ptr(out["s_next"]), _ptr(out["action"]),
                                      _ptr(out["reward"]), _ptr(out["done"])))
        return out

    def set_exploration_stream(self, u, a_rand):
        if u is None:
            _check(self.lib.crl_set_exploration_stream(self.h, 0, None, None))
            return
        u, a = _arr(u, np.float32), _arr(a_rand, np.int32)
        n_steps = u.shape[0]
        if u.size != n_steps * self.N or a.size != u.size:
            raise ValueError("stream arrays must be [n_steps][n_envs]")
        _check(self.lib.crl_set_exploration_stream(self.h, n_steps, _ptr(u), _ptr(a)))

    def device_ptr(self, which):
        p = C.c_void_p()
        _check(self.lib.crl_device_ptr(self.h, which, C.byref(p)))
        return p.value

    def set_persist_spin_limit(self, polls):
        _check(self.lib.crl_set_persist_spin_limit(self.h, polls))

    def set_persist_clocks(self, on):
        _check(self.lib.crl_set_persist_clocks(self.h, 1 if on else 0))

    def persist_clocks(self):
        """Per-phase shader clocks of the last one-launch shared-table launch that ran with the
        clocks armed: (first, last workgroup) x 8."""
        out = np.zeros(20 + 8 * 256, np.uint64)
        _check(self.lib.crl_get_persist_clocks(self.h, _ptr(out), out.size))
        self.persist_stamps = out[20:].reshape(256, 8)  # 100 MHz wall clock of every workgroup at the marks of the middle step
        return out[:20].reshape(2, 10)

    def fused_kernel_info(self, n_steps=0):
        """Plan of crl_run_fused(n_steps); 0 = a long launch."""
        name = C.create_string_buffer(128)
        g, b, l = C.c_int32(), C.c_int32(), C.c_int32()
        _check(self.lib.crl_fused_kernel_info(self.h, n_steps, name, 128, C.byref(g), C.byref(b), C.byref(l)))
        return dict(name=name.value.decode(), grid=g.value, block=b.value, lds_bytes=l.value)
