"""Shared fixtures: the engine's ctypes view, the CPU oracle, and a GPU probe."""
import ctypes as C
import importlib.util
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "cudarl-arena_amd")
ORACLE_DIR = os.path.join(ROOT, "oracle")
# (CRL_ORACLE_SO: another build of the same source, e.g. the sanitized one of `make -C oracle asan`)
ORACLE_SO = os.environ.get("CRL_ORACLE_SO") or os.path.join(ORACLE_DIR, "libcrl_oracle.so")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _load_module(name, path):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def pycrl():
    return sys.modules.get("pycrl") or _load_module("pycrl", os.path.join(PKG, "pycrl.py"))


class Oracle:
    """ctypes view of oracle/libcrl_oracle.so (the checker, never the product)."""

    def __init__(self, lib):
        self.lib = lib
        vp, i32, f32, u64 = C.c_void_p, C.c_int32, C.c_float, C.c_uint64
        lib.orc_philox4x32_10.argtypes = [vp, vp, vp]
        lib.orc_philox4x32_10.restype = None
        lib.orc_explore_draw.argtypes = [u64, C.c_uint32, u64, i32, C.POINTER(f32), C.POINTER(i32)]
        lib.orc_explore_draw.restype = None
        ip = C.POINTER(C.c_int)
        lib.orc_reset_xy.argtypes = [C.c_int, C.c_int, ip, ip, C.POINTER(f32), ip]
        lib.orc_reset_xy.restype = None
        lib.orc_step_e1.argtypes = [C.c_int, C.c_int, ip, ip, C.POINTER(f32), ip, C.c_int]
        lib.orc_step_e1.restype = None
        lib.orc_step_e2.argtypes = [vp, C.c_int, C.c_int, ip, ip, C.POINTER(f32), ip, C.c_int]
        lib.orc_step_e2.restype = None
        lib.orc_classify.argtypes = [f32]
        lib.orc_classify.restype = C.c_uint8
        lib.orc_step_cls.argtypes = [vp, vp, vp, C.POINTER(i32), C.c_int, C.POINTER(f32)]
        lib.orc_argmax.argtypes = [vp, C.c_int]
        lib.orc_select.argtypes = [vp, C.c_int, f32, f32, C.c_int]
        lib.orc_next_max.argtypes = [vp, C.c_int, C.c_int, C.c_int]
        lib.orc_next_max.restype = f32
        lib.orc_td_value.argtypes = [f32] * 5
        lib.orc_td_value.restype = f32
        lib.orc_td_delta.argtypes = [f32] * 5
        lib.orc_td_delta.restype = f32
        lib.orc_td_update_one.argtypes = [vp, C.c_int, C.c_int, C.c_int, f32, C.c_int, C.c_int, f32, f32,
                                          C.c_int]
        lib.orc_td_update_one.restype = None
        lib.orc_td_update_batch.argtypes = [vp, C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp, f32, f32,
                                            C.c_int]
        lib.orc_tree_sum.argtypes = [vp, vp, C.c_int, C.c_int, vp]
        lib.orc_tree_sum_bruteforce.argtypes = [vp, vp, C.c_int, C.c_int, vp]
        lib.orc_eps_table.argtypes = [vp, vp, C.c_int]
        lib.orc_run.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, u64, i32, vp, vp, i32, vp, vp,
                                vp, vp, vp, vp, vp, vp, vp]
        lib.orc_run_range.argtypes = [vp, i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, u64, i32]

    @staticmethod
    def _p(a):
        return None if a is None else a.ctypes.data_as(C.c_void_p)

    def philox(self, ctr, key):
        c = np.asarray(ctr, np.uint32)
        k = np.asarray(key, np.uint32)
        out = np.zeros(4, np.uint32)
        self.lib.orc_philox4x32_10(self._p(c), self._p(k), self._p(out))
        return out

    def explore_draw(self, seed, env, t, A):
        u, a = C.c_float(), C.c_int32()
        self.lib.orc_explore_draw(seed, env, t, A, C.byref(u), C.byref(a))
        return u.value, a.value

    def step_e1(self, W, H, x, y, done, action):
        cx, cy, cd, r = C.c_int(x), C.c_int(y), C.c_int(done), C.c_float(0)
        self.lib.orc_step_e1(W, H, C.byref(cx), C.byref(cy), C.byref(r), C.byref(cd), action)
        return cx.value, cy.value, r.value, cd.value

    def step_e2(self, grid, W, H, x, y, done, action):
        g = np.ascontiguousarray(grid, np.float32)
        cx, cy, cd, r = C.c_int(x), C.c_int(y), C.c_int(done), C.c_float(0)
        self.lib.orc_step_e2(self._p(g), W, H, C.byref(cx), C.byref(cy), C.byref(r), C.byref(cd), action)
        return cx.value, cy.value, r.value, cd.value

    def reset_xy(self, W, H):
        cx, cy, cd, r = C.c_int(-1), C.c_int(-1), C.c_int(1), C.c_float(7)
        self.lib.orc_reset_xy(W, H, C.byref(cx), C.byref(cy), C.byref(r), C.byref(cd))
        return cx.value, cy.value, r.value, cd.value

    def step_cls(self, cfg, cls, cr, s, action):
        cls = np.ascontiguousarray(cls, np.uint8)
        cr = None if cr is None else np.ascontiguousarray(cr, np.float32)
        cs, r = C.c_int32(s), C.c_float(0)
        hit = self.lib.orc_step_cls(C.byref(cfg), self._p(cls), self._p(cr), C.byref(cs), action,
                                    C.byref(r))
        return cs.value, r.value, hit

    def argmax(self, row):
        row = np.ascontiguousarray(row, np.float32)
        return self.lib.orc_argmax(self._p(row), row.size)

    def td_update_batch(self, Q, S, A, s, a, r, s2, done, lr, gamma, mode):
        s, a, s2 = (np.ascontiguousarray(v, np.int32) for v in (s, a, s2))
        r = np.ascontiguousarray(r, np.float32)
        done = np.ascontiguousarray(done, np.uint8)
        rc = self.lib.orc_td_update_batch(self._p(Q), S, A, s.size, self._p(s), self._p(a), self._p(r),
                                          self._p(s2), self._p(done), lr, gamma, mode)
        assert rc == 0

    def tree_sum(self, key, d, K, brute=False):
        key = np.ascontiguousarray(key, np.int32)
        d = np.ascontiguousarray(d, np.float32)
        out = np.empty(K, np.float32)
        fn = self.lib.orc_tree_sum_bruteforce if brute else self.lib.orc_tree_sum
        assert fn(self._p(key), self._p(d), key.size, K, self._p(out)) == 0
        return out

    def eps_table(self, cfg):
        n = self.lib.orc_eps_table(C.byref(cfg), None, 0)
        out = np.empty(n, np.float32)
        self.lib.orc_eps_table(C.byref(cfg), self._p(out), n)
        return out

    def new_state(self, cfg, start):
        N = cfg.n_envs
        return dict(s=np.array(start, np.int32).copy(), ep_step=np.zeros(N, np.int32),
                    episode=np.zeros(N, np.int32), reward=np.zeros(N, np.float32),
                    done=np.zeros(N, np.uint8), action=np.zeros(N, np.uint8))

    @staticmethod
    def new_stats(n):
        return dict(ret_acc=np.zeros(n, np.float32), last_return=np.zeros(n, np.float32),
                    return_sum=np.zeros(n, np.float32), last_length=np.zeros(n, np.int32),
                    length_sum=np.zeros(n, np.int32))

    def run(self, cfg, cls, cr, start, Q, st, t0, n_steps, u=None, a_rand=None, trace_n=0, stats=None):
        """Advance `st` and `Q` (and `stats`, from new_stats) in place; returns the
        trace dict (or None)."""
        cls = np.ascontiguousarray(cls, np.uint8)
        cr = None if cr is None else np.ascontiguousarray(cr, np.float32)
        start = np.ascontiguousarray(start, np.int32)
        u = None if u is None else np.ascontiguousarray(u, np.float32)
        a_rand = None if a_rand is None else np.ascontiguousarray(a_rand, np.int32)
        tr = None
        if trace_n:
            tr = dict(s_next=np.zeros((n_steps, trace_n), np.int32),
                      action=np.zeros((n_steps, trace_n), np.uint8),
                      reward=np.zeros((n_steps, trace_n), np.float32),
                      done=np.zeros((n_steps, trace_n), np.uint8))
        rc = self.lib.orc_run(C.byref(cfg), self._p(cls), self._p(cr), self._p(start), self._p(Q),
                              self._p(st["s"]), self._p(st["ep_step"]), self._p(st["episode"]),
                              self._p(st["reward"]), self._p(st["done"]), self._p(st["action"]), t0,
                              n_steps, self._p(u), self._p(a_rand), trace_n,
                              self._p(tr["s_next"]) if tr else None, self._p(tr["action"]) if tr else None,
                              self._p(tr["reward"]) if tr else None, self._p(tr["done"]) if tr else None,
                              self._p(stats["ret_acc"]) if stats else None,
                              self._p(stats["last_return"]) if stats else None,
                              self._p(stats["return_sum"]) if stats else None,
                              self._p(stats["last_length"]) if stats else None,
                              self._p(stats["length_sum"]) if stats else None)
        assert rc == 0
        return tr


def oracle_run_slice(orc, cfg, lo, hi, cls, start, t0, n_steps, cr=None):
    """Oracle results for envs [lo, hi) of a larger per-env-table batch (envs are
    independent and the draws are keyed by the global env index).  cls / start / cr
    hold only the slice.  Returns (Q[hi-lo, S, A], state dict of the slice)."""
    n = hi - lo
    S, A = cfg.width * cfg.height, cfg.n_actions
    K = S * A
    Q = np.zeros((n, S, A), np.float32)
    st = dict(s=np.array(start, np.int32).copy(), ep_step=np.zeros(n, np.int32), episode=np.zeros(n, np.int32),
              reward=np.zeros(n, np.float32), done=np.zeros(n, np.uint8), action=np.zeros(n, np.uint8))
    cls = np.ascontiguousarray(cls, np.uint8)
    start = np.ascontiguousarray(start, np.int32)
    cr = None if cr is None else np.ascontiguousarray(cr, np.float32)

    def shifted(a, per_env_bytes):  # address such that index `lo` lands on a[0]
        return C.c_void_p(a.ctypes.data - lo * per_env_bytes)

    per_map = 0 if cfg.map_mode == 1 else S
    rc = orc.lib.orc_run_range(C.byref(cfg), lo, hi, shifted(cls, per_map),
                               None if cr is None else shifted(cr, per_map * 4), shifted(start, 4),
                               shifted(Q, K * 4), shifted(st["s"], 4), shifted(st["ep_step"], 4),
                               shifted(st["episode"], 4), shifted(st["reward"], 4), shifted(st["done"], 1),
                               shifted(st["action"], 1), t0, n_steps)
    assert rc == 0
    return Q, st


def host_threads():
    """Threads a test may use: the job's share of the host's cores."""
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    share = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
    return max(1, min(usable, share) if share > 0 else usable)


def oracle_run_threads(orc, cfg, cls, start, t0, n_steps, cr=None, threads=None):
    """Oracle results for ALL envs of a per-env-table batch, the envs spread over host
    threads (they are independent, and the draws are keyed by the env index).
    Returns (Q[N, S, A], state dict)."""
    import threading
    n = cfg.n_envs
    S, A = cfg.width * cfg.height, cfg.n_actions
    Q = np.zeros((n, S, A), np.float32)
    st = orc.new_state(cfg, start)
    cls = np.ascontiguousarray(cls, np.uint8)
    start = np.ascontiguousarray(start, np.int32)
    cr = None if cr is None else np.ascontiguousarray(cr, np.float32)
    threads = threads or host_threads()
    bounds = [n * i // threads for i in range(threads + 1)]
    p = Oracle._p
    rcs = [None] * threads

    def work(i):
        rcs[i] = orc.lib.orc_run_range(C.byref(cfg), bounds[i], bounds[i + 1], p(cls), p(cr), p(start), p(Q),
                                       p(st["s"]), p(st["ep_step"]), p(st["episode"]), p(st["reward"]),
                                       p(st["done"]), p(st["action"]), t0, n_steps)

    ths = [threading.Thread(target=work, args=(i,)) for i in range(threads)]
    for t in ths:
        t.start()
    for t in ths:
        t.join()
    assert rcs == [0] * threads, rcs
    return Q, st


@pytest.fixture(scope="session")
def oracle():
    if not os.path.exists(ORACLE_SO):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "-s"])
    return Oracle(C.CDLL(ORACLE_SO))


@pytest.fixture(scope="session")
def gpu(pycrl):
    """The engine library on a box with a device; the tests that take this are
    marked gpu and must not silently pass without one."""
    lib = pycrl.load()
    n = lib.crl_device_count()
    assert n >= 1, "no HIP device: %s" % lib.crl_last_error().decode()
    return pycrl
