"""CPU-side checks of the C ABI library: it loads, exports every symbol
include/crl.h declares, and its host-only helpers (Philox, epsilon tables, map
generators, configuration checks) behave.  No compute call needs a GPU here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "crl.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(crl_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pycrl):
    lib = pycrl.load()
    names = declared_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), "libcrl.so does not export %s" % n
    assert sorted(pycrl.EXPORTS) == names
    assert lib.crl_version().decode() == "0.1.0"  # src/python_bindings.cpp:24


def test_config_struct_matches_header(pycrl):
    # 24 four-byte fields then one uint64 at an 8-byte boundary
    assert C.sizeof(pycrl.Config) == 104
    assert pycrl.Config.seed.offset == 96


def test_philox_matches_oracle_and_kat(pycrl, oracle):
    lib = pycrl.load()
    rng = np.random.default_rng(0)
    for _ in range(100):
        ctr = rng.integers(0, 2**32, 4, dtype=np.uint64).astype(np.uint32)
        key = rng.integers(0, 2**32, 2, dtype=np.uint64).astype(np.uint32)
        out = np.zeros(4, np.uint32)
        lib.crl_philox4x32_10(ctr.ctypes.data, key.ctypes.data, out.ctypes.data)
        assert np.array_equal(out, oracle.philox(ctr, key))
    z4, z2, out = np.zeros(4, np.uint32), np.zeros(2, np.uint32), np.zeros(4, np.uint32)
    lib.crl_philox4x32_10(z4.ctypes.data, z2.ctypes.data, out.ctypes.data)
    assert [hex(int(x)) for x in out] == ["0x6627e8d5", "0xe169c58d", "0xbc57ac4c", "0x9b00dbd8"]
    for seed, env, t in [(0, 0, 0), (2**40 + 3, 123456, 2**33 + 1), (7, 2**31, 999)]:
        u, a = C.c_float(), C.c_int32()
        lib.crl_explore_draw(seed, env, t, 8, C.byref(u), C.byref(a))
        assert (u.value, a.value) == oracle.explore_draw(seed, env, t, 8)


def test_create_rejects_bad_configs_without_touching_a_device(pycrl):
    lib = pycrl.load()
    bad = [dict(n_envs=0), dict(width=0), dict(n_actions=5), dict(table_mode=3), dict(max_mode=2),
           dict(episode_len=-1), dict(reward_flags=2), dict(eps_mode=1, eps_span=0), dict(auto_reset=2),
           dict(max_episodes=-1), dict(track_returns=2)]
    for kw in bad:
        base = dict(n_envs=4, width=4, height=4)
        base.update(kw)
        cfg = pycrl.make_config(**base)
        h = C.c_void_p()
        assert lib.crl_create(C.byref(cfg), 0, C.byref(h)) == -1, kw
        assert h.value is None and lib.crl_last_error()
    cfg = pycrl.make_config(4, 4, 4)
    cfg.struct_size = 12
    h = C.c_void_p()
    assert lib.crl_create(C.byref(cfg), 0, C.byref(h)) == -1
    assert b"struct_size" in lib.crl_last_error()
    assert lib.crl_destroy(None) == 0


def test_engine_fails_loudly_without_a_device(pycrl):
    """No CPU fallback: on a box without a HIP device crl_create reports
    CRL_E_DEVICE (on a GPU box this test has nothing to check)."""
    lib = pycrl.load()
    if lib.crl_device_count() >= 1:
        pytest.skip("a HIP device is present")
    with pytest.raises(pycrl.CrlError) as e:
        pycrl.Engine(pycrl.make_config(4, 4, 4))
    assert e.value.code == -2 and "no CPU path" in str(e.value)


def test_bernoulli_maps(pycrl):
    N, W, H = 500, 16, 16
    cls, start = pycrl.gen_maps_bernoulli(5, N, N, W, H, 0.1, 0.02)
    cls2, start2 = pycrl.gen_maps_bernoulli(5, N, N, W, H, 0.1, 0.02)
    assert np.array_equal(cls, cls2) and np.array_equal(start, start2)  # reproducible
    assert ((cls == 1).sum(axis=1) == 1).all()  # exactly one goal per map
    assert (cls[np.arange(N), start] == 0).all()  # starts are free cells (so never the goal)
    assert abs((cls == 3).mean() - 0.1) < 0.01
    assert abs((cls == 2).mean() - 0.9 * 0.02) < 0.004
    other, _ = pycrl.gen_maps_bernoulli(6, N, N, W, H, 0.1, 0.02)
    assert not np.array_equal(cls, other)
    # shared map, per-env starts
    cls, start = pycrl.gen_maps_bernoulli(1, 1, 4000, 64, 64, 0.15)
    assert cls.shape == (1, 4096) and (cls[0, start] == 0).all()
    assert len(np.unique(start)) > 1500
    # degenerate: all walls still leaves a start and a goal
    cls, start = pycrl.gen_maps_bernoulli(1, 3, 3, 2, 2, 1.0)
    assert ((cls == 1).sum(axis=1) == 1).all() and (cls[np.arange(3), start] == 0).all()


def test_noise_maps(pycrl):
    N, W, H = 3, 64, 64
    cls, start, cr = pycrl.gen_maps_noise(9, N, W, H, 16, 0.25, 0.05, 10.0)
    assert ((cls == 3).sum(axis=1) == W * H // 4).all()
    assert ((cls == 1).sum(axis=1) == 1).all() and (cls[np.arange(N), start] == 0).all()
    goal = np.argmax(cls == 1, axis=1)
    assert (cr[np.arange(N), goal] > 9.0).all()
    rest = np.delete(cr[0], goal[0])
    assert abs(rest.mean()) < 0.005 and abs(rest.std() - 0.05) < 0.005
    # walls are spatially coherent (value noise), unlike Bernoulli cells
    walls = (cls[0] == 3).reshape(H, W)
    same_right = (walls[:, 1:] == walls[:, :-1]).mean()
    assert same_right > 0.9


def test_npy_agent_files_match_numpy(pycrl, tmp_path):
    """QTableAgent.save / load files (src/train.py:150-168): float64 (W, H, A)
    indexed [x, y, a], exchanged with numpy in both directions."""
    import sys
    sys.path.insert(0, os.path.join(ROOT, "cudarl-arena_amd", "lib"))
    import cudarl_core
    W, H, A = 7, 5, 4
    rng = np.random.default_rng(0)
    q = rng.normal(0, 1, (W * H, A)).astype(np.float32)
    path = str(tmp_path / "agent.npy")
    cudarl_core.save_agent_npy(path, q, W, H, A)
    ref = np.load(path)
    assert ref.dtype == np.float64 and ref.shape == (W, H, A)
    for x in range(W):
        for y in range(H):
            assert np.array_equal(ref[x, y], q[y * W + x].astype(np.float64))
    assert np.array_equal(cudarl_core.load_agent_npy(path, W, H, A), q)
    # a file written by numpy, as the reference's agent.save would
    table = rng.normal(0, 1, (W, H, A))
    np.save(path, table)
    got = cudarl_core.load_agent_npy(path, W, H, A)
    assert got.dtype == np.float32 and got.shape == (W * H, A)
    assert np.array_equal(got.reshape(H, W, A), np.transpose(table, (1, 0, 2)).astype(np.float32))
    np.save(path, table.astype(np.float32))
    assert np.array_equal(cudarl_core.load_agent_npy(path, W, H, A), got)
    with pytest.raises(RuntimeError, match="Invalid Q-table size"):
        cudarl_core.load_agent_npy(path, W + 1, H, A)
    np.save(path, np.asfortranarray(table))
    with pytest.raises(RuntimeError):
        cudarl_core.load_agent_npy(path, W, H, A)
    np.save(path, np.arange(5))
    with pytest.raises(RuntimeError):
        cudarl_core.load_agent_npy(path, W, H, A)
    with pytest.raises(RuntimeError):
        cudarl_core.load_agent_npy(str(tmp_path / "missing.npy"), W, H, A)
    # raw fp32 tables of any shape
    big = rng.normal(0, 1, (3, 6, 8)).astype(np.float32)
    cudarl_core.save_table_npy(path, big)
    back = np.load(path)
    assert back.dtype == np.float32 and np.array_equal(back, big)
    cudarl_core.save_table_npy(path, big[0, 0])
    assert np.array_equal(np.load(path), big[0, 0])
