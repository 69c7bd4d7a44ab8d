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


def test_host_only_entry_points_leave_an_error_text(pycrl):
    """crl_last_error() names the calling thread's last failure also for the entry
    points that touch no device (map generators, epsilon table, grid classifier)."""
    lib = pycrl.load()
    with pytest.raises(pycrl.CrlError, match="wall_frac") as e:
        pycrl.gen_maps_noise(0, 2, 8, 8, 4, 1.5, 0.05, 10.0)
    assert e.value.code == -1
    with pytest.raises(pycrl.CrlError, match="one shared map or one map per env"):
        pycrl.gen_maps_bernoulli(0, 3, 7, 4, 4, 0.1)
    with pytest.raises(pycrl.CrlError, match="2 to 2\\^30 cells"):
        pycrl.gen_maps_bernoulli(0, 1, 1, 1, 1, 0.1)
    cfg = pycrl.make_config(4, 4, 4, eps_mode=1, eps_span=0)
    n = C.c_int32()
    assert lib.crl_eps_table(C.byref(cfg), None, 0, C.byref(n)) == -1
    assert b"eps_span" in lib.crl_last_error()
    assert lib.crl_classify_grid(None, 4, C.c_float(-0.01), None, None) == -1
    assert b"crl_classify_grid" in lib.crl_last_error()
    # another thread's failures are its own
    import threading
    seen = []
    t = threading.Thread(target=lambda: seen.append(lib.crl_last_error()))
    t.start()
    t.join()
    assert seen == [b""]


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


def test_noise_map_matches_a_hand_worked_restatement(pycrl, oracle):
    """One tiny value-noise map recomputed from the Philox words up: lattice values,
    smoothstep-bilinear cell values, the k highest as walls, goal and start among
    the free cells, Box-Muller rewards of two known words.  A wrong lattice index,
    a swapped interpolation axis or a sign slip in the rewards changes it."""
    seed, W, H, pitch, frac, sigma, bonus = 11, 6, 5, 4, 0.3, 0.05, 10.0
    cls, start, cr = pycrl.gen_maps_noise(seed, 2, W, H, pitch, frac, sigma, bonus)
    f32 = np.float32
    for m in range(2):
        def word(stream, i):  # counter (map, stream id, i // 4, 0), key = seed
            return int(oracle.philox([m, stream, i // 4, 0], [seed & 0xFFFFFFFF, seed >> 32])[i % 4])
        lw, lh = (W + pitch - 1) // pitch + 1, (H + pitch - 1) // pitch + 1
        assert (lw, lh) == (3, 3)
        lat = np.array([f32(word(5, i) >> 8) * f32(2.0 ** -24) for i in range(lw * lh)], f32).reshape(lh, lw)
        val = np.zeros((H, W), f32)
        for y in range(H):
            for x in range(W):
                gx, gy = x // pitch, y // pitch
                fx, fy = f32(x % pitch) / f32(pitch), f32(y % pitch) / f32(pitch)
                fx = fx * fx * (f32(3) - f32(2) * fx)
                fy = fy * fy * (f32(3) - f32(2) * fy)
                top = lat[gy, gx] + (lat[gy, gx + 1] - lat[gy, gx]) * fx
                bot = lat[gy + 1, gx] + (lat[gy + 1, gx + 1] - lat[gy + 1, gx]) * fx
                val[y, x] = top + (bot - top) * fy
        # corners of a lattice square reproduce the lattice values exactly
        assert val[0, 0] == lat[0, 0] and val[4, 4] == lat[1, 1] and val[0, 4] == lat[0, 1]
        n_wall = int(frac * W * H)
        assert n_wall == 9
        order = sorted(range(W * H), key=lambda c: (-val.ravel()[c], c))
        want = np.zeros(W * H, np.uint8)
        want[order[:n_wall]] = 3
        free = [c for c in range(W * H) if want[c] == 0]
        goal = free[(word(2, 0) * len(free)) >> 32]
        want[goal] = 1
        free.remove(goal)
        assert start[m] == free[(word(2, 1) * len(free)) >> 32]
        assert np.array_equal(cls[m], want)
        for c in range(0, W * H, 2):
            u1 = (f32(word(4, c) >> 8) + f32(1)) * f32(2.0 ** -24)
            u2 = f32(word(4, c + 1) >> 8) * f32(2.0 ** -24)
            rad = np.sqrt(f32(-2) * np.log(u1, dtype=f32), dtype=f32)
            ang = f32(6.28318530717958647692) * u2
            pair = [sigma * rad * np.cos(ang, dtype=f32), sigma * rad * np.sin(ang, dtype=f32)]
            for j in (0, 1):
                if c + j < W * H:
                    got = cr[m, c + j] - (bonus if c + j == goal else 0.0)
                    assert abs(got - pair[j]) <= 2e-6, (m, c + j)
        assert cr[m, goal] > 9.0


def test_every_valid_configuration_has_a_launch_plan_that_fits(pycrl):
    """The fused launch plan over a grid of shapes, host only: at most 160 KB of
    LDS per workgroup and a non-empty grid, also where large per-env maps leave
    room for fewer waves per workgroup than the planner would like."""
    checked = 0
    for A in (4, 8):
        for W, H in ((4, 4), (16, 16), (32, 32), (33, 33), (40, 40), (48, 48), (64, 64), (65, 65), (128, 96),
                     (256, 256)):
            for N in (1, 100, 4096, 16384, 65536, 131072, 262144, 1 << 20):
                if N * W * H * A * 4 > 64 << 30:
                    continue
                for n_steps in (1, 8, 20, 64, 128, 1000):
                    for kw in (dict(), dict(eps_mode=pycrl.EPS_EPISODE_LINEAR, eps0=1.0, eps_end=0.1, eps_span=10),
                               dict(goal_mode=pycrl.GOAL_ON_RESULT)):
                        cfg = pycrl.make_config(N, W, H, n_actions=A, episode_len=128, **kw)
                        plan = pycrl.fused_plan_for_config(cfg, n_steps)  # raises on a plan that does not fit
                        assert 0 <= plan["lds_bytes"] <= 160 * 1024, (N, W, H, A, n_steps, plan)
                        assert plan["grid"] >= 1 and plan["block"] in (64, 128, 192, 256, 320), plan
                        checked += 1
    assert checked > 2000
    # the two cases that used to ask for 192 KB and 256 KB
    for N, n in ((131072, 1000), (65536, 8)):
        plan = pycrl.fused_plan_for_config(pycrl.make_config(N, 64, 64, episode_len=128), n)
        assert plan["lds_bytes"] == 128 * 1024 and plan["block"] == 128
    # the tuned configurations keep their plans
    c4 = pycrl.make_config(1 << 20, 16, 16, episode_len=128, gamma=0.95)
    assert pycrl.fused_plan_for_config(c4, 1000) == dict(name="k_fused_tickets<4,fast,hbm+lds>", grid=256, block=256,
                                                         lds_bytes=152064)
    c2 = pycrl.make_config(4096, 32, 32, episode_len=256)
    assert pycrl.fused_plan_for_config(c2, 10000) == dict(name="k_fused_tickets<4,fast,hbm>", grid=256, block=64,
                                                          lds_bytes=65536)  # 16 envs to a wave: a wave per compute unit
    with pytest.raises(pycrl.CrlError):
        pycrl.fused_plan_for_config(pycrl.make_config(64, 8, 8, table_mode=pycrl.TABLE_SHARED), 10)


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
    # a header that promises more than the file holds is refused before anything is allocated
    def write_npy(shape_text, payload):
        head = "{'descr': '<f8', 'fortran_order': False, 'shape': %s, }" % shape_text
        head += " " * ((64 - (10 + len(head) + 1) % 64) % 64) + "\n"
        with open(path, "wb") as f:
            f.write(b"\x93NUMPY\x01\x00" + len(head).to_bytes(2, "little") + head.encode() + payload)
    payload = table.tobytes()
    write_npy("(%d, %d, %d)" % (W, H, A), payload)
    assert np.array_equal(np.load(path), table)  # the helper writes what numpy reads
    assert np.array_equal(cudarl_core.load_agent_npy(path, W, H, A), got)
    write_npy("(%d, %d, %d)" % (W, H, A), payload[:-8])
    with pytest.raises(RuntimeError, match="truncated"):
        cudarl_core.load_agent_npy(path, W, H, A)
    write_npy("(%d, %d, %d)" % (W, H, 4000000000000000), payload)
    with pytest.raises(RuntimeError, match="truncated"):
        cudarl_core.load_agent_npy(path, W, H, A)
    write_npy("(%d, %d, %d)" % (1 << 62, 1 << 62, 16), payload)  # the element count wraps around 2^64
    with pytest.raises(RuntimeError, match="truncated"):
        cudarl_core.load_agent_npy(path, W, H, A)
    write_npy("(%d, %d, %d)" % (W, -H, A), payload)
    with pytest.raises(RuntimeError, match="negative"):
        cudarl_core.load_agent_npy(path, W, H, A)
    # raw fp32 tables of any shape
    big = rng.normal(0, 1, (3, 6, 8)).astype(np.float32)
    cudarl_core.save_table_npy(path, big)
    back = np.load(path)
    assert back.dtype == np.float32 and np.array_equal(back, big)
    cudarl_core.save_table_npy(path, big[0, 0])
    assert np.array_equal(np.load(path), big[0, 0])
