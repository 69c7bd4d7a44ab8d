"""Pins the CPU oracle to what the reference itself fixes: the Catch2 cases of
tests/test_environment.cpp, the training.log vector, Random123 known answers,
and what the mathematics fixes (closed forms, brute force, float64 restatement
of src/train.py).  No GPU."""
import json
import math
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def load(name):
    with open(os.path.join(GOLD, name)) as f:
        return json.load(f)


# ---- Philox4x32-10 ----------------------------------------------------------

def test_philox_known_answers(oracle):
    for v in load("philox4x32_10_kat.json")["vectors"]:
        out = oracle.philox([int(x, 16) for x in v["ctr"]], [int(x, 16) for x in v["key"]])
        assert [int(x) for x in out] == [int(x, 16) for x in v["out"]]


def test_philox_numpy_restatement(oracle):
    """An independent numpy restatement of the published round function."""
    rng = np.random.default_rng(1)

    def ref(ctr, key):
        c = [int(x) for x in ctr]
        k = [int(x) for x in key]
        for _ in range(10):
            p0 = 0xD2511F53 * c[0]
            p1 = 0xCD9E8D57 * c[2]
            c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & 0xFFFFFFFF, (p0 >> 32) ^ c[3] ^ k[1], p0 & 0xFFFFFFFF]
            k = [(k[0] + 0x9E3779B9) & 0xFFFFFFFF, (k[1] + 0xBB67AE85) & 0xFFFFFFFF]
        return c

    for _ in range(50):
        ctr = rng.integers(0, 2**32, 4, dtype=np.uint64)
        key = rng.integers(0, 2**32, 2, dtype=np.uint64)
        assert [int(x) for x in oracle.philox(ctr, key)] == ref(ctr, key)


def test_explore_draw_layout(oracle):
    """Two steps share one block: even t -> words 0,1; odd t -> words 2,3."""
    seed, env, A = 0x1234567890ABCDEF, 77, 4
    for t in (0, 1, 10, 11, 2**33 + 5):
        blk = t >> 1
        w = oracle.philox([env, 0, blk & 0xFFFFFFFF, blk >> 32], [seed & 0xFFFFFFFF, seed >> 32])
        w0, w1 = (int(w[2]), int(w[3])) if t & 1 else (int(w[0]), int(w[1]))
        u, a = oracle.explore_draw(seed, env, t, A)
        assert u == (w0 >> 8) / 2.0**24
        assert a == (w1 * A) >> 32
        assert 0.0 <= u < 1.0 and 0 <= a < A


def test_explore_draw_statistics(oracle):
    us, acts = [], []
    for env in range(200):
        for t in range(50):
            u, a = oracle.explore_draw(0, env, t, 4)
            us.append(u)
            acts.append(a)
    us = np.array(us)
    assert abs(us.mean() - 0.5) < 0.01
    counts = np.bincount(acts, minlength=4)
    chi2 = ((counts - 2500.0) ** 2 / 2500.0).sum()
    assert chi2 < 16.27  # p = 0.001, 3 dof


# ---- E0 / E1: the Catch2 cases ------------------------------------------------

def test_catch2_environment_cases(oracle):
    """tests/test_environment.cpp, every REQUIRE, against orc_reset_xy/orc_step_e1."""
    g = load("catch2_environment.json")
    for case in g["cases"]:
        W, H = case["width"], case["height"]
        x, y, r, d = oracle.reset_xy(W, H)
        if "reset_expect" in case:
            assert [x, y, r, d] == case["reset_expect"], case["name"]
        for a in case.get("actions", []):
            x, y, r, d = oracle.step_e1(W, H, x, y, d, a)
        if case.get("reset_after"):
            x, y, r, d = oracle.reset_xy(W, H)
        e = case["expect"]
        if "x" in e:
            assert x == e["x"], case["name"]
        if "y" in e:
            assert y == e["y"], case["name"]
        if "reward" in e:
            assert r == pytest.approx(e["reward"], rel=1e-6), case["name"]
        if "done" in e:
            assert bool(d) == e["done"], case["name"]


def test_e1_done_is_sticky_and_refires(oracle):
    # src/environment.cu:43-46: done never cleared; goal test on the resulting cell
    x, y, r, d = 4, 0, 0.0, 0
    x, y, r, d = oracle.step_e1(5, 5, 3, 0, 0, 1)
    assert (x, y, r, d) == (4, 0, 1.0, 1)
    x, y, r, d = oracle.step_e1(5, 5, x, y, d, 3)  # walk off the goal
    assert (x, y, d) == (3, 0, 1) and r == pytest.approx(-0.01)
    x, y, r, d = oracle.step_e1(5, 5, 4, 0, 0, 0)  # bump the top wall while on the goal
    assert (x, y, r, d) == (4, 0, 1.0, 1)
    x, y, r, d = oracle.step_e1(5, 5, 2, 2, 0, 9)  # invalid action: no move
    assert (x, y, d) == (2, 2, 0) and r == pytest.approx(-0.01)


# ---- E2: walls / traps / goal by cell value -----------------------------------

EDGE_VALUES = [-2.0, -1.0, np.nextafter(np.float32(-1.0), np.float32(0.0)), -0.5, -0.1,
               np.float32(-1e-30), -0.0, 0.0, 0.25, 0.5, np.nextafter(np.float32(0.99), np.float32(0.0)),
               np.float32(0.99), 1.0, 3.0]


def classify_py(v):
    v = np.float32(v)
    if v >= np.float32(0.99):
        return 1
    if np.float32(-1.0) < v < np.float32(0.0):
        return 2
    if v < np.float32(0.0):
        return 3
    return 0


def test_classify_thresholds(oracle):
    for v in EDGE_VALUES:
        assert oracle.lib.orc_classify(float(np.float32(v))) == classify_py(v), v
    # -0.0 is not < 0: FREE.  exactly -1.0 is a wall, not a trap (src/kernels.cu:60)
    assert oracle.lib.orc_classify(-0.0) == 0
    assert oracle.lib.orc_classify(-1.0) == 3


def test_e2_invariants_brute_force(oracle):
    """Every (cell, action) on a grid holding every class and edge value:
    the invariants src/kernels.cu:13-66 implies."""
    W, H = 5, 4
    rng = np.random.default_rng(3)
    vals = np.array(EDGE_VALUES, np.float32)
    for trial in range(6):
        grid = vals[rng.integers(0, len(vals), W * H)].astype(np.float32)
        for y in range(H):
            for x in range(W):
                for a in range(-1, 6):
                    nx, ny, r, d = oracle.step_e2(grid, W, H, x, y, 0, a)
                    dx, dy = {0: (0, -1), 1: (1, 0), 2: (0, 1), 3: (-1, 0)}.get(a, (0, 0))
                    tx, ty = x + dx, y + dy
                    inb = 0 <= tx < W and 0 <= ty < H
                    assert 0 <= nx < W and 0 <= ny < H
                    if not inb:
                        assert (nx, ny) == (x, y) and r == np.float32(-0.01) and d == 0
                        continue
                    v = grid[ty * W + tx]
                    if v < 0:  # blocked: never enter
                        assert (nx, ny) == (x, y)
                    else:
                        assert (nx, ny) == (tx, ty)
                    if v >= np.float32(0.99):
                        assert r == 1.0 and d == 1
                    elif np.float32(-1.0) < v < 0:
                        assert r == v and d == 0
                    else:
                        assert r == np.float32(-0.01) and d == 0


def test_e2_reduces_to_e1_without_obstacles(oracle):
    rng = np.random.default_rng(5)
    W, H = 6, 5
    grid = (rng.random(W * H) * 0.5).astype(np.float32)
    grid[W - 1] = 1.0  # src/environment.cu:146
    for _ in range(300):
        x, y = int(rng.integers(W)), int(rng.integers(H))
        a = int(rng.integers(4))
        r1 = oracle.step_e1(W, H, x, y, 0, a)
        r2 = oracle.step_e2(grid, W, H, x, y, 0, a)
        if (x, y) == (W - 1, 0) and r1[:2] == (x, y):
            continue  # the bump-on-goal case is where the two kernels differ
        assert r1 == r2


def test_step_cls_equals_e2_on_classified_grids(oracle, pycrl):
    """The class-based rule the engine uses == the float rule of the reference."""
    W, H = 5, 4
    rng = np.random.default_rng(7)
    vals = np.array(EDGE_VALUES, np.float32)
    cfg = pycrl.make_config(1, W, H, reward_flags=pycrl.REWARD_CELLS, auto_reset=0)
    for trial in range(8):
        grid = vals[rng.integers(0, len(vals), W * H)].astype(np.float32)
        cls = np.array([classify_py(v) for v in grid], np.uint8)
        cr = np.where(cls == 1, np.float32(1.0), np.where(cls == 2, grid, np.float32(-0.01))).astype(np.float32)
        for s in range(W * H):
            for a in range(-1, 6):
                x, y = s % W, s // W
                nx, ny, r, d = oracle.step_e2(grid, W, H, x, y, 0, a)
                s2, r2, hit = oracle.step_cls(cfg, cls, cr, s, a)
                assert (s2, r2, hit) == (ny * W + nx, r, d)
    # the library's classifier agrees with the oracle's
    big = vals[rng.integers(0, len(vals), 1000)]
    lc, lr = pycrl.classify_grid(big)
    assert list(lc) == [classify_py(v) for v in big]
    assert np.array_equal(lr, np.where(lc == 1, np.float32(1.0), np.where(lc == 2, big, np.float32(-0.01))))


def test_step_cls_result_goal_mode_equals_e1(oracle, pycrl):
    W, H = 5, 5
    cls = np.zeros(W * H, np.uint8)
    cls[W - 1] = 1
    cfg = pycrl.make_config(1, W, H, goal_mode=pycrl.GOAL_ON_RESULT, auto_reset=0)
    for s in range(W * H):
        for a in range(-1, 6):
            x, y, r, d = oracle.step_e1(W, H, s % W, s // W, 0, a)
            s2, r2, hit = oracle.step_cls(cfg, cls, None, s, a)
            assert (s2, r2, hit) == (y * W + x, r, d)


def test_step_cls_diagonals(oracle, pycrl):
    W, H = 4, 4
    cls = np.zeros(W * H, np.uint8)
    cls[1 * W + 2] = 3  # wall at (2,1)
    cfg = pycrl.make_config(1, W, H, n_actions=8, auto_reset=0)
    s = 2 * W + 1  # (1,2)
    expect = {4: s, 5: 3 * W + 2, 6: 3 * W + 0, 7: 1 * W + 0}  # UR blocked by the wall
    for a, e in expect.items():
        assert oracle.step_cls(cfg, cls, None, s, a)[0] == e
    assert oracle.step_cls(cfg, cls, None, 0, 7)[0] == 0  # UL out of bounds


# A 4x3 map holding every class, with per-cell rewards cr[c] = c + 0.5 so that a
# reward names the cell it was read from.  Expectations are worked by hand from the
# rule (goal / trap pay on the TARGET cell, anything else on the cell the env stands
# on after the move when CRL_REWARD_BASE_CELLS is set, else the step reward):
#      x0  x1  x2  x3
#  y0  F0  F1  G2  F3
#  y1  F4  T5  W6  F7
#  y2  F8  F9  F10 F11
HAND_MAP = dict(W=4, H=3, cls=[0, 0, 1, 0, 0, 2, 3, 0, 0, 0, 0, 0], cr=[c + 0.5 for c in range(12)])
# (reward_flags, goal_mode, s, action) -> (s after, reward, hit)
HAND_CASES = [
    # per-cell base rewards, goal test on the target cell
    (3, 0, 1, 1, (2, 2.5, 1)),    # right onto the goal: moves, goal cell pays
    (3, 0, 1, 2, (1, 5.5, 0)),    # down into the trap: stays, the trap cell pays
    (3, 0, 7, 3, (7, 7.5, 0)),    # left into the wall: stays, own cell pays
    (3, 0, 0, 0, (0, 0.5, 0)),    # up out of the grid: stays, own cell pays
    (3, 0, 0, 1, (1, 1.5, 0)),    # plain move: the cell moved onto pays
    (3, 0, 9, 4, (9, 9.5, 0)),    # up-right (2,1) is the wall: stays
    (3, 0, 8, 4, (8, 5.5, 0)),    # up-right (1,1) is the trap: stays, trap pays
    (3, 0, 7, 7, (2, 2.5, 1)),    # up-left (2,0) is the goal
    (3, 0, 4, 5, (9, 9.5, 0)),    # down-right (1,2) free
    (3, 0, 3, 6, (3, 3.5, 0)),    # down-left (2,1) is the wall
    (3, 0, 11, 5, (11, 11.5, 0)),  # down-right out of the grid
    (3, 0, 2, 0, (2, 2.5, 0)),    # on the goal, bump: target test does not fire again
    # goal / trap rewards from the cells only: a plain step pays the step reward
    (1, 0, 0, 1, (1, -0.01, 0)),
    (1, 0, 1, 1, (2, 2.5, 1)),
    (1, 0, 1, 2, (1, 5.5, 0)),
    (1, 0, 7, 3, (7, -0.01, 0)),
    (1, 0, 4, 5, (9, -0.01, 0)),
    # goal test on the resulting cell (src/environment.cu:43): fires again on a bump
    (3, 1, 2, 0, (2, 2.5, 1)),
    (3, 1, 2, 2, (2, 2.5, 1)),
    (3, 1, 1, 2, (1, 5.5, 0)),
    (3, 1, 1, 1, (2, 2.5, 1)),
    (3, 1, 0, 1, (1, 1.5, 0)),
    (3, 1, 7, 7, (2, 2.5, 1)),
    # class rewards (no cell array): step -0.01, goal 1, trap -0.75
    (0, 0, 1, 2, (1, -0.75, 0)),
    (0, 0, 1, 1, (2, 1.0, 1)),
    (0, 0, 8, 4, (8, -0.75, 0)),
    (0, 0, 9, 4, (9, -0.01, 0)),
]


def test_step_cls_hand_worked_cell_rewards(oracle, pycrl):
    m = HAND_MAP
    cls, cr = np.array(m["cls"], np.uint8), np.array(m["cr"], np.float32)
    for flags, goal_mode, s, a, want in HAND_CASES:
        cfg = pycrl.make_config(1, m["W"], m["H"], n_actions=8, reward_flags=flags, goal_mode=goal_mode,
                                auto_reset=0, trap_reward=-0.75)
        s2, r, hit = oracle.step_cls(cfg, cls, cr if flags else None, s, a)
        assert (s2, r, hit) == (want[0], np.float32(want[1]), want[2]), (flags, goal_mode, s, a)


# ---- S2 argmax ---------------------------------------------------------------

def test_argmax_lowest_index_on_ties(oracle):
    assert oracle.argmax([0, 0, 0, 0]) == 0  # src/q_learning.cu:200-206
    assert oracle.argmax([-1, 2, 2, 1]) == 1
    rng = np.random.default_rng(11)
    for _ in range(200):
        row = rng.integers(-2, 3, rng.choice([4, 8])).astype(np.float32)
        assert oracle.argmax(row) == int(np.argmax(row))  # src/train.py:108


# ---- Q1 / Q2 TD update: closed forms ------------------------------------------

def test_td_single_sample_zero_table(oracle):
    q = np.zeros(16, np.float32)
    oracle.lib.orc_td_update_one(oracle._p(q), 4, 1, 2, -0.01, 3, 0, 0.1, 0.99, 0)
    assert q[1 * 4 + 2] == np.float32(np.float32(0.1) * np.float32(-0.01))
    assert np.count_nonzero(q) == 1


def test_td_summed_form_single_sample_is_two_roundings(oracle):
    """One sample on one table through the batch / shared-table form: Q + lr*(target - Q)
    with the product rounded before the add (the form that sums over duplicates) -
    equal to the numpy float32 expression, and off the contracted fmaf(lr, target - Q, Q)
    that the per-env path and nvcc's single-sample update use by no more than that one
    extra rounding (half an ulp of the product, plus the final rounding)."""
    rng = np.random.default_rng(3)
    f32 = np.float32
    lr, gamma = f32(0.1), f32(0.99)
    differ = 0
    for _ in range(2000):
        q0, r, m = (f32(v) for v in rng.normal(0, 1, 3))
        Q = np.zeros((2, 4), f32)
        Q[0, 1], Q[1] = q0, [m, m - f32(1), m - f32(2), m - f32(3)]
        oracle.td_update_batch(Q, 2, 4, [0], [1], [r], [1], [0], float(lr), float(gamma), 0)
        target = f32(np.float64(gamma) * np.float64(m) + np.float64(r))  # fmaf(gamma, m, r): one rounding
        prod = f32(lr * f32(target - q0))
        want = f32(q0 + prod)
        assert Q[0, 1] == want
        fused = f32(oracle.lib.orc_td_value(q0, r, m, lr, gamma))
        bound = 0.5 * float(np.spacing(np.abs(prod))) + float(np.spacing(np.abs(want)))
        assert abs(float(fused) - float(want)) <= bound
        differ += fused != want
    assert 0 < differ < 1500  # the two forms do differ on a fair share of inputs


def test_td_self_loop_geometric_series(oracle):
    lr, gamma, r, n = 0.1, 0.99, -0.01, 400
    for mode in (0, 1):
        q = np.zeros(4, np.float32)
        for _ in range(n):
            oracle.lib.orc_td_update_one(oracle._p(q), 4, 0, 0, r, 0, 0, lr, gamma, mode)
        if mode == 0:
            # the row is (q,0,0,0): max is 0 while q < 0 -> same as the floored form here,
            # so use a row whose other entries are very negative to expose the true max
            pass
        exact_floor = r * (1 - (1 - lr) ** n)
        assert q[0] == pytest.approx(exact_floor, rel=2e-5)
    # true max with a one-action-like row: other actions far below
    q = np.array([0, -100, -100, -100], np.float32)
    for _ in range(n):
        oracle.lib.orc_td_update_one(oracle._p(q), 4, 0, 0, r, 0, 0, lr, gamma, 0)
    exact = r / (1 - gamma) * (1 - (1 - lr * (1 - gamma)) ** n)
    assert q[0] == pytest.approx(exact, rel=2e-5)
    # floored max on the same row stays on the other series
    q = np.array([0, -100, -100, -100], np.float32)
    for _ in range(n):
        oracle.lib.orc_td_update_one(oracle._p(q), 4, 0, 0, r, 0, 0, lr, gamma, 1)
    assert q[0] == pytest.approx(r * (1 - (1 - lr) ** n), rel=2e-5)


def test_td_done_drops_bootstrap(oracle):
    q = np.full(8, 5.0, np.float32)
    oracle.lib.orc_td_update_one(oracle._p(q), 4, 0, 1, 1.0, 1, 1, 0.5, 0.9, 0)
    assert q[1] == pytest.approx(5.0 + 0.5 * (1.0 - 5.0))
    q = np.full(8, 5.0, np.float32)
    oracle.lib.orc_td_update_one(oracle._p(q), 4, 0, 1, 1.0, 1, 0, 0.5, 0.9, 0)
    assert q[1] == pytest.approx(5.0 + 0.5 * (1.0 + 0.9 * 5.0 - 5.0))


def test_td_matches_float64_train_py(oracle):
    """src/train.py:127-138 in float64 on a [x,y,a] table, same transitions."""
    rng = np.random.default_rng(13)
    W, H, A, lr, gamma = 6, 5, 4, 0.1, 0.99
    q32 = np.zeros(W * H * A, np.float32)
    q64 = np.zeros((W, H, A))
    for _ in range(3000):
        x, y, nx, ny = (int(rng.integers(W)), int(rng.integers(H)), int(rng.integers(W)),
                        int(rng.integers(H)))
        a, done = int(rng.integers(A)), bool(rng.random() < 0.05)
        r = float(rng.choice([-0.01, 1.0, -0.5]))
        oracle.lib.orc_td_update_one(oracle._p(q32), A, y * W + x, a, r, ny * W + nx, int(done), lr,
                                     gamma, 0)
        cur = q64[x, y, a]
        nxt = 0 if done else np.max(q64[nx, ny])
        q64[x, y, a] += lr * (r + gamma * nxt - cur)
    ref = np.transpose(q64, (1, 0, 2)).reshape(-1)  # [x,y,a] -> (y*W+x)*A+a
    assert np.allclose(q32, ref, rtol=1e-5, atol=1e-6)


def tree_sum_py(key, d, K):
    """The ordered tree by its definition: blocks of 256 samples, groups of 16
    blocks, each level added left to right from +0.0f."""
    f = np.float32
    total = np.zeros(K, np.float32)
    n = len(key)
    for k in range(K):
        tot = f(0)
        for g0 in range(0, n, 256 * 16):
            gs = f(0)
            for b0 in range(g0, min(n, g0 + 256 * 16), 256):
                bs = f(0)
                for i in range(b0, min(n, b0 + 256)):
                    if key[i] == k:
                        bs = f(bs + d[i])
                gs = f(gs + bs)
            tot = f(tot + gs)
        total[k] = tot
    return total


def test_ordered_tree_sum(oracle):
    """The touched-keys implementation == the definition, in C and in Python;
    deltas of mixed magnitude make any other association visible."""
    rng = np.random.default_rng(23)
    for n, K in ((1, 4), (200, 8), (256, 3), (257, 3), (4096, 5), (4097, 5), (9000, 7), (70000, 6)):
        key = rng.integers(-1, K, n).astype(np.int32)
        d = (rng.normal(0, 1, n) * 10.0 ** rng.integers(-4, 4, n)).astype(np.float32)
        fast = oracle.tree_sum(key, d, K)
        assert np.array_equal(fast, oracle.tree_sum(key, d, K, brute=True)), (n, K)
        if n <= 9000:
            assert np.array_equal(fast, tree_sum_py(key, d, K)), (n, K)
    # the order matters: one long run of a key is not summed left to right past a block edge
    key = np.zeros(600, np.int32)
    d = (rng.normal(0, 1, 600) * 10.0 ** rng.integers(-4, 4, 600)).astype(np.float32)
    ltr = np.float32(0)
    for v in d:
        ltr = np.float32(ltr + v)
    tree = oracle.tree_sum(key, d, 1)[0]
    assert tree == tree_sum_py(key, d, 1)[0]
    assert abs(float(tree) - float(ltr)) <= 1e-5 * abs(float(ltr)) + 1e-3  # same sum, other rounding
    # up to 256 samples it IS left to right
    assert oracle.tree_sum(key[:256], d[:256], 1)[0] == np.float32(sum_ltr(d[:256]))


def sum_ltr(d):
    acc = np.float32(0)
    for v in d:
        acc = np.float32(acc + v)
    return acc


def test_td_batch_rule_brute_force(oracle):
    """Pre-batch reads, per-(s,a) sums in sample order from +0, then apply
    (n <= 256 here, where the tree is plain left-to-right summation)."""
    rng = np.random.default_rng(17)
    S, A, lr, gamma = 6, 4, np.float32(0.1), np.float32(0.99)
    for mode in (0, 1):
        for n in (1, 5, 64, 256):
            Q = rng.normal(0, 1, S * A).astype(np.float32)
            s, a, s2 = rng.integers(0, S, n), rng.integers(0, A, n), rng.integers(0, S, n)
            r = rng.normal(0, 1, n).astype(np.float32)
            done = (rng.random(n) < 0.2).astype(np.uint8)
            pre = Q.copy()
            lists = {}
            for i in range(n):
                row = pre[s2[i] * A:(s2[i] + 1) * A]
                m = np.float32(0) if done[i] else row.max()
                if mode == 1 and not done[i]:
                    m = max(np.float32(0), m)
                k = s[i] * A + a[i]
                target = np.float32(np.float64(gamma) * np.float64(m) + np.float64(r[i]))  # one rounding
                lists.setdefault(k, []).append(np.float32(lr * np.float32(target - pre[k])))
            want = pre.copy()
            for k, ds in lists.items():
                acc = np.float32(0)
                for d in ds:
                    acc = np.float32(acc + d)
                want[k] = np.float32(pre[k] + acc)
            oracle.td_update_batch(Q, S, A, s, a, r, s2, done, float(lr), float(gamma), mode)
            assert np.array_equal(Q, want)


# ---- eps schedule and the driver loop: training.log ---------------------------

def test_training_log_vector(oracle, pycrl):
    """training.log:24931-24953: mock env (always (0,0), reward -0.01, never done),
    10 episodes x 500 steps, eps0 = 1.0 decaying x0.995 per update."""
    g = load("training_log_vector.json")
    W = H = 10
    cfg = pycrl.make_config(1, W, H, auto_reset=1, episode_len=g["max_steps"], eps_mode=pycrl.EPS_STEP_MULT,
                            eps0=1.0, eps_decay=0.995, eps_span=g["episodes"] * g["max_steps"] + 1, seed=0)
    # the mock env never moves: wall the agent in at (0,0)
    cls = np.full(W * H, 3, np.uint8)
    cls[0] = 0
    tab = oracle.eps_table(cfg)
    Q = np.zeros(W * H * 4, np.float32)
    st = oracle.new_state(cfg, [0])
    for ep in range(g["episodes"]):
        ret = 0.0
        for k in range(g["max_steps"]):
            oracle.run(cfg, cls, None, [0], Q, st, ep * g["max_steps"] + k, 1)
            ret += float(st["reward"][0])
            assert st["done"][0] == 0
        assert "%.2f" % ret == g["episode_return"]
        assert st["episode"][0] == ep + 1 and st["ep_step"][0] == 0
        eps_after = float(tab[(ep + 1) * g["max_steps"]])
        assert "%.3f" % eps_after == g["epsilon_after_episode"][ep]
    # src/train.py:140-141 in Python floats gives the same table
    e, ref = 1.0, []
    for _ in range(len(tab)):
        ref.append(np.float32(e))
        e *= float(np.float32(0.995))
    assert np.array_equal(tab, np.array(ref, np.float32))
    assert np.array_equal(tab, pycrl.eps_table(cfg))
    # evaluation: 1000 steps of -0.01 print as -10.00
    assert "%.2f" % (1000 * float(np.float32(-0.01))) == g["eval_return"]


def test_eps_tables(oracle, pycrl):
    for mode, kw in ((pycrl.EPS_FIXED, dict(eps0=0.1)),
                     (pycrl.EPS_EPISODE_MULT, dict(eps0=1.0, eps_decay=0.995, eps_span=1000)),
                     (pycrl.EPS_EPISODE_LINEAR, dict(eps0=1.0, eps_end=0.05, eps_span=100))):
        cfg = pycrl.make_config(2, 4, 4, eps_mode=mode, **kw)
        assert np.array_equal(oracle.eps_table(cfg), pycrl.eps_table(cfg))
    cfg = pycrl.make_config(2, 4, 4, eps_mode=pycrl.EPS_EPISODE_LINEAR, eps0=1.0, eps_end=0.05, eps_span=100)
    tab = oracle.eps_table(cfg)
    assert len(tab) == 101 and tab[0] == 1.0 and tab[100] == np.float32(0.05)
    assert tab[50] == np.float32(1.0 + (float(np.float32(0.05)) - 1.0) * 0.5)


# ---- the batched loop against a pure-Python restatement ------------------------

def python_loop(cfg, cls, start, n_steps, draws, W, A):
    """src/train.py:198-222 with auto-reset, float32 arithmetic via numpy scalars."""
    f = np.float32
    N, S = cfg.n_envs, cfg.width * cfg.height
    Q = np.zeros((N, S, A), np.float32)
    s = np.array(start).copy()
    ep = np.zeros(N, int)
    trace = []
    dxy = {0: (0, -1), 1: (1, 0), 2: (0, 1), 3: (-1, 0)}
    for k in range(n_steps):
        row_t = []
        for i in range(N):
            u, ar = draws[k][i]
            a = ar if u < cfg.eps0 else int(np.argmax(Q[i, s[i]]))
            x, y = s[i] % W, s[i] // W
            nx, ny = x + dxy[a][0], y + dxy[a][1]
            inb = 0 <= nx < W and 0 <= ny < cfg.height
            c = cls[i][ny * W + nx] if inb else 0
            s2 = ny * W + nx if inb and c < 2 else s[i]
            r, d = f(cfg.step_reward), 0
            if inb and c == 1:
                r, d = f(cfg.goal_reward), 1
            elif inb and c == 2:
                r = f(cfg.trap_reward)
            m = f(0) if d else Q[i, s2].max()
            target = f(np.float64(f(cfg.gamma)) * np.float64(m) + np.float64(r))
            q = Q[i, s[i], a]
            Q[i, s[i], a] = f(np.float64(f(cfg.lr)) * np.float64(f(target - q)) + np.float64(q))
            ep[i] += 1
            row_t.append((s2, a, float(r), d))
            if d or (cfg.episode_len and ep[i] >= cfg.episode_len):
                s[i], ep[i] = start[i], 0
            else:
                s[i] = s2
        trace.append(row_t)
    return Q, trace


def test_run_matches_python_loop(oracle, pycrl):
    W, H, A, N, T = 6, 5, 4, 5, 120
    cls, start = pycrl.gen_maps_bernoulli(42, N, N, W, H, 0.2, 0.1)
    cfg = pycrl.make_config(N, W, H, episode_len=17, eps0=0.3, seed=9, gamma=0.95)
    draws = [[oracle.explore_draw(9, i, t, A) for i in range(N)] for t in range(T)]
    Qp, trp = python_loop(cfg, cls, start, T, draws, W, A)
    Q = np.zeros((N, W * H, A), np.float32)
    st = oracle.new_state(cfg, start)
    tr = oracle.run(cfg, cls, None, start, Q, st, 0, T, trace_n=N)
    for k in range(T):
        for i in range(N):
            assert (tr["s_next"][k, i], tr["action"][k, i], float(tr["reward"][k, i]), tr["done"][k, i]) == trp[k][i]
    assert np.array_equal(Q, Qp)
    assert tr["done"].sum() > 0  # goals were reached, so the restart path ran


def test_run_shared_table_order(oracle, pycrl):
    """Shared table: per-(s,a) sums in env order from the pre-step table (64
    envs: one block, so the tree is left-to-right; larger N in the next test)."""
    W, H, A, N = 4, 4, 4, 64
    cls, start = pycrl.gen_maps_bernoulli(1, 1, N, W, H, 0.1)
    cfg = pycrl.make_config(N, W, H, table_mode=pycrl.TABLE_SHARED, map_mode=pycrl.MAP_SHARED, eps0=0.5,
                            lr=0.05, seed=3)
    rng = np.random.default_rng(0)
    Q = rng.normal(0, 0.1, W * H * A).astype(np.float32)
    pre = Q.copy()
    st = oracle.new_state(cfg, start)
    s_before = st["s"].copy()
    tr = oracle.run(cfg, cls, None, start, Q, st, 0, 1, trace_n=N)
    lists = {}
    for i in range(N):
        a, s2, r, d = int(tr["action"][0, i]), int(tr["s_next"][0, i]), tr["reward"][0, i], tr["done"][0, i]
        m = np.float32(0) if d else pre[s2 * A:(s2 + 1) * A].max()
        target = np.float32(np.float64(np.float32(0.99)) * np.float64(m) + np.float64(r))
        k = int(s_before[i]) * A + a
        lists.setdefault(k, []).append(np.float32(np.float32(0.05) * np.float32(target - pre[k])))
    want = pre.copy()
    for k, ds in lists.items():
        acc = np.float32(0)
        for d in ds:
            acc = np.float32(acc + d)
        want[k] = np.float32(pre[k] + acc)
    assert max(len(v) for v in lists.values()) > 1  # collisions exist
    assert np.array_equal(Q, want)


def test_run_shared_table_uses_the_tree(oracle, pycrl):
    """N > 256: one shared-table step == deltas from the pre-step table pushed
    through the block/group tree."""
    W, H, A, N = 5, 5, 4, 9000
    cls, start = pycrl.gen_maps_bernoulli(2, 1, N, W, H, 0.1)
    cfg = pycrl.make_config(N, W, H, table_mode=pycrl.TABLE_SHARED, map_mode=pycrl.MAP_SHARED, eps0=0.5,
                            lr=0.001, seed=4)
    rng = np.random.default_rng(1)
    Q = rng.normal(0, 0.1, W * H * A).astype(np.float32)
    pre = Q.copy()
    st = oracle.new_state(cfg, start)
    s_before = st["s"].copy()
    tr = oracle.run(cfg, cls, None, start, Q, st, 0, 1, trace_n=N)
    f = np.float32
    key = s_before.astype(np.int64) * A + tr["action"][0]
    d = np.empty(N, np.float32)
    for i in range(N):
        s2 = int(tr["s_next"][0, i])
        m = f(0) if tr["done"][0, i] else pre[s2 * A:(s2 + 1) * A].max()
        target = f(np.float64(f(0.99)) * np.float64(m) + np.float64(tr["reward"][0, i]))
        d[i] = f(f(0.001) * f(target - pre[key[i]]))
    want = (pre + oracle.tree_sum(key, d, W * H * A)).astype(np.float32)
    assert np.array_equal(Q, want)


def test_episode_budget_and_return_accumulators(oracle, pycrl):
    """max_episodes / return tracking (src/train.py:186-226): the accumulators
    equal what the trace says, episode by episode, and an env that has used its
    budget does nothing more."""
    W, H, A, N, T, E = 6, 6, 4, 40, 400, 5
    cls, start = pycrl.gen_maps_bernoulli(77, N, N, W, H, 0.1, 0.05)
    cfg = pycrl.make_config(N, W, H, episode_len=23, eps0=0.4, seed=6, max_episodes=E, track_returns=1)
    Q = np.zeros((N, W * H, A), np.float32)
    st, stats = oracle.new_state(cfg, start), oracle.new_stats(N)
    tr = oracle.run(cfg, cls, None, start, Q, st, 0, T, trace_n=N, stats=stats)
    assert (st["episode"] == E).all()  # everyone finished the budget within T steps
    f = np.float32
    for i in range(N):
        rets, lens, acc, n, k = [], [], f(0), 0, 0
        while len(rets) < E:
            acc = f(acc + tr["reward"][k, i])
            n += 1
            if tr["done"][k, i] or n >= 23:
                rets.append(acc)
                lens.append(n)
                acc, n = f(0), 0
            k += 1
        assert stats["last_return"][i] == rets[-1] and stats["last_length"][i] == lens[-1]
        tot = f(0)
        for r in rets:
            tot = f(tot + r)
        assert stats["return_sum"][i] == tot and stats["length_sum"][i] == sum(lens)
        assert stats["ret_acc"][i] == 0
        # after the budget: idle rows, the env stays on its start cell
        assert (tr["s_next"][k:, i] == start[i]).all() and (tr["reward"][k:, i] == 0).all()
        assert (tr["action"][k:, i] == 0).all() and (tr["done"][k:, i] == 0).all()
    # the frozen steps changed nothing: a run cut at the last active step gives the same tables
    Q2 = np.zeros((N, W * H, A), np.float32)
    st2 = oracle.new_state(cfg, start)
    oracle.run(cfg, cls, None, start, Q2, st2, 0, 2 * T)
    assert np.array_equal(Q, Q2) and np.array_equal(st["s"], st2["s"])
