"""Pins for the oracle's BipedalWalker and HalfCheetah: layout / constants algebra, reset invariants,
reward and termination decision tables, sanity of the dynamics."""
import ctypes as C
import math

import numpy as np

BW_BOD, BW_JNT, BW_EDG, BW_META = 24, 104, 173, 942
HC_BOD, HC_JNT, HC_META = 17, 129, 245
STEP = 14 / 30
TH = 400 / 30 / 4
LEG_H = 34 / 30


def bw_fresh(orc, seed=3, env=0):
    row = np.zeros(950, np.float32)
    orc.orc_bw_reset(row, (seed * 2654435761 + (env + 1) * 12345) & (2**64 - 1))
    return row


def bw_step(orc, row, a):
    r, d = np.zeros(1, np.float32), np.zeros(1, np.float32)
    orc.orc_bw_step(row, np.asarray(a, np.float32), r, d)
    return float(r[0]), float(d[0])


def test_bw_layout_and_reset(orc, orcmod):
    L = orcmod.Layout(); orc.orc_bw_layout(C.byref(L))
    assert (L.bodies_off, L.joints_off, L.edges_off, L.meta_off, L.state_size) == (BW_BOD, BW_JNT, BW_EDG, BW_META, 950)
    row = bw_fresh(orc)
    assert row[940 + 1] == 128 and row[BW_EDG - 1] == 4            # edge_count, joint_count
    e = row[BW_EDG:BW_EDG + 768].reshape(128, 6)
    np.testing.assert_allclose(e[:, 0], np.arange(128, dtype=np.float32) * np.float32(STEP), rtol=1e-6)
    np.testing.assert_array_equal(e[:-1, 2:4], e[1:, 0:2])          # continuous polyline
    np.testing.assert_allclose(np.hypot(e[:, 4], e[:, 5]), 1, atol=1e-6)
    assert (e[:, 5] > 0).all()
    # start pad: the walk is deterministic for the first 21 points (no random term): it descends by
    # the damped 0.01 drift and stays within a few cm of TERRAIN_HEIGHT
    assert np.abs(e[:20, 1] - TH).max() < 0.2 and np.abs(e[:, 1] - TH).max() < 3.0
    v, y = 0.0, np.float32(TH)
    for i in range(3):
        v = np.float32(0.8) * np.float32(v) + np.float32(0.01) * np.float32(1.0 if np.float32(TH) > y else -1.0)
        y = np.float32(y + v)
        assert e[i, 1] == y
    b = row[BW_BOD:BW_BOD + 65].reshape(5, 13)
    iy = TH + 2 * LEG_H
    np.testing.assert_allclose(b[0, :2], [20 * STEP, iy], rtol=1e-6)
    up_y = iy - 8 / 30 - LEG_H / 2
    np.testing.assert_allclose(b[[1, 3], 1], up_y, rtol=1e-6)
    np.testing.assert_allclose(b[[2, 4], 1], up_y - LEG_H, rtol=1e-6)
    np.testing.assert_allclose(b[:, 10], [0.2, 1.25, 2, 1.25, 2], rtol=1e-6)
    np.testing.assert_allclose(b[:, 11], [0.5, 10, 20, 10, 20], rtol=1e-6)
    assert list(b[:, 12]) == [0, 1, 2, 3, 4] and (np.abs(b[:, 3:5]) <= 0.1).all()
    j = row[BW_JNT:BW_JNT + 68].reshape(4, 17)
    assert list(j[:, 1]) == [0, 1, 0, 3] and list(j[:, 2]) == [1, 2, 3, 4] and (j[:, 14] == 3).all()
    np.testing.assert_allclose(j[:, 8:11], [[-0.8, 1.1, 80], [-1.6, -0.1, 80]] * 2, rtol=1e-6)
    # joint anchors coincide at reset: hull anchor (0, LEG_DOWN), upper-leg top, knee
    assert abs((b[0, 1] + j[0, 4]) - (b[1, 1] + j[0, 6])) < 1e-5
    assert abs((b[1, 1] + j[1, 4]) - (b[2, 1] + j[1, 6])) < 1e-5
    # observation: joint angles 0, contacts 0, lidar looking down hits the ground below the hull
    o = row[:24]
    assert o[0] == 0 and (o[4:14:1][[0, 2, 4, 5, 7, 9]] == 0).all()
    np.testing.assert_allclose(o[2:4], [b[0, 3] * 20 / 50, b[0, 4] * (400 / 30) / 50], rtol=1e-5)
    assert abs(o[14] - (iy - TH) / (160 / 30)) < 0.05            # ray 0 points straight down
    assert (o[14:24] > 0.3).all() and (np.diff(o[14:24]) > -1e-3).all()   # shallower rays travel further
    assert abs(row[BW_META + 2] - 130 * b[0, 0] / 30) < 1e-4


def test_bw_motors_and_reward_terms(orc):
    row = bw_fresh(orc)
    prev = float(row[BW_META + 2])
    a = [0.5, -2.0, -0.25, 1.0]
    x0 = float(row[BW_BOD])
    r, d = bw_step(orc, row, a)
    j = row[BW_JNT:BW_JNT + 68].reshape(4, 17)
    np.testing.assert_allclose(j[:, 11], [4, -6, -4, 6])           # sign(a) * (hip 4 | knee 6)
    np.testing.assert_allclose(j[:, 10], [40, 80, 20, 80])         # 80 * |clamp(a)|
    hull = row[BW_BOD:BW_BOD + 6]
    sh = 130 * hull[0] / 30
    vel = float(row[2])
    want = (sh - prev) - 5 * abs(hull[2]) - 0.00035 * 80 * (0.5 + 2.0 + 0.25 + 1.0)   # raw |a| in the energy term
    want += 3 * vel if vel > 0 else -5 * abs(vel)
    assert hull[1] > TH + 1.5 * LEG_H and d == 0.0
    assert abs(r - want) < 2e-4
    assert row[BW_META] == 1 and abs(row[BW_META + 4] - (hull[0] - 4.0)) < 1e-5


def test_bw_termination_table(orc):
    crit, minh = TH + 1.2 * LEG_H, TH + 1.5 * LEG_H
    # frozen (static) bodies make the physics a no-op so each branch can be set up exactly
    def frozen(y=None, x=None, game_over=0.0, steps=0):
        row = bw_fresh(orc)
        b = row[BW_BOD:BW_BOD + 65].reshape(5, 13)
        b[:, 10:12] = 0; b[:, 3:6] = 0
        if y is not None: b[:, 1] += y - b[0, 1]
        if x is not None: b[:, 0] += x - b[0, 0]
        row[BW_META + 7] = game_over; row[BW_META] = steps
        row[BW_META + 2] = np.float32(130.0 * float(b[0, 0]) / 30.0)
        return row
    r, d = bw_step(orc, frozen(), [0, 0, 0, 0]); assert d == 0 and abs(r) < 1e-5
    r, d = bw_step(orc, frozen(y=(crit + minh) / 2), [0, 0, 0, 0])
    assert d == 0 and abs(r + 10 * (minh - (crit + minh) / 2)) < 1e-4        # height penalty only
    r, d = bw_step(orc, frozen(y=crit - 0.3), [0, 0, 0, 0]); assert (r, d) == (-50.0, 1.0)
    r, d = bw_step(orc, frozen(y=crit - 0.3, game_over=1.0), [0, 0, 0, 0]); assert (r, d) == (-100.0, 1.0)
    r, d = bw_step(orc, frozen(x=-0.5), [0, 0, 0, 0]); assert (r, d) == (-100.0, 1.0)
    r, d = bw_step(orc, frozen(x=190 * STEP + 0.1), [0, 0, 0, 0]); assert d == 1.0 and abs(r) < 1e-3
    r, d = bw_step(orc, frozen(steps=1999), [0, 0, 0, 0]); assert d == 1.0
    r, d = bw_step(orc, frozen(steps=1998), [0, 0, 0, 0]); assert d == 0.0


def test_bw_falls_and_touches_down(orc):
    row = bw_fresh(orc)
    saw_leg, done = False, 0.0
    for t in range(200):
        r, done = bw_step(orc, row, [0, 0, 0, 0])
        saw_leg |= bool(row[BW_META + 5] or row[BW_META + 6])
        if done:
            break
    assert saw_leg                    # legs reach the ground
    assert done == 1.0 and r in (-100.0, -50.0)   # an unactuated walker collapses
    assert row[8] in (0.0, 1.0) and row[13] in (0.0, 1.0)


def hc_fresh(orc, seed=3, env=0):
    row = np.zeros(253, np.float32)
    orc.orc_hc_reset(row, (seed * 2654435761 + (env + 1) * 12345) & (2**64 - 1))
    return row


def hc_step(orc, row, a):
    r, d = np.zeros(1, np.float32), np.zeros(1, np.float32)
    orc.orc_hc_step(row, np.asarray(a, np.float32), r, d)
    return float(r[0]), float(d[0])


def test_hc_reset(orc, orcmod):
    L = orcmod.Layout(); orc.orc_hc_layout(C.byref(L))
    assert (L.bodies_off, L.joints_off, L.meta_off, L.state_size) == (HC_BOD, HC_JNT, HC_META, 253)
    row = hc_fresh(orc)
    b = row[HC_BOD:HC_BOD + 91].reshape(7, 13)
    lens = [1.0, 0.145, 0.15, 0.094, 0.133, 0.106, 0.07]
    np.testing.assert_allclose(b[:, 0], [0, -.5, -.5, -.5, .5, .5, .5], atol=1e-7)
    np.testing.assert_allclose(b[:, 1], [0.7, 0.7 - .0725, 0.7 - .145 - .075, 0.7 - .295 - .047,
                                         0.7 - .0665, 0.7 - .133 - .053, 0.7 - .239 - .035], rtol=1e-6)
    np.testing.assert_allclose(b[:, 10], [1 / 6.25] + [1] * 6, rtol=1e-6)
    np.testing.assert_allclose(b[:, 11], [12 / (m * l * l) for m, l in zip([6.25] + [1] * 6, lens)], rtol=1e-6)
    j = row[HC_JNT:HC_JNT + 102].reshape(6, 17)
    assert list(j[:, 1]) == [0, 1, 2, 0, 4, 5] and list(j[:, 2]) == [1, 2, 3, 4, 5, 6] and (j[:, 14] == 3).all()
    for k in range(6):                                   # anchors coincide in the rest pose
        a, bb = b[int(j[k, 1])], b[int(j[k, 2])]
        assert abs((a[0] + j[k, 3]) - (bb[0] + j[k, 5])) < 1e-6 and abs((a[1] + j[k, 4]) - (bb[1] + j[k, 6])) < 1e-6
    o = row[:17]
    np.testing.assert_allclose(o[:2], [0.7, 0]); assert (o[2:8] == 0).all() and (o[10:] == 0).all()
    np.testing.assert_array_equal(o[8:10], b[0, 3:5])
    assert row[HC_META] == 0 and row[HC_META + 1] == 0 and row[253 - 8 - 1] == 0 and row[HC_JNT + 102] == 6


def test_hc_reward_terms_and_obs(orc):
    row = hc_fresh(orc)
    a = [0.3, -1.7, 0.0, 1.0, -0.2, 0.6]
    x0 = float(row[HC_BOD])
    r, d = hc_step(orc, row, a)
    b = row[HC_BOD:HC_BOD + 91].reshape(7, 13)
    ac = np.clip(a, -1, 1)
    j = row[HC_JNT:HC_JNT + 102].reshape(6, 17)
    np.testing.assert_allclose(j[:, 11], np.where(ac >= 0, 1000.0, -1000.0))
    np.testing.assert_allclose(j[:, 10], np.abs(ac), rtol=1e-6)
    want = (float(b[0, 0]) - x0) / 0.05 - 0.1 * float((ac ** 2).sum()) + min(float(b[0, 1]), 0.5)
    assert abs(r - want) < 1e-4 and d == 0.0                  # in the air: no contact penalty
    o = row[:17]
    np.testing.assert_allclose(o[2:8], [b[1, 2] - b[0, 2], b[2, 2] - b[1, 2], b[3, 2] - b[2, 2],
                                        b[4, 2] - b[0, 2], b[5, 2] - b[4, 2], b[6, 2] - b[5, 2]], atol=1e-6)
    np.testing.assert_allclose(o[11:17], [b[1, 5] - b[0, 5], b[2, 5] - b[1, 5], b[3, 5] - b[2, 5],
                                          b[4, 5] - b[0, 5], b[5, 5] - b[4, 5], b[6, 5] - b[5, 5]], atol=1e-5)
    assert row[HC_META] == 1 and abs(row[HC_META + 1] - b[0, 0]) < 1e-7
    # five sub-steps of dt = 0.01 under g = -9.81 while airborne: system momentum check
    m = np.array([6.25, 1, 1, 1, 1, 1, 1.0])
    row2 = hc_fresh(orc); vy0 = float(row2[HC_BOD + 4])
    hc_step(orc, row2, [0] * 6)
    b2 = row2[HC_BOD:HC_BOD + 91].reshape(7, 13)
    assert abs((m * b2[:, 4]).sum() / m.sum() - (vy0 - 9.81 * 0.05)) < 2e-3


def test_hc_lands_on_feet_and_penalty(orc):
    row = hc_fresh(orc)
    pen_seen = False
    for t in range(120):
        x0 = float(row[HC_BOD])
        r, d = hc_step(orc, row, [0] * 6)
        b = row[HC_BOD:HC_BOD + 91].reshape(7, 13)
        base = (float(b[0, 0]) - x0) / 0.05 + (min(float(b[0, 1]), 0.5) if b[0, 1] > 0.1 else 0.0)
        k = round((base - r) / 0.5)
        assert abs((base - r) - 0.5 * k) < 2e-3 and k >= 0        # penalty = 0.5 * (# non-foot contacts)
        pen_seen |= k > 0
        assert d == 0.0
    assert b[:, 1].min() > -0.06                                  # nothing sinks through the floor
    row[HC_META] = 999
    assert hc_step(orc, row, [0] * 6)[1] == 1.0                   # time limit at 1000 steps


def test_batch_wrappers(orc):
    n = 9
    s = np.zeros((n, 950), np.float32); orc.orc_bw_reset_batch(s, None, n, 5)
    np.testing.assert_array_equal(s[4], bw_fresh(orc, 5, 4))
    acts = np.random.default_rng(0).uniform(-1, 1, (n, 4)).astype(np.float32)
    r, d, o = np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros((n, 24), np.float32)
    one = s[2].copy(); orc.orc_bw_step_batch(s, acts, r, d, o, n, 2)
    r1, d1 = bw_step(orc, one, acts[2])
    np.testing.assert_array_equal(s[2], one); assert r[2] == np.float32(r1)
    np.testing.assert_array_equal(o, s[:, :24])
    h = np.zeros((n, 253), np.float32); orc.orc_hc_reset_batch(h, None, n, 5)
    np.testing.assert_array_equal(h[7], hc_fresh(orc, 5, 7))
    dn = np.zeros(n, np.float32); dn[1] = 1
    h2 = h.copy(); orc.orc_hc_reset_batch(h2, dn.ctypes.data, n, 6)
    assert not np.array_equal(h2[1], h[1]) and np.array_equal(h2[0], h[0])


def test_bw_terrain_recurrence_over_all_edges(orc):
    """bipedal_walker_v2.mojo:395-466: y_i from the damped random walk, one Philox draw per point past
    the start pad (stream seed + 1000, successive step_uniform calls, element 0), all 128 edges kept."""
    for seed, env in ((3, 0), (11, 7)):
        cseed = (seed * 2654435761 + (env + 1) * 12345) & (2**64 - 1)
        row = np.zeros(950, np.float32)
        orc.orc_bw_reset(row, cseed)
        e = row[BW_EDG:BW_EDG + 768].reshape(128, 6)
        f = np.float32
        y, v, ys, u = f(TH), f(0.0), [], np.zeros(4, np.float32)
        for i in range(129):
            v = f(0.8) * v + f(0.01) * (f(1.0) if f(TH) > y else f(-1.0))
            if i > 20:
                orc.orc_philox_uniform4((cseed + 1000) & (2**64 - 1), 0, i - 21, u)
                v = v + (f(u[0]) * f(2.0) - f(1.0)) / f(30.0)
            y = f(y + v)
            ys.append(y)
        ys = np.array(ys, np.float32)
        np.testing.assert_array_equal(e[:, 1], ys[:128])
        np.testing.assert_array_equal(e[:, 3], ys[1:129])
        x = np.arange(129, dtype=np.float32) * np.float32(14.0 / 30.0)
        np.testing.assert_array_equal(e[:, 0], x[:128])
        np.testing.assert_array_equal(e[:, 2], x[1:])
        # unit normals, turned upwards, perpendicular to the edge
        dx, dy = e[:, 2] - e[:, 0], e[:, 3] - e[:, 1]
        ln = np.sqrt(dx * dx + dy * dy)
        np.testing.assert_array_equal(e[:, 4], -dy / ln)
        np.testing.assert_array_equal(e[:, 5], dx / ln)
        assert np.ptp(ys[21:]) > 0.05            # the random term is there


def test_hc_joint_limits_and_motor_constants(orc):
    """half_cheetah/constants.mojo:103-120 (limits), :83-89 (topology): back thigh / shin / foot,
    front thigh / shin / foot."""
    row = hc_fresh(orc)
    j = row[HC_JNT:HC_JNT + 102].reshape(6, 17)
    limits = [(-0.52, 1.05), (-0.785, 0.785), (-0.4, 0.785), (-1.0, 0.7), (-1.2, 0.87), (-0.5, 0.5)]
    np.testing.assert_array_equal(j[:, 8], np.array([l for l, _ in limits], np.float32))
    np.testing.assert_array_equal(j[:, 9], np.array([h for _, h in limits], np.float32))
    assert (j[:, 7] == 0).all()                                   # reference angle: rest pose
    # a joint pushed past its upper limit is brought back by the position solve, one inside is left alone
    b = row[HC_BOD:HC_BOD + 91].reshape(7, 13)
    for k, (lo, hi) in enumerate(limits):
        r2 = row.copy()
        b2 = r2[HC_BOD:HC_BOD + 91].reshape(7, 13)
        child = int(j[k, 2])
        b2[child, 2] = hi + 0.3
        rel0 = b2[child, 2] - b2[int(j[k, 1]), 2]
        hc_step(orc, r2, [0.0] * 6)
        rel1 = b2[child, 2] - b2[int(j[k, 1]), 2]
        assert rel1 < rel0 - 0.05, (k, rel0, rel1)
