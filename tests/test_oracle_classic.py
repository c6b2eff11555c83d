"""Pins for the oracle's CartPole and Pendulum (closed forms evaluated independently in float64)."""
import math

import numpy as np


def cartpole_f64(s, action):
    g, mc, mp, l, fm, tau = 9.8, 1.0, 0.1, 0.5, 10.0, 0.02
    x, xd, th, thd = s
    f = fm if action == 1 else -fm
    c, sn = math.cos(th), math.sin(th)
    temp = (f + mp * l * thd * thd * sn) / (mc + mp)
    tha = (g * sn - c * temp) / (l * (4.0 / 3.0 - mp * c * c / (mc + mp)))
    xa = temp - mp * l * tha * c / (mc + mp)
    return [x + tau * xd, xd + tau * xa, th + tau * thd, thd + tau * tha]


def test_cartpole_one_step_hand_value(orc):
    # From (0, 0, 0.05, 0), push right: Gymnasium CartPole-v1 equations in float64.
    s = np.array([[0.0, 0.0, 0.05, 0.0]], np.float32)
    steps = np.zeros(1, np.int32)
    r, d, o = np.zeros(1, np.float32), np.zeros(1, np.float32), np.zeros((1, 4), np.float32)
    orc.orc_cartpole_step_batch(s, steps, np.array([1.0], np.float32), r, d, o, 1)
    want = cartpole_f64([0.0, 0.0, float(np.float32(0.05)), 0.0], 1)
    np.testing.assert_allclose(s[0], want, rtol=2e-6, atol=1e-8)
    assert s[0, 0] == 0.0  # x advances with the PRE-step velocity
    assert abs(want[1] - 0.19512195) < 1e-3 and r[0] == 1.0 and d[0] == 0.0 and steps[0] == 1
    np.testing.assert_array_equal(o, s)


def test_cartpole_trajectory_and_termination(orc):
    rng = np.random.default_rng(1)
    s = rng.uniform(-0.05, 0.05, (64, 4)).astype(np.float32)
    ref = s.astype(np.float64).tolist()
    steps = np.zeros(64, np.int32)
    r, d, o = np.zeros(64, np.float32), np.zeros(64, np.float32), np.zeros((64, 4), np.float32)
    alive = np.ones(64, bool)
    for t in range(40):
        a = rng.integers(0, 2, 64).astype(np.float32)
        orc.orc_cartpole_step_batch(s, steps, a, r, d, o, 64)
        for i in range(64):
            ref[i] = cartpole_f64(ref[i], int(a[i]))
            if alive[i]:
                np.testing.assert_allclose(s[i], ref[i], rtol=1e-4, atol=1e-5)
                term = abs(ref[i][0]) > 2.4 or abs(ref[i][2]) > 0.2095
                margin = min(abs(abs(ref[i][0]) - 2.4), abs(abs(ref[i][2]) - 0.2095))
                if margin > 1e-4:
                    assert bool(d[i]) == term
                    assert r[i] == (0.0 if term else 1.0)  # CPU path: reward 0 on termination
                if d[i]:
                    alive[i] = False


def test_cartpole_truncates_at_500(orc):
    s = np.zeros((1, 4), np.float32)
    steps = np.array([498], np.int32)
    r, d, o = np.zeros(1, np.float32), np.zeros(1, np.float32), np.zeros((1, 4), np.float32)
    orc.orc_cartpole_step_batch(s, steps, np.array([0.0], np.float32), r, d, o, 1)
    assert d[0] == 0.0
    orc.orc_cartpole_step_batch(s, steps, np.array([1.0], np.float32), r, d, o, 1)
    assert d[0] == 1.0 and r[0] == 1.0 and steps[0] == 500


def test_cartpole_reset_range_and_determinism(orc):
    s1, s2 = np.zeros((256, 4), np.float32), np.zeros((256, 4), np.float32)
    st = np.ones(256, np.int32)
    orc.orc_cartpole_reset_batch(s1, st, 256, 12345)
    orc.orc_cartpole_reset_batch(s2, st, 256, 12345)
    np.testing.assert_array_equal(s1, s2)
    assert (np.abs(s1) <= 0.05 + 1e-7).all() and st.sum() == 0
    assert len(np.unique(s1[:, 0])) > 250
    # independent evaluation of env 3: xorshift32 chain, u = f32(x)/f32(2^32-1), lo + u*(hi-lo)
    M = 0xFFFFFFFF

    def xs(x):
        x ^= (x << 13) & M; x ^= x >> 17; x ^= (x << 5) & M
        return x
    x = xs((3 * 2654435761 + 12345) & M)
    vals = []
    for _ in range(4):
        x = xs(x)
        u = np.float32(x) / np.float32(M)
        vals.append(np.float32(-0.05) + u * (np.float32(0.05) - np.float32(-0.05)))
    np.testing.assert_array_equal(s1[3], np.array(vals, np.float32))


def pendulum_f64(th, thd, a):
    u = max(-2.0, min(2.0, 2.0 * a))
    acc = 3 * 10.0 / 2.0 * math.sin(th) + 3.0 * u
    thd = thd + acc * 0.05
    th = th + thd * 0.05
    thd = max(-8.0, min(8.0, thd))
    while th > math.pi: th -= 2 * math.pi
    while th < -math.pi: th += 2 * math.pi
    return th, thd, -(th * th + 0.1 * thd * thd + 0.001 * u * u), u


def test_pendulum_three_steps_hand_value(orc):
    th0, thd0 = 1.0, 0.5
    s = np.zeros((1, 8), np.float32)
    s[0, :4] = [math.cos(th0), math.sin(th0), thd0, th0]
    r, d, o = np.zeros(1, np.float32), np.zeros(1, np.float32), np.zeros((1, 3), np.float32)
    th, thd, tot = th0, thd0, 0.0
    for k, a in enumerate([0.3, -1.7, 0.9]):
        orc.orc_pendulum_step_batch(s, np.array([a], np.float32), r, d, o, 1)
        th, thd, rew, u = pendulum_f64(th, thd, float(np.float32(a)))
        tot += rew
        np.testing.assert_allclose(s[0], [math.cos(th), math.sin(th), thd, th, k + 1, 0, tot, u],
                                   rtol=3e-6, atol=1e-6)
        np.testing.assert_allclose(r[0], rew, rtol=3e-6)
        np.testing.assert_array_equal(o[0], s[0, :3])
    # order: velocity first, then angle with the NEW velocity, then the clip; reward on post-step theta
    s[0, :4] = [1, 0, 7.9, 0.0]; s[0, 4:] = 0
    orc.orc_pendulum_step_batch(s, np.array([1.0], np.float32), r, d, o, 1)
    assert s[0, 2] == 8.0 and abs(s[0, 3] - (7.9 + 6 * 0.05) * 0.05) < 1e-6


def test_pendulum_wrap_and_truncation(orc):
    s = np.zeros((1, 8), np.float32)
    s[0, :4] = [math.cos(3.1), math.sin(3.1), 8.0, 3.1]
    s[0, 4] = 198
    r, d, o = np.zeros(1, np.float32), np.zeros(1, np.float32), np.zeros((1, 3), np.float32)
    orc.orc_pendulum_step_batch(s, np.array([0.0], np.float32), r, d, o, 1)
    assert -math.pi <= s[0, 3] <= math.pi and s[0, 3] < 0 and d[0] == 0.0
    orc.orc_pendulum_step_batch(s, np.array([0.0], np.float32), r, d, o, 1)
    assert d[0] == 1.0 and s[0, 4] == 200 and s[0, 5] == 1.0


def test_pendulum_reset(orc):
    s = np.ones((512, 8), np.float32)
    orc.orc_pendulum_reset_batch(s, 512, 7)
    th, thd = s[:, 3], s[:, 2]
    assert (np.abs(th) <= math.pi).all() and (np.abs(thd) <= 1).all()
    np.testing.assert_allclose(s[:, 0], np.cos(th.astype(np.float64)), atol=1e-7)
    np.testing.assert_allclose(s[:, 1], np.sin(th.astype(np.float64)), atol=1e-7)
    assert (s[:, 4:] == 0).all() and th.std() > 1.5
    # selective: only done rows change, and their done flag is cleared
    s2 = s.copy()
    dn = np.zeros(512, np.float32); dn[::2] = 1
    orc.orc_pendulum_selective_reset_batch(s2, dn, 512, 8)
    assert (s2[1::2] == s[1::2]).all() and (s2[::2, 3] != s[::2, 3]).all() and dn.sum() == 0
