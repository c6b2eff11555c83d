"""Pins for the oracle's LunarLander: constants algebra, reset invariants, reward/done decision table."""
import ctypes as C
import math

import numpy as np

H, W = 400.0 / 30.0, 20.0
BOD, JNT, EDG, META = 8, 56, 91, 188


def fresh(orc, seed=5, env=0):
    row = np.zeros(192, np.float32)
    orc.orc_ll_reset(row, orc.orc_ll_combined_seed(seed, env))
    return row


def step(orc, row, action, env=0):
    r, d = np.zeros(1, np.float32), np.zeros(1, np.float32)
    contacts = np.zeros(72, np.float32)
    n = C.c_int(0)
    orc.orc_ll_step(row, env, action, r, d, contacts.ctypes.data, C.addressof(n))
    return float(r[0]), float(d[0]), contacts, n.value


def test_reset_invariants(orc):
    row = fresh(orc)
    assert row[90] == 2 and row[187] == 10                    # joint / edge counts
    b = row[BOD:BOD + 39].reshape(3, 13)
    np.testing.assert_allclose(b[0, :3], [10.0, H, 0.0], rtol=1e-7)
    np.testing.assert_allclose(b[1, :2], [10 - 20 / 30, H - 10 / 30 - 18 / 30], rtol=1e-6)
    np.testing.assert_allclose(b[2, :2], [10 + 20 / 30, H - 10 / 30 - 18 / 30], rtol=1e-6)
    assert (np.abs(b[:, 3:5]) <= 4.0).all() and (b[:, 3:5] == b[0, 3:5]).all()
    np.testing.assert_allclose(b[:, 9:12], [[5, .2, .5], [.2, 5, 50], [.2, 5, 50]], rtol=1e-6)
    assert list(b[:, 12]) == [0, 1, 2]
    e = row[EDG:EDG + 60].reshape(10, 6)
    np.testing.assert_allclose(e[:, 0], np.arange(10) * 2.0)
    np.testing.assert_allclose(e[:, 2], np.arange(1, 11) * 2.0)
    np.testing.assert_array_equal(e[:-1, 3], e[1:, 1])         # polyline is continuous
    assert (e[3:7, 1] == np.float32(H / 4)).all() and (e[2:7, 3] == np.float32(H / 4)).all()  # flat helipad
    assert (e[:, 1] >= 0).all() and (e[:, 1] <= H / 2).all()
    np.testing.assert_allclose(np.hypot(e[:, 4], e[:, 5]), 1.0, atol=1e-6)
    j = row[JNT:JNT + 34].reshape(2, 17)
    np.testing.assert_allclose(j[0, :10], [0, 0, 1, -20 / 30, -10 / 30, 0, 8 / 30, 0, 0.4, 0.9], rtol=1e-6)
    np.testing.assert_allclose(j[1, :10], [0, 0, 2, 20 / 30, -10 / 30, 0, 8 / 30, 0, -0.9, -0.4], rtol=1e-6)
    assert (j[:, 12] == 400).all() and (j[:, 13] == 40).all() and (j[:, 14] == 5).all()
    # observation algebra from the constants: y_n = (H - (H/4 + (18/30)/30)) / (H/2)
    y_n = (H - (H / 4 + 18 / 30 / 30)) / (H / 2)
    obs = row[:8]
    np.testing.assert_allclose(obs, [0, y_n, b[0, 3] * 10 / 50, b[0, 4] * (H / 2) / 50, 0, 0, 0, 0],
                               rtol=1e-6, atol=1e-7)
    shaping = -100 * math.hypot(obs[0], obs[1]) - 100 * math.hypot(obs[2], obs[3])
    assert abs(row[META + 2] - shaping) < 1e-3 and row[META] == 0 and row[META + 3] == 0
    # different env / seed -> different terrain and velocity; same -> identical
    assert not np.array_equal(fresh(orc, 5, 1), row) and np.array_equal(fresh(orc, 5, 0), row)
    assert orc.orc_ll_combined_seed(3, 4) == (3 * 2654435761 + 5 * 12345)


def test_gravity_only_noop_steps(orc):
    # the reference's own "gravity only" parity idea: 20 no-op steps, lander in free flight
    row = fresh(orc)
    vy0, y0, vx0 = row[BOD + 4], row[BOD + 1], row[BOD + 3]
    for k in range(1, 21):
        r, d, _, n = step(orc, row, 0)
        assert n == 0 and d == 0.0 and row[META] == k
    # the legs (4% of the mass each) swing in on their springs, so the hull only approximately free-falls
    assert abs(row[BOD + 4] - (vy0 - 10 * 0.02 * 20)) < 0.3
    assert abs(row[BOD + 3] - vx0) < 0.3
    # whole-system linear momentum follows gravity exactly
    m = np.array([5.0, 0.2, 0.2])
    b = row[BOD:BOD + 39].reshape(3, 13)
    np.testing.assert_allclose((m * b[:, 4]).sum() / m.sum(), vy0 - 4.0, atol=2e-3)
    np.testing.assert_allclose((m * b[:, 3]).sum() / m.sum(), vx0, atol=2e-3)
    # joints hold the legs on: anchors coincide to within slop-ish tolerance
    for leg, ax in ((1, -20 / 30), (2, 20 / 30)):
        a = b[0]
        wa = (a[0] + ax * math.cos(a[2]) + 10 / 30 * math.sin(a[2]), a[1] + ax * math.sin(a[2]) - 10 / 30 * math.cos(a[2]))
        l = b[leg]
        wb = (l[0] - 8 / 30 * math.sin(l[2]), l[1] + 8 / 30 * math.cos(l[2]))
        assert math.hypot(wa[0] - wb[0], wa[1] - wb[1]) < 0.02
    # legs end up inside their angular limits
    assert 0.35 < b[1, 2] - b[0, 2] < 0.95 and -0.95 < b[2, 2] - b[0, 2] < -0.35


def test_reward_is_shaping_difference_minus_fuel(orc):
    for action, fuel in ((0, 0.0), (2, 0.30), (1, 0.03), (3, 0.03)):
        row = fresh(orc, 9)
        prev = float(row[META + 2])
        r, d, _, _ = step(orc, row, action)
        o = row[:8]
        sh = (-100 * math.hypot(o[0], o[1]) - 100 * math.hypot(o[2], o[3]) - 100 * abs(o[4])
              + 10 * o[6] + 10 * o[7])
        assert abs(r - (sh - prev - fuel)) < 2e-3 and abs(row[META + 2] - sh) < 1e-3
        np.testing.assert_allclose(o[:2], [(row[BOD] - 10) / 10, (row[BOD + 1] - (H / 4 + 0.02)) / (H / 2)], rtol=1e-5, atol=1e-7)
        np.testing.assert_allclose(o[2:6], [row[BOD + 3] * 10 / 50, row[BOD + 4] * (H / 2) / 50, row[BOD + 2], 20 * row[BOD + 5] / 50], rtol=1e-5, atol=1e-7)


def test_main_engine_pushes_up_side_engines_turn(orc):
    base = fresh(orc, 11)
    rows = {a: base.copy() for a in range(4)}
    for a, row in rows.items():
        step(orc, row, a)
    assert rows[2][BOD + 4] > rows[0][BOD + 4] + 0.2           # main engine: ~13*(4/30)/5 upward
    assert abs((rows[2][BOD + 4] - rows[0][BOD + 4]) - 13 * (4 / 30) / 5) < 0.25
    assert rows[1][BOD + 5] * rows[3][BOD + 5] < 0              # side engines spin opposite ways
    # at angle 0: o_x = -(3 d_y + dir * 12/30) * (-1), impulse_x = -0.6 * o_x, dv_x = impulse_x / 5
    assert abs((rows[1][BOD + 3] - rows[0][BOD + 3]) - (-0.6 * 0.4 / 5)) < 0.02
    assert abs((rows[3][BOD + 3] - rows[0][BOD + 3]) - (+0.6 * 0.4 / 5)) < 0.02


def test_dispersion_stream_depends_on_env_and_step(orc):
    a, b = fresh(orc, 11), fresh(orc, 11)
    step(orc, a, 2, env=0); step(orc, b, 2, env=1)
    assert a[BOD + 3] != b[BOD + 3]
    c = fresh(orc, 11)
    c[META] = 5
    step(orc, c, 2, env=0)
    assert a[BOD + 3] != c[BOD + 3]


def place(orc, x=10.0, y=None, vy=0.0, vx=0.0, angle=0.0):
    """Lander (with legs attached at rest pose) moved rigidly; helipad terrain is flat at H/4."""
    row = fresh(orc, 21)
    b = row[BOD:BOD + 39].reshape(3, 13)
    dy = (y if y is not None else b[0, 1]) - b[0, 1]
    dx = x - b[0, 0]
    b[:, 0] += dx; b[:, 1] += dy
    b[:, 3] = vx; b[:, 4] = vy
    b[0, 2] = angle
    obs0 = np.zeros(8, np.float32)
    return row


def test_termination_table(orc):
    # out of bounds: |x_norm| >= 1 -> reward == -100 exactly, done
    row = place(orc, x=20.5)
    r, d, _, _ = step(orc, row, 0)
    assert (r, d) == (-100.0, 1.0) and row[META + 3] == 1.0
    # done rows are frozen: reward 0, done 1, state untouched
    snap = row.copy()
    r, d, _, _ = step(orc, row, 2)
    assert (r, d) == (0.0, 1.0) and np.array_equal(snap, row)
    # hull touching the ground -> -100
    row = place(orc, y=H / 4 + 0.2, vy=-1.0)
    r, d, c, n = step(orc, row, 0)
    assert n > 0 and 0 in c[:n * 9:9] and (r, d) == (-100.0, 1.0)
    # step limit: the 1000th step ends the episode without touching the reward
    row = fresh(orc, 21); row[META] = 999
    r, d, _, _ = step(orc, row, 0)
    assert d == 1.0 and abs(r) < 50 and row[META] == 1000
    row = fresh(orc, 21); row[META] = 998
    assert step(orc, row, 0)[1] == 0.0


def test_landing_at_rest_bonus(orc):
    # The at-rest branch is exercised with every body made static (inverse mass 0), which the
    # integrator and both solvers leave untouched, standing on the pad with the hull clear of it.
    def standing(vx=0.0, omega=0.0, lift=0.0):
        row = place(orc, y=H / 4 + 1.195 + lift)
        b = row[BOD:BOD + 39].reshape(3, 13)
        b[:, 10:12] = 0.0
        b[0, 3] = vx; b[0, 5] = omega
        return row
    row = standing()
    prev = float(row[META + 2])
    r, d, c, n = step(orc, row, 0)
    o = row[:8]
    assert n > 0 and 0 not in c[:n * 9:9]                   # only leg contacts
    assert o[6] == 1.0 and o[7] == 1.0 and d == 1.0
    sh = -100 * math.hypot(o[0], o[1]) + 20.0
    assert abs(r - (sh - prev + 100.0)) < 1e-3              # bonus is ADDED to the shaping delta
    # moving or spinning at or above the 0.01 thresholds: no bonus, episode continues
    for kw in (dict(vx=0.011), dict(omega=-0.011)):
        row = standing(**kw)
        prev = float(row[META + 2])
        r, d, _, _ = step(orc, row, 0)
        assert d == 0.0 and abs(r - (float(row[META + 2]) - prev)) < 1e-3
    # legs 0.025 above the pad (tolerance is 0.01): no leg contact, no bonus
    row = standing(lift=0.03)
    r, d, _, _ = step(orc, row, 0)
    assert d == 0.0 and row[6] == 0.0


def test_resting_contact_keeps_hull_off_the_ground(orc):
    # drop onto the pad from 1.2 units: legs take the load, the hull never touches, no termination
    row = place(orc, y=H / 4 + 1.4, vy=-0.2)
    for _ in range(300):
        r, d, c, n = step(orc, row, 0)
        assert d == 0.0 and 0 not in c[:n * 9:9]
    assert row[6] == 1.0 and row[7] == 1.0 and row[BOD + 1] > H / 4 + 0.5


def test_batch_matches_single(orc):
    n = 33
    s = np.zeros((n, 192), np.float32)
    orc.orc_ll_reset_batch(s, n, 77)
    singles = np.stack([fresh(orc, 77, i) for i in range(n)])
    np.testing.assert_array_equal(s, singles)
    acts = (np.arange(n) % 4).astype(np.float32)
    r, d, o = np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros((n, 8), np.float32)
    for _ in range(5):
        orc.orc_ll_step_batch(s, acts, r, d, o, n, 4)
        for i in range(n):
            step(orc, singles[i], int(acts[i]), env=i)
    np.testing.assert_array_equal(s, singles)
    np.testing.assert_array_equal(o, s[:, :8])
    dn = np.zeros(n, np.float32); dn[3] = 1
    s2 = s.copy()
    orc.orc_ll_selective_reset_batch(s2, dn, n, 78)
    assert np.array_equal(s2[np.arange(n) != 3], s[np.arange(n) != 3]) and s2[3, META] == 0


# ---------------------------------------------------------------- continuous-action overload

def step_c(orc, row, a0, a1, env=0):
    r, d = np.zeros(1, np.float32), np.zeros(1, np.float32)
    orc.orc_ll_step_continuous(row, env, a0, a1, r, d, None, None)
    return float(r[0]), float(d[0])


def test_continuous_corner_actions_are_the_discrete_actions(orc):
    """Full throttle / full side control / nothing decode to the powers of the four discrete
    actions, so the whole step (state, reward, done) must agree bit for bit -- also beyond the
    clipping range and for several steps in a row."""
    table = {0: (-1.0, 0.0), 2: (1.0, 0.3), 1: (-1.0, -1.0), 3: (-1.0, 1.0)}
    beyond = {0: (-3.0, -0.5), 2: (7.0, 0.5), 1: (-1.5, -4.0), 3: (-2.0, 9.0)}
    for tab in (table, beyond):
        for action, (a0, a1) in tab.items():
            a, b = fresh(orc, 13, env=3), fresh(orc, 13, env=3)
            for _ in range(5):
                ra, da, _, _ = step(orc, a, action, env=3)
                rb, db = step_c(orc, b, a0, a1, env=3)
                assert (ra, da) == (rb, db)
                assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_continuous_powers_scale_the_engine_impulse_and_the_fuel_cost(orc):
    base = fresh(orc, 17)
    vy0 = {}
    # main engine: the velocity change of the hull against the unpowered step is linear in the throttle
    noop = base.copy(); step_c(orc, noop, -1.0, 0.0)
    full = base.copy(); step_c(orc, full, 1.0, 0.0)
    for a0 in (-0.5, 0.0, 0.5):
        p = (a0 + 1.0) / 2.0
        row = base.copy()
        prev = float(row[META + 2])
        r, _ = step_c(orc, row, a0, 0.0)
        for k in (3, 4, 5):
            want = noop[BOD + k] + p * (full[BOD + k] - noop[BOD + k])
            assert abs(row[BOD + k] - want) < 2e-5, (a0, k)
        o = row[:8]
        sh = (-100 * math.hypot(o[0], o[1]) - 100 * math.hypot(o[2], o[3]) - 100 * abs(o[4]) + 10 * o[6] + 10 * o[7])
        assert abs(r - (sh - prev - 0.30 * p)) < 2e-3
    # side engine: dead band up to |a1| = 0.5, then power (|a1| - 0.5) * 2 with the sign as direction
    for a1 in (-0.5, -0.2, 0.0, 0.5):
        row = base.copy(); step_c(orc, row, -1.0, a1)
        assert np.array_equal(row.view(np.uint32), noop.view(np.uint32))
    left = base.copy(); step_c(orc, left, -1.0, -1.0)
    right = base.copy(); step_c(orc, right, -1.0, 1.0)
    for a1, ref in ((-0.75, left), (0.75, right), (0.9, right)):
        s = (abs(a1) - 0.5) * 2.0
        row = base.copy()
        prev = float(row[META + 2])
        r, _ = step_c(orc, row, -1.0, a1)
        for k in (3, 4, 5):
            want = noop[BOD + k] + s * (ref[BOD + k] - noop[BOD + k])
            assert abs(row[BOD + k] - want) < 2e-5, (a1, k)
        o = row[:8]
        sh = (-100 * math.hypot(o[0], o[1]) - 100 * math.hypot(o[2], o[3]) - 100 * abs(o[4]) + 10 * o[6] + 10 * o[7])
        assert abs(r - (sh - prev - 0.03 * s)) < 2e-3
    # both engines at once: the impulses add
    both = base.copy(); step_c(orc, both, 0.0, 0.75)
    half = base.copy(); step_c(orc, half, 0.0, 0.0)
    side = base.copy(); step_c(orc, side, -1.0, 0.75)
    for k in (3, 4, 5):
        assert abs(both[BOD + k] - (half[BOD + k] + side[BOD + k] - noop[BOD + k])) < 2e-5


def test_continuous_batch_matches_single(orc):
    n = 6
    states = np.zeros((n, 192), np.float32)
    orc.orc_ll_reset_batch(states, n, 21)
    singles = states.copy()
    g = np.random.default_rng(2)
    acts = g.uniform(-1.3, 1.3, size=(n, 2)).astype(np.float32)
    rew, don, obs = np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros((n, 8), np.float32)
    orc.orc_ll_step_continuous_batch(states, acts, rew, don, obs, n)
    for i in range(n):
        r, d = step_c(orc, singles[i], float(acts[i, 0]), float(acts[i, 1]), env=i)
        assert r == rew[i] and d == don[i]
    assert np.array_equal(states, singles) and np.array_equal(obs, states[:, :8])


def _engine_delta(angle, u0, u1, m_power, s_power, direction):
    """Velocity change of the lander from the engines, lunar_lander_v2.mojo:1025-1095, in float64
    vector form: the nozzle offset o is built in the lander's frame from the (tip, side) basis, the
    impulse is -power * o, and it acts at o (main engine) or at o + (-17/30 tip_x, 14/30 tip_y) (side)."""
    tip = np.array([math.sin(angle), math.cos(angle)])
    side = np.array([-tip[1], tip[0]])
    d = np.array([(u0 * 2.0 - 1.0) / 30.0, (u1 * 2.0 - 1.0) / 30.0])
    flip = np.array([1.0, -1.0])                 # the reference negates the y component of o
    cross = lambda a, b: a[0] * b[1] - a[1] * b[0]
    dv, dw = np.zeros(2), 0.0
    if m_power > 0:
        o = flip * (tip * (4.0 / 30.0 + 2.0 * d[0]) + side * d[1])
        imp = -o * 13.0 * m_power
        dv += imp / 5.0
        dw += cross(o, imp) / 2.0
    if s_power > 0:
        o = flip * (tip * d[0] + side * (3.0 * d[1] + direction * 12.0 / 30.0))
        imp = -o * 0.6 * s_power
        dv += imp / 5.0
        r = o + np.array([-tip[0] * 17.0 / 30.0, tip[1] * 14.0 / 30.0])
        dw += cross(r, imp) / 2.0
    return dv, dw


def test_engine_impulses_to_1e6_on_a_free_tilted_lander(orc):
    """Engines pinned tightly: with the leg joints removed the lander is a free body, so one step
    leaves it at v0 + dv_engine + g dt exactly.  The uniforms are read back from the oracle's own
    stream (Philox(env + 12345, offset = step_count), elements 0 and 1)."""
    env, step_count, angle = 2, 7, 0.37
    u = np.zeros(4, np.float32)
    orc.orc_philox_uniform4(env + 12345, step_count, 0, u)
    assert 0.05 < abs(2 * u[0] - 1) and 0.05 < abs(2 * u[1] - 1) and abs(u[0] - u[1]) > 0.05   # a swap would show
    def free_lander():
        row = fresh(orc, 9)
        row[90] = 0                                    # joint count: no legs attached
        b = row[BOD:BOD + 39].reshape(3, 13)
        b[0, 2], b[0, 5] = angle, 0.11
        row[META] = step_count
        return row
    base = free_lander()
    v0 = base[BOD + 3:BOD + 6].astype(np.float64).copy()
    x0 = base[BOD:BOD + 3].astype(np.float64).copy()
    cases = [("discrete", 2, (1.0, 0.0, 0.0)), ("discrete", 1, (0.0, 1.0, -1.0)), ("discrete", 3, (0.0, 1.0, 1.0)),
             ("continuous", (0.5, -0.8), (0.75, 0.6, -1.0)), ("continuous", (-0.2, 0.9), (0.4, 0.8, 1.0))]
    for kind, action, (mp, sp, direction) in cases:
        row = free_lander()
        r, d = np.zeros(1, np.float32), np.zeros(1, np.float32)
        if kind == "discrete":
            orc.orc_ll_step(row, env, action, r, d, None, None)
        else:
            orc.orc_ll_step_continuous(row, env, action[0], action[1], r, d, None, None)
        dv, dw = _engine_delta(angle, float(u[0]), float(u[1]), mp, sp, direction)
        want_v = v0[:2] + dv + np.array([0.0, -10.0 * 0.02])
        want_w = v0[2] + dw
        got = row[BOD + 3:BOD + 6].astype(np.float64)
        np.testing.assert_allclose(got[:2], want_v, rtol=0, atol=1e-6, err_msg=str((kind, action)))
        np.testing.assert_allclose(got[2], want_w, rtol=0, atol=1e-6, err_msg=str((kind, action)))
        # semi-implicit Euler: the position moves with the NEW velocity
        np.testing.assert_allclose(row[BOD:BOD + 2], x0[:2] + want_v * 0.02, rtol=0, atol=2e-6)
        np.testing.assert_allclose(row[BOD + 2], x0[2] + want_w * 0.02, rtol=0, atol=1e-6)
        assert np.abs(dv).max() > 0.03                 # the effect is 4 orders above the tolerance


def _twin_step(orc, row, wind, power=15.0, turbulence=1.5, cont=False):
    """One no-op step of a copy of `row` with the wind setting on or off."""
    twin = row.copy()
    orc.orc_ll_set_wind(1 if wind else 0, power, turbulence)
    try:
        if cont:
            step_c(orc, twin, -1.0, 0.0)
        else:
            step(orc, twin, 0)
    finally:
        orc.orc_ll_set_wind(0, 15.0, 1.5)
    return twin


def _momenta(row, about):
    """Linear momentum in x of lander + legs, and their angular momentum about the point `about`."""
    b = row[BOD:BOD + 39].reshape(3, 13).astype(np.float64)
    m, inertia = 1.0 / b[:, 10], 1.0 / b[:, 11]
    x, y = b[:, 0] - about[0], b[:, 1] - about[1]
    return (m * b[:, 3]).sum(), (inertia * b[:, 5] + m * (x * b[:, 4] - y * b[:, 3])).sum()


def _gust(t, power):
    return math.tanh(math.sin(0.02 * t) + math.sin(math.pi * 0.01 * t)) * power


def test_wind_is_an_impulse_on_the_lander_in_free_flight(orc):
    """_apply_wind (lunar_lander_v2.mojo:983-1023): force tanh(sin(0.02 t) + sin(pi 0.01 t)) * WIND_POWER on
    the lander for one DT, torque with TURBULENCE_POWER likewise, t = the row's step count.  The joints
    pass momentum between lander and legs but create none, so the system's momenta show the impulses:
    p_x gains F DT, the angular momentum about a fixed point P gains tau DT - (y_lander - y_P) F DT
    (P = where the centre of mass was before the step, which keeps the terms small in fp32)."""
    for cont in (False, True):
        for t0 in (0, 40, 130, 333):
            row = fresh(orc, 9)
            for _ in range(20):     # the legs are reset a third of a unit below their joints: let them swing in
                step(orc, row, 0)
            row[META] = t0
            b = row[BOD:BOD + 39].reshape(3, 13).astype(np.float64)
            m = 1.0 / b[:, 10]
            P = ((m * b[:, 0]).sum() / m.sum(), (m * b[:, 1]).sum() / m.sum())
            y = float(row[BOD + 1]) - P[1]
            assert 0.01 < y < 0.1       # the legs hang below the lander
            calm, windy = _twin_step(orc, row, False, cont=cont), _twin_step(orc, row, True, cont=cont)
            (p0, l0), (p1, l1) = _momenta(calm, P), _momenta(windy, P)
            f, tau = _gust(t0, 15.0), _gust(t0, 1.5)
            if t0 == 0:     # sin(0) + sin(0): no gust at the first step of an episode
                np.testing.assert_array_equal(calm, windy)
                continue
            assert abs(f) > 4.0
            np.testing.assert_allclose(p1 - p0, f * 0.02, rtol=2e-3)
            np.testing.assert_allclose(l1 - l0, tau * 0.02 - y * f * 0.02, rtol=1e-2)
            # turbulence alone: only the spin changes; wind alone: the spin of the system about its own
            # centre of mass stays (the force acts at the lander's centre, the legs hang symmetrically)
            spin = _twin_step(orc, row, True, power=0.0, turbulence=1.5, cont=cont)
            ps, ls = _momenta(spin, P)
            np.testing.assert_allclose(ps, p0, atol=1e-5)
            np.testing.assert_allclose(ls - l0, tau * 0.02, rtol=1e-2)
            # a stronger wind, same time: the impulse scales with the power
            strong = _twin_step(orc, row, True, power=30.0, turbulence=0.0, cont=cont)
            np.testing.assert_allclose(_momenta(strong, P)[0] - p0, 2 * f * 0.02, rtol=2e-3)


def test_wind_stops_with_a_leg_on_the_ground_and_is_off_by_default(orc):
    row = fresh(orc, 9)
    row[META] = 40
    calm = _twin_step(orc, row, False)
    never_set = row.copy()
    step(orc, never_set, 0)
    np.testing.assert_array_equal(calm, never_set)
    for leg in (6, 7):      # the contact flags of the previous observation gate the wind
        grounded = row.copy()
        grounded[leg] = 1.0
        np.testing.assert_array_equal(_twin_step(orc, grounded, True), _twin_step(orc, grounded, False))
    assert not np.array_equal(_twin_step(orc, row, True), calm)
