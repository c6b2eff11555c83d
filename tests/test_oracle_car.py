"""Pins for the oracle's CarRacingV2: tile geometry against an independent point-in-polygon test,
the tyre model against closed forms and invariants, the track generator's recurrence, reward and
termination decision table."""
import math

import numpy as np

S, OBS, HULL, WHEELS, CTRL, META, TRACK, VISITED = 3040, 13, 13, 19, 31, 34, 40, 2740
SIZE = 0.02
DT = np.float32(0.02)


def fresh(orc, seed=3, env=0):
    row = np.zeros(S, np.float32)
    orc.orc_cr_reset(row, orc.orc_cr_combined_seed(seed, env))
    return row


def step(orc, row, a):
    r, d = np.zeros(1, np.float32), np.zeros(1, np.float32)
    orc.orc_cr_step(row, np.asarray(a, np.float32), r, d)
    return float(r[0]), float(d[0])


def tiles(row):
    n = int(row[META + 5])
    return row[TRACK:TRACK + 9 * n].reshape(n, 9), n


def test_reset_and_track(orc):
    """car_racing_v2.mojo:1155-1485: 12 checkpoints on a noisy circle of radius 75 .. 150, a pen that
    turns by at most 0.31 rad per 3.5-unit stroke towards the next checkpoint, a tile of width 40/6 per
    stroke; the car starts on the middle of tile 0's first edge, at rest."""
    assert orc.orc_cr_combined_seed(7, 5) == 7 * 2654435761 + 5 * 12345
    seen = set()
    for seed, env in ((3, 0), (3, 1), (11, 40)):
        row = fresh(orc, seed, env)
        T, n = tiles(row)
        seen.add(n)
        assert 100 < n <= 299 and (row[TRACK + 9 * n:VISITED] == 0).all() and (row[VISITED:] == 0).all()
        assert (T[:, 8] == 1.0).all()
        # consecutive strokes: tile i ends where tile i + 1 begins (mid-points of the shared edge), length 3.5
        mid_in = (T[:, 0:2] + T[:, 6:8]) / 2
        mid_out = (T[:, 2:4] + T[:, 4:6]) / 2
        np.testing.assert_allclose(mid_out[:-1], mid_in[1:], atol=2e-4)
        np.testing.assert_allclose(np.hypot(*(mid_out - mid_in).T), 21.0 / 6.0, rtol=2e-5)
        # width 40/6 across the stroke direction, heading change per stroke at most the turn rate
        np.testing.assert_allclose(np.hypot(*(T[:, 4:6] - T[:, 2:4]).T), 40.0 / 6.0, rtol=2e-5)
        d = mid_out - mid_in
        beta = np.unwrap(np.arctan2(d[:, 1], d[:, 0]))
        assert np.abs(np.diff(beta)).max() <= 0.31 + 1e-4
        # the pen starts at (150, 0) heading up and goes once round the origin, anticlockwise
        np.testing.assert_allclose(mid_in[0], [150.0, 0.0], atol=1e-4)
        assert 4.0 < beta[-1] - beta[0] < 8.5          # it stops within 45 units of checkpoint 0, short of closing the loop
        rad = np.hypot(*mid_out.T)
        assert 30.0 < rad.min() and rad.max() < 175.0       # checkpoints at radius 75 .. 150, corners cut by up to 45
        # first stroke from the oracle's own uniforms: checkpoint 1 at angle 2 pi / 12 + noise, radius
        # 150 (0.5 + u1 / 2); the first turn is +-0.31 towards it (or the exact difference when small)
        u = np.zeros(4, np.float32)
        orc.orc_philox_uniform4(orc.orc_cr_combined_seed(seed, env), 0, 1, u)
        alpha = 2 * math.pi / 12 + (float(u[0]) - 0.5) * 2 * math.pi / 12 * 0.5
        c1 = 150.0 * (0.5 + float(u[1]) * 0.5) * np.array([math.cos(alpha), math.sin(alpha)])
        want = math.atan2(c1[1] - 0.0, c1[0] - 150.0)          # the generator's series arctangent is clamped:
        diff = (want - math.pi / 2 + math.pi) % (2 * math.pi) - math.pi
        assert abs(beta[0] - (math.pi / 2 + math.copysign(0.31, diff))) < 1e-4 or abs(diff) < 0.8
        # start pose: middle of tile 0's first edge, observation = pose, everything else zero
        np.testing.assert_allclose(row[HULL:HULL + 3], [(T[0, 0] + T[0, 6]) / 2, (T[0, 1] + T[0, 7]) / 2, row[2]], rtol=1e-6)
        np.testing.assert_array_equal(row[:3], row[HULL:HULL + 3])
        assert (row[3:HULL] == 0).all() and (row[HULL + 3:META + 5] == 0).all()
        assert row[META + 5] == n
    assert len(seen) > 1                     # different seeds, different tracks
    assert np.array_equal(fresh(orc, 3, 0), fresh(orc, 3, 0))


def test_tile_lookup_against_independent_point_in_polygon(orc):
    """tile_collision.mojo:52-90, :232-262: first tile in list order that holds the point."""
    row = fresh(orc, 5, 2)
    T, n = tiles(row)
    rng = np.random.default_rng(0)
    centre = T[:, :8].reshape(n, 4, 2).mean(1)
    pts = centre[rng.integers(0, n, 400)] + rng.normal(0, 3.0, (400, 2))

    def inside(p, quad):                      # winding by signed areas, float64
        q = quad.astype(np.float64)
        s = [(q[(k + 1) % 4, 0] - q[k, 0]) * (p[1] - q[k, 1]) - (q[(k + 1) % 4, 1] - q[k, 1]) * (p[0] - q[k, 0]) for k in range(4)]
        return min(s), max(s)
    checked = hits = 0
    for p in pts.astype(np.float32):
        got = orc.orc_cr_tile_at(row, float(p[0]), float(p[1]), n)
        first, clear = -1, True
        for i in range(n):
            lo, hi = inside(p.astype(np.float64), T[i, :8].reshape(4, 2))
            if min(abs(lo), abs(hi)) < 1e-3:
                clear = False                 # within rounding of an edge: either answer is fine
                break
            if lo > 0 or hi < 0:
                first = i
                break
        if clear:
            assert got == first
            checked += 1; hits += first >= 0
    assert checked > 300 and 50 < hits < checked - 20


def _car(orc, vx=0.0, vy=0.0, omega=0.0, angle=0.0, wheel_omega=0.0, on_road=True):
    """A car on a hand-made track: one big road tile around the origin (or none)."""
    row = np.zeros(S, np.float32)
    row[META + 5] = 50                       # 49 specks far away keep the lap fraction low
    for k in range(50):
        row[TRACK + 9 * k:TRACK + 9 * k + 9] = [900 + k, 900, 900.5 + k, 900, 900.5 + k, 900.5, 900 + k, 900.5, 1.0]
    if on_road:
        row[TRACK:TRACK + 9] = [-50, -50, 50, -50, 50, 50, -50, 50, 1.0]
    row[HULL:HULL + 6] = [0, 0, angle, vx, vy, omega]
    for w in range(4):
        row[WHEELS + 3 * w] = wheel_omega
    return row


def test_steering_joint_follows_the_input(orc):
    """car_dynamics.mojo:68-150: target 0.4 * input, rate min(50 * error, 3) rad/s, limit +-0.4."""
    row = _car(orc)
    angles = []
    for _ in range(12):
        step(orc, row, [1.0, -1.0, -1.0])
        angles.append(float(row[WHEELS + 1]))
    want, a = [], np.float32(0.0)
    for _ in range(12):
        speed = min((np.float32(0.4) - a) * np.float32(50.0), np.float32(3.0))
        a = min(np.float32(a + speed * DT), np.float32(0.4))
        want.append(float(a))
    np.testing.assert_allclose(angles, want, rtol=0, atol=1e-7)
    assert angles[0] == float(np.float32(3.0) * DT) and abs(angles[-1] - 0.4) < 1e-6
    assert row[WHEELS + 1] == row[WHEELS + 4] and row[WHEELS + 7] == 0 and row[WHEELS + 10] == 0   # front pair only
    assert row[6] == row[WHEELS + 1] and row[7] == row[WHEELS + 4]


def test_tyre_model_single_step_closed_form(orc):
    """wheel_friction.mojo:100-215 for a car at rest, full gas, no brake, heading up (angle 0): the rear
    wheels spin up by dt * P / (I * 5), the slip force (-vf + omega r) * 82 exceeds the road limit 400
    and is cut to it, both rear wheels push forward (+y), the torques cancel."""
    row = _car(orc)
    r, d = step(orc, row, [0.0, 1.0, -1.0])
    P, I, R, K = 1e8 * SIZE * SIZE, 4000 * SIZE * SIZE, 27 * SIZE, 205000 * SIZE * SIZE
    spin = 0.02 * P / (I * 5.0)
    f = min(spin * R * K, 400.0)
    assert spin * R * K > 400.0
    omega_after = spin - 0.02 * f * R / I
    np.testing.assert_allclose(row[WHEELS + 6], omega_after, rtol=1e-6)
    np.testing.assert_allclose(row[WHEELS + 9], omega_after, rtol=1e-6)
    assert row[WHEELS + 0] == 0 and row[WHEELS + 3] == 0                       # front wheels: no engine, no slip
    vy = 2 * f / 10.0 * 0.02
    np.testing.assert_allclose(row[HULL + 4], vy, rtol=1e-6)
    np.testing.assert_allclose(row[HULL + 1], vy * 0.02, rtol=1e-6)           # semi-implicit: moves with the new velocity
    assert abs(row[HULL + 3]) < 1e-6 and abs(row[HULL + 5]) < 1e-6 and abs(row[HULL + 0]) < 1e-7
    np.testing.assert_allclose(row[12], vy, rtol=1e-6)                         # speed entry of the observation
    np.testing.assert_allclose(row[WHEELS + 8], omega_after * 0.02, rtol=1e-6)  # wheel phase integrates the spin
    # on grass the limit is 0.6 * 400
    g = _car(orc, on_road=False)
    step(orc, g, [0.0, 1.0, -1.0])
    np.testing.assert_allclose(g[HULL + 4], 2 * 240.0 / 10.0 * 0.02, rtol=1e-6)


def test_tyre_model_sideways_slide_and_brake(orc):
    """A car sliding sideways (vx along its lateral axis) is slowed by all four tyres, each force cut to
    the limit; the full brake zeroes the wheel spin, a partial brake takes 15 * brake off it."""
    row = _car(orc, vx=10.0, wheel_omega=3.0)
    step(orc, row, [0.0, -1.0, 1.0])                         # brake = 1 >= 0.9: wheels stop dead
    # lateral slip 10 * 82 = 820 > 400 per wheel; forward slip (0 - 0) = 0 after the brake
    np.testing.assert_allclose(row[HULL + 3], 10.0 - 4 * 400.0 / 10.0 * 0.02, rtol=1e-6)
    assert all(row[WHEELS + 3 * w] == 0 for w in range(4))
    row = _car(orc, wheel_omega=30.0)
    step(orc, row, [0.0, -1.0, 0.0])                         # brake 0.5: spin drops by 7.5, then friction acts
    w0 = 30.0 - 15.0 * 0.5
    f = min(w0 * 27 * SIZE * 82.0, 400.0)
    np.testing.assert_allclose(row[WHEELS + 0], w0 - 0.02 * f * 27 * SIZE / 1.6, rtol=1e-6)
    # forces never exceed the limit: total push <= 4 * 400
    assert abs(row[HULL + 4]) <= 4 * 400.0 / 10.0 * 0.02 * (1 + 1e-6)


def test_front_wheels_take_the_steering_input_as_their_angle(orc):
    """wheel_friction.mojo:268-281 passes the steering INPUT (not the joint angle) to the front tyres:
    a car rolling straight ahead with input 1.0 feels front tyres turned by 1 rad at once."""
    roll = 5.0 / (27 * SIZE)                                 # wheels rolling without slip at 5 units / s
    row = _car(orc, vy=5.0, wheel_omega=roll)
    step(orc, row, [1.0, -1.0, -1.0])
    assert abs(row[WHEELS + 1] - 0.06) < 1e-6                # the joint itself has only moved 3 rad/s * dt
    # front tyres at 1 rad to the motion: forward slip (5 - 5 cos 1) * 82, lateral slip -5 sin 1 * 82,
    # cut to 400 in all if above; rear tyres roll freely.  Force per front tyre in the world frame:
    f, p = (5.0 - 5.0 * math.cos(1.0)) * 82.0, -5.0 * math.sin(1.0) * 82.0
    scale = min(1.0, 400.0 / math.hypot(f, p))
    fx = (p * math.cos(1.0) + f * -math.sin(1.0)) * scale
    fy = (p * math.sin(1.0) + f * math.cos(1.0)) * scale
    np.testing.assert_allclose(row[HULL + 3], 2 * fx / 10.0 * 0.02, rtol=1e-5)
    np.testing.assert_allclose(row[HULL + 4], 5.0 + 2 * fy / 10.0 * 0.02, rtol=1e-6)
    np.testing.assert_allclose(row[HULL + 5], -2 * 1.6 * fx / 10.0 * 0.02, rtol=1e-5)   # torque = sum(wx fy - wy fx), wy = 1.6
    assert fx < -100 and row[HULL + 5] > 0.5                 # turns left at once
    straight = _car(orc, vy=5.0, wheel_omega=roll)
    step(orc, straight, [0.0, -1.0, -1.0])
    assert abs(straight[HULL + 5]) < 1e-4 and abs(straight[HULL + 3]) < 1e-4


def test_reward_and_termination_table(orc):
    """car_racing_v2.mojo:781-846: -0.1 per step, + 100 / tiles for a tile not seen before, once;
    -100 and done off the playfield; done at 95 % of the tiles; done + truncated at 500 steps;
    a done row returns (0, 1) untouched."""
    row = fresh(orc, 3, 0)
    T, n = tiles(row)
    r, d = step(orc, row, [0, -1, -1])
    assert d == 0 and row[VISITED] == 1 and row[META + 4] == 1
    np.testing.assert_allclose(r, -0.1 + 100.0 / n, rtol=1e-6)
    r, d = step(orc, row, [0, -1, -1])
    np.testing.assert_allclose(r, -0.1, rtol=1e-6)           # same tile again
    np.testing.assert_allclose(row[META + 1], 2 * -0.1 + 100.0 / n, rtol=1e-5)
    assert row[META + 0] == 2
    # off the playfield (2000 / 6)
    out = fresh(orc, 3, 0); out[HULL] = 334.0
    r, d = step(orc, out, [0, -1, -1])
    assert (r, d) == (-100.0, 1.0) and out[META + 2] == 1
    before = out.copy()
    assert step(orc, out, [1, 1, 1]) == (0.0, 1.0) and np.array_equal(out, before)
    inside = fresh(orc, 3, 0); inside[HULL] = 333.0; inside[HULL + 1] = -333.0
    assert step(orc, inside, [0, -1, -1])[1] == 0.0
    # lap complete: tiles_visited / n >= 0.95
    lap = fresh(orc, 3, 0)
    need = math.ceil(0.95 * n)
    lap[META + 4] = need - 1
    r, d = step(orc, lap, [0, -1, -1])
    assert d == 1.0 and lap[META + 4] == need and lap[META + 3] == 0
    np.testing.assert_allclose(r, -0.1 + 100.0 / n, rtol=1e-6)
    # step limit
    late = fresh(orc, 3, 0); late[META + 0] = 498
    assert step(orc, late, [0, -1, -1])[1] == 0.0
    r, d = step(orc, late, [0, -1, -1])
    assert d == 1.0 and late[META + 3] == 1 and late[META + 0] == 500
    # action decoding: gas and brake map [-1, 1] to [0, 1], clamped
    c = fresh(orc, 3, 0)
    step(orc, c, [1.7, 0.5, -3.0])
    np.testing.assert_array_equal(c[CTRL:CTRL + 3], np.float32([1.0, 0.75, 0.0]))


def test_driving_round_the_track_collects_tiles(orc):
    """A follow-the-next-tile controller on the oracle visits tiles in order and earns 100 / n each."""
    row = fresh(orc, 4, 3)
    T, n = tiles(row)
    centre = T[:, :8].reshape(n, 4, 2).mean(1)
    total, visited_order = 0.0, []
    for t in range(400):
        x, y, ang = row[HULL:HULL + 3]
        nxt = int(row[META + 4]) + 3
        tx, ty = centre[min(nxt, n - 1)]
        want = math.atan2(ty - y, tx - x) - math.pi / 2          # the car's forward axis is its +y
        err = (want - ang + math.pi) % (2 * math.pi) - math.pi
        speed = row[12]
        r, d = step(orc, row, [float(np.clip(-err * 2.0, -1, 1)) * -1.0, 0.2 if speed < 12 else -1.0, -1.0])
        total += r
        if d:
            break
    seen = int(row[META + 4])
    flags = row[VISITED:VISITED + n]
    assert seen > 20 and flags.sum() == seen and flags[:seen].sum() >= seen - 4      # in order, a tile or two skipped
    np.testing.assert_allclose(total, -0.1 * row[META + 0] + seen * 100.0 / n, rtol=1e-4)


def test_trait_step_form_reward_and_termination(orc):
    """orc_cr_set_step_form(1) = the GPU trait's step_kernel_gpu (car_racing_v2.mojo:1556-1716), pinned
    against the CPU form and against the formula evaluated independently in float64:
    the row after a step is the CPU form's except for the episode total (same dynamics, controls,
    visited flags, observation); reward = 0.5 * (vx cos(angle) + vy sin(angle)) - 0.01 from the hull state
    AFTER the physics (+ 100 / n on a new tile, once); -100 off the playfield, and there the episode total
    takes the penalty (the CPU form's takes the step reward it had before); lap and step-limit
    terminations as in the CPU form."""
    try:
        rng = np.random.default_rng(5)
        a_row, b_row = fresh(orc, 4, 3), fresh(orc, 4, 3)
        T, n = tiles(a_row)
        centre = T[:, :8].reshape(n, 4, 2).mean(1)
        total64, new_tiles = 0.0, 0
        for t in range(150):
            x, y, ang = a_row[HULL:HULL + 3]                    # the follow-the-next-tile controller, plus jitter
            tx, ty = centre[min(int(a_row[META + 4]) + 3, n - 1)]
            err = (math.atan2(ty - y, tx - x) - math.pi / 2 - ang + math.pi) % (2 * math.pi) - math.pi
            act = [float(np.clip(err * 2.0, -1, 1)) + float(rng.uniform(-0.05, 0.05)),
                   0.2 if a_row[12] < 12 else -1.0, -1.0]
            seen = a_row[META + 4]
            orc.orc_cr_set_step_form(0)
            r0, d0 = step(orc, a_row, act)
            orc.orc_cr_set_step_form(1)
            r1, d1 = step(orc, b_row, act)
            same = np.ones(S, bool); same[META + 1] = False
            np.testing.assert_array_equal(a_row[same], b_row[same])
            assert d0 == d1 == 0.0
            x, y, ang, vx, vy = (float(v) for v in b_row[HULL:HULL + 5])
            fresh_tile = b_row[META + 4] - seen
            want = 0.5 * (vx * math.cos(ang) + vy * math.sin(ang)) - 0.01 + fresh_tile * 100.0 / n
            assert abs(r1 - want) < 2e-6 * max(1.0, abs(want)), (t, r1, want)
            np.testing.assert_allclose(r0, -0.1 + fresh_tile * 100.0 / n, rtol=1e-6)
            total64 += want; new_tiles += int(fresh_tile)
            np.testing.assert_allclose(b_row[META + 1], total64, rtol=1e-5, atol=1e-5)
        assert new_tiles > 5 and b_row[12] > 5.0            # the car drove: the speed term is not a constant
        # the axis of the speed term is (cos angle, sin angle), as the kernel writes it (the tyres' rolling
        # direction is (-sin, cos), so this is across the wheels and a step's tyre forces eat into it)
        for ang, vx, vy, fwd in ((0.0, 7.0, 0.0, 7.0), (math.pi / 2, 0.0, 7.0, 7.0), (0.0, 0.0, 7.0, 0.0)):
            row = fresh(orc, 3, 0); row[VISITED] = 1.0
            row[HULL + 2], row[HULL + 3], row[HULL + 4] = ang, vx, vy
            r1, _ = step(orc, row, [0, -1, -1])
            v = row[HULL + 3] * math.cos(row[HULL + 2]) + row[HULL + 4] * math.sin(row[HULL + 2])
            assert abs(r1 - (0.5 * v - 0.01)) < 1e-5 and abs(v - fwd) < 3.0
        # off the playfield: -100, done, and the total takes the penalty
        out = fresh(orc, 3, 0); out[HULL] = 334.0; out[META + 1] = 5.0
        assert step(orc, out, [0, -1, -1]) == (-100.0, 1.0) and out[META + 1] == -95.0 and out[META + 2] == 1
        before = out.copy()
        assert step(orc, out, [1, 1, 1]) == (0.0, 1.0) and np.array_equal(out, before)
        orc.orc_cr_set_step_form(0)
        out0 = fresh(orc, 3, 0); out0[HULL] = 334.0; out0[META + 1] = 5.0
        assert step(orc, out0, [0, -1, -1]) == (-100.0, 1.0)
        np.testing.assert_allclose(out0[META + 1], 5.0 - 0.1, rtol=1e-6)          # no tile under a car out there
        orc.orc_cr_set_step_form(1)
        # lap complete and step limit
        lap = fresh(orc, 3, 0)
        T, n = tiles(lap)
        lap[META + 4] = math.ceil(0.95 * n) - 1
        r, d = step(orc, lap, [0, -1, -1])
        assert d == 1.0 and lap[META + 3] == 0 and abs(r - (100.0 / n - 0.01)) < 1e-3     # at rest: no speed term to speak of
        late = fresh(orc, 3, 0); late[META + 0] = 499
        r, d = step(orc, late, [0, -1, -1])
        assert d == 1.0 and late[META + 3] == 1 and late[META + 0] == 500
    finally:
        orc.orc_cr_set_step_form(0)
