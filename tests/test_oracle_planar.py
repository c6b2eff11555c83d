"""Pins for the oracle's HopperPlanar / Walker2dPlanar (envs/mujoco_planar/hopper_planar.mojo,
walker_planar.mojo): closed forms of the simplified physics (joint integration, the standing height a foot
contact leaves, the walker's double push), forward kinematics against complex-number geometry, the
reward by hand, the termination thresholds, the reset's draws.  The reference holds no golden vectors
for these envs; its own tests (tests/test_hopper_planar.mojo, test_walker_planar.mojo) check dimensions,
the initial height and that a step returns finite numbers, which are asserted here too."""
import numpy as np
import pytest

HOPPER, WALKER = 0, 1
DT, G = 0.008, -9.81
MODELS = {
    HOPPER: dict(obs=11, state=62, nj=3, gear=200.0, foot=0.39, min_z=0.7, max_z=None, max_angle=0.2,
                 lim=[(-2.61799, 0.0), (-2.61799, 0.0), (-0.785398, 0.785398)], hips=[0.0]),
    WALKER: dict(obs=17, state=98, nj=6, gear=100.0, foot=0.2, min_z=0.8, max_z=2.0, max_angle=1.0,
                 lim=[(-1.0, 0.7), (-1.2, 0.0), (-0.5, 0.5)], hips=[0.1, -0.1]),
}
TORSO, THIGH, LEG, RADIUS = 0.4, 0.45, 0.5, 0.06


def view(which, row):
    m = MODELS[which]
    d = row[m["obs"] + 1:].view(np.float64)
    nj = m["nj"]
    return dict(torso=d[0:6], body=d[6:6 + 3 * nj].reshape(nj, 3), ja=d[6 + 3 * nj:6 + 4 * nj],
                jv=d[6 + 4 * nj:6 + 5 * nj], meta=d[6 + 5 * nj:6 + 5 * nj + 4])


def fresh(orc, which, cseed=12345, quiet=False):
    row = np.zeros(MODELS[which]["state"], np.float32)
    orc.orc_planar_reset(which, row, cseed)
    if quiet:   # without the reset noise: closed forms below start from joints at rest at angle 0
        v = view(which, row)
        v["ja"][:] = 0.0
        v["jv"][:] = 0.0
    return row


def step(orc, which, row, a):
    r, d = np.zeros(1, np.float32), np.zeros(1, np.float32)
    orc.orc_planar_step(which, row, np.asarray(a, np.float32), r, d)
    return float(r[0]), float(d[0])


@pytest.mark.parametrize("which", [HOPPER, WALKER])
def test_dimensions_and_reset(orc, which):
    """hopper_planar.mojo:203-322 / walker_planar.mojo:198-337: torso at (0, 1.25) at rest, the leg bodies
    stacked below it, joint angles and velocities (u - 0.5) * 0.01 from one draw each, angle first."""
    m = MODELS[which]
    assert orc.orc_planar_state_size(which) == m["state"] == m["obs"] + 1 + 2 * (6 + 5 * m["nj"] + 4)
    row = fresh(orc, which, cseed=777)
    v = view(which, row)
    assert list(v["torso"]) == [0.0, 1.25, 0.0, 0.0, 0.0, 0.0] and list(v["meta"]) == [0.0] * 4
    thigh_y = 1.25 - 0.2 - 0.225
    leg_y = thigh_y - 0.225 - 0.25
    foot_y = leg_y - 0.25 - m["foot"] / 2
    for l, dx in enumerate(m["hips"]):
        np.testing.assert_allclose(v["body"][3 * l:3 * l + 3], [[dx, thigh_y, 0], [dx, leg_y, 0], [dx, foot_y, 0]],
                                   rtol=0, atol=1e-15)
    u = np.concatenate([_uniform4(orc, 777, b) for b in range(3)]).astype(np.float64)
    nj = m["nj"]
    np.testing.assert_array_equal(v["ja"], (u[0:2 * nj:2] - 0.5) * 0.01)
    np.testing.assert_array_equal(v["jv"], (u[1:2 * nj:2] - 0.5) * 0.01)
    assert np.abs(v["ja"]).max() <= 0.005 and len(set(v["ja"])) == nj
    # the observation: [z, angle, joint angles, vx, vz, omega, joint velocities], cast to fp32
    o = row[:m["obs"]]
    assert o[0] == np.float32(1.25) and o[1] == 0
    np.testing.assert_array_equal(o[2:2 + nj], v["ja"].astype(np.float32))
    np.testing.assert_array_equal(o[2 + nj:5 + nj], 0)
    np.testing.assert_array_equal(o[5 + nj:], v["jv"].astype(np.float32))
    # another seed gives other noise; the same seed the same row
    assert not np.array_equal(fresh(orc, which, cseed=778), row) and np.array_equal(fresh(orc, which, cseed=777), row)


def _uniform4(orc, cseed, block):
    u = np.zeros(4, np.float32)
    orc.orc_philox_uniform4(cseed, 0, block, u)
    return u


@pytest.mark.parametrize("which", [HOPPER, WALKER])
def test_joint_integration_closed_form_and_limits(orc, which):
    """_physics_step: velocity += torque * dt * 0.01, then angle += velocity * dt, four times per step:
    after one step from rest  v = 4 c,  angle = 10 c dt  with c = clip(a) * gear * dt * 0.01; an angle
    that passes a limit is set to it with velocity 0."""
    m = MODELS[which]
    nj = m["nj"]
    row = fresh(orc, which, quiet=True)
    a = np.linspace(-0.05, 0.04, nj).astype(np.float32).astype(np.float64)   # actions arrive as fp32
    a[1] = 0.0                     # a joint without torque stays where it is
    a[1::3] = -np.abs(a[1::3])     # knees bend one way only: 0 is their upper limit
    step(orc, which, row, a)
    v = view(which, row)
    c = a * m["gear"] * DT * 0.01
    np.testing.assert_allclose(v["jv"], 4 * c, rtol=1e-14, atol=0)
    np.testing.assert_allclose(v["ja"], 10 * c * DT, rtol=1e-14, atol=0)
    # |a| > 1 acts as 1
    r1, r2 = fresh(orc, which, quiet=True), fresh(orc, which, quiet=True)
    step(orc, which, r1, np.full(nj, 7.5)); step(orc, which, r2, np.full(nj, 1.0))
    np.testing.assert_array_equal(view(which, r1)["jv"], view(which, r2)["jv"])
    # limits: drive every joint down, then up; an angle never leaves [low, high], reaches both ends and
    # has velocity 0 in the sub-step that clamps it
    for sign in (-1.0, 1.0):
        row = fresh(orc, which, quiet=True)
        view(which, row)["torso"][1] = 1.5
        hit = np.zeros(nj, bool)
        for _ in range(400):
            view(which, row)["meta"][1] = 0.0      # keep stepping whatever the health check says
            view(which, row)["torso"][1] = 1.5
            step(orc, which, row, np.full(nj, sign))
            v = view(which, row)
            for j in range(nj):
                low, high = m["lim"][j % 3]
                assert low <= v["ja"][j] <= high
                end = low if sign < 0 else high
                if v["ja"][j] == end:
                    hit[j] = True
                    # clamped in the last sub-step: velocity 0; or clamped earlier in this step and pushed on since
                    assert v["jv"][j] == 0.0
        assert hit.all()


def _chain(which, hip, angles):
    """Body centres and angles from complex arithmetic: a segment of length L at cumulative angle t
    runs from its upper joint p to p - 1j * L * exp(1j * t)."""
    m = MODELS[which]
    out = []
    p, t = hip, 0.0
    for L, ang in zip((THIGH, LEG, m["foot"]), angles):
        t = t + ang
        seg = -1j * L * np.exp(1j * t)
        out.append((p + seg / 2, t))
        p = p + seg
    return out


@pytest.mark.parametrize("which", [HOPPER, WALKER])
def test_forward_kinematics_geometry(orc, which):
    """_update_body_positions: the thigh hangs from the torso's lower end (x offset +-0.1 for the walker's
    two legs), each next segment from the end of the one before, at the cumulative joint angle."""
    m = MODELS[which]
    nj = m["nj"]
    rng = np.random.default_rng(5)
    for _ in range(20):
        row = fresh(orc, which, quiet=True)
        v = view(which, row)
        v["torso"][0:2] = [rng.uniform(-1, 1), rng.uniform(1.6, 1.9)]      # high up: no ground contact
        ja = np.array([rng.uniform(*m["lim"][j % 3]) for j in range(nj)]) * 0.9
        v["ja"][:] = ja
        step(orc, which, row, np.zeros(nj))
        v = view(which, row)
        np.testing.assert_array_equal(v["ja"], ja)
        tx, ty = v["torso"][0], v["torso"][1]
        for l, dx in enumerate(m["hips"]):
            want = _chain(which, complex(tx + dx, ty - TORSO / 2), ja[3 * l:3 * l + 3])
            for b, (p, t) in enumerate(want):
                np.testing.assert_allclose(v["body"][3 * l + b], [p.real, p.imag, t], rtol=0, atol=5e-16 * 8)


def test_hopper_stands_on_its_foot(orc):
    """_handle_ground_collision: a foot below the ground lifts the torso by the penetration and stops its
    fall.  With a straight leg the foot's lowest point is torso_y - (0.2 + 0.45 + 0.5 + 0.195 + 0.06), so
    from the reset pose (foot 0.155 under ground) every sub-step ends at torso_y = 1.405 with vy = 0."""
    row = fresh(orc, HOPPER, quiet=True)
    r, d = step(orc, HOPPER, row, np.zeros(3))
    v = view(HOPPER, row)
    np.testing.assert_allclose(v["torso"][1], 1.405, rtol=0, atol=1e-15)
    assert v["torso"][4] == 0.0 and v["torso"][0] == 0.0 and v["torso"][3] == 0.0
    assert (r, d) == (1.0, 0.0) and list(v["meta"]) == [1.0, 0.0, 1.0, 0.0]
    # the foot body was placed before the push: it still shows the pre-push height
    np.testing.assert_allclose(v["body"][2][1] - RADIUS, 1.405 + G * DT * DT - 1.405, rtol=0, atol=1e-15)
    # airborne: free fall, vy -= 9.81 * 0.008 per sub-step, y from the new velocity (semi-implicit)
    row = fresh(orc, HOPPER, quiet=True)
    view(HOPPER, row)["torso"][1] = 1.6
    step(orc, HOPPER, row, np.zeros(3))
    v = view(HOPPER, row)
    np.testing.assert_allclose(v["torso"][4], 4 * G * DT, rtol=1e-15)
    np.testing.assert_allclose(v["torso"][1], 1.6 + 10 * G * DT * DT, rtol=0, atol=1e-15)


def test_walker_feet_push_in_turn_from_stale_positions(orc):
    """walker_planar.mojo:606-639: both feet are tested against the ground with the positions the forward
    kinematics left, so two straight legs push the torso up twice: a sub-step that starts at height y
    (after the fall) ends at y + 2 * (0.06 - (y - 1.25)).  From the reset pose that is 2.62 - (1.25 +
    g dt^2) after the first sub-step, then three sub-steps of free fall from rest."""
    row = fresh(orc, WALKER, quiet=True)
    r, d = step(orc, WALKER, row, np.zeros(6))
    v = view(WALKER, row)
    y1 = 2.62 - (1.25 + G * DT * DT)
    np.testing.assert_allclose(v["torso"][1], y1 + (1 + 2 + 3) * G * DT * DT, rtol=0, atol=1e-15)
    np.testing.assert_allclose(v["torso"][4], 3 * G * DT, rtol=1e-15)
    assert (r, d) == (1.0, 0.0)
    # one leg lifted (knee bent back so that its foot is clear of the ground): a single push per sub-step,
    # which puts the standing foot's lowest point on the ground: the walker stands at 1.25 + 0.06
    row = fresh(orc, WALKER, quiet=True)
    view(WALKER, row)["ja"][4] = -1.1
    step(orc, WALKER, row, np.zeros(6))
    v = view(WALKER, row)
    np.testing.assert_allclose(v["torso"][1], 1.31, rtol=0, atol=1e-15)
    assert v["torso"][4] == 0.0


@pytest.mark.parametrize("which", [HOPPER, WALKER])
def test_reward_and_termination(orc, which):
    """step(): reward = forward velocity + 1 (while healthy) - 0.001 * sum(clip(a)^2); nothing in the
    simplified physics moves the torso sideways, so the forward term is the torso's own vx; healthy means
    z >= MIN_Z, |angle| <= MAX_ANGLE and, for the walker, z <= MAX_Z; a finished row is left alone."""
    m = MODELS[which]
    nj = m["nj"]
    a = np.array([0.5, -2.0, 0.25, 1.5, -0.125, 0.0][:nj])
    row = fresh(orc, which)
    r, d = step(orc, which, row, a)
    want = 1.0 - 0.001 * float((np.clip(a, -1, 1) ** 2).sum())
    assert d == 0.0 and r == np.float32(want)
    # a torso that drifts: forward velocity = (x_after - x_before) / (4 dt) = vx
    row = fresh(orc, which)
    view(which, row)["torso"][3] = 0.75
    r, d = step(orc, which, row, np.zeros(nj))
    assert abs(r - 1.75) < 1e-6 and abs(view(which, row)["torso"][0] - 0.75 * 4 * DT) < 1e-15
    assert row[2 + nj] == np.float32(0.75)
    # thresholds
    def outcome(y=None, angle=None):
        row = fresh(orc, which, quiet=True)
        v = view(which, row)
        if y is not None:
            v["torso"][1] = y
            v["ja"][0::3] = -2.0 if which == HOPPER else -1.0     # legs folded up behind: no ground push
            v["ja"][1::3] = -2.0 if which == HOPPER else -1.2
            v["ja"][2::3] = 0.0 if which == HOPPER else -0.5
        if angle is not None:
            v["torso"][2] = angle
        r, d = step(orc, which, row, np.zeros(nj))
        return r, d, row
    fall = 10 * G * DT * DT          # height lost in one step of free fall from rest
    assert outcome(y=m["min_z"] - fall + 1e-9)[:2] == (1.0, 0.0)
    assert outcome(y=m["min_z"] - fall - 1e-9)[:2] == (0.0, 1.0)
    assert outcome(angle=m["max_angle"])[:2] == (1.0, 0.0)
    assert outcome(angle=-m["max_angle"] - 1e-12)[:2] == (0.0, 1.0)
    if m["max_z"] is None:
        assert outcome(y=5.0)[:2] == (1.0, 0.0)
    else:
        assert outcome(y=m["max_z"] - fall)[:2] == (1.0, 0.0)
        assert outcome(y=m["max_z"] - fall + 1e-9)[:2] == (0.0, 1.0)
    # finished row: (0, 1), nothing moves, the counters stay
    r, d, row = outcome(angle=1.5)
    assert view(which, row)["meta"][1] == 1.0 and view(which, row)["meta"][0] == 1.0
    before = row.copy()
    assert step(orc, which, row, np.ones(nj)) == (0.0, 1.0)
    np.testing.assert_array_equal(row, before)


@pytest.mark.parametrize("which", [HOPPER, WALKER])
def test_batch_form_and_reference_smoke_properties(orc, which):
    """The batched calls are the single-row calls over rows with seed * 2654435761 + (env + 1) * 12345
    (the combined seed of the reference's GPU envs); as in the reference's own tests, observations have
    the stated width and stay finite over random actions, and an episode ends sooner or later."""
    m = MODELS[which]
    n, nj = 64, m["nj"]
    states = np.zeros((n, m["state"]), np.float32)
    orc.orc_planar_reset_batch(which, states.reshape(-1), None, n, 9)
    for i in (0, 17, 63):
        np.testing.assert_array_equal(states[i], fresh(orc, which, cseed=9 * 2654435761 + (i + 1) * 12345))
    rng = np.random.default_rng(1)
    mirror = states.copy()
    ended = np.zeros(n, bool)
    for t in range(300):
        a = rng.uniform(-1.5, 1.5, (n, nj)).astype(np.float32)
        r, d, o = np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros((n, m["obs"]), np.float32)
        orc.orc_planar_step_batch(which, states.reshape(-1), a.reshape(-1), r, d, o.reshape(-1), n, 2)
        assert np.isfinite(o).all() and np.isfinite(r).all()
        np.testing.assert_array_equal(o, states[:, :m["obs"]])
        if t < 3:
            for i in (0, 31):
                ri, di = step(orc, which, mirror[i], a[i])
                assert (ri, di) == (float(r[i]), float(d[i]))
                np.testing.assert_array_equal(mirror[i], states[i])
        ended |= d > 0.5
    assert ended.any()
    # selective reset: only rows whose flag is set
    before = states.copy()
    flags = (np.arange(n) % 3 == 0).astype(np.float32)
    orc.orc_planar_reset_batch(which, states.reshape(-1), flags.ctypes.data, n, 11)
    for i in range(n):
        if flags[i] > 0.5:
            np.testing.assert_array_equal(states[i], fresh(orc, which, cseed=11 * 2654435761 + (i + 1) * 12345))
        else:
            np.testing.assert_array_equal(states[i], before[i])
