"""Pins for the oracle's physics2d pieces: closed forms, invariants, brute force on tiny inputs."""
import ctypes as C
import math

import numpy as np

BS, JS, CS = 13, 17, 9


def make_row(orcmod, orc, nb=2, mc=8, mj=2, me=4, obs=2, meta=2, ns=2):
    L = orcmod.make_layout(orc, nb, mc, mj, me, obs, meta, ns)
    return L, np.zeros(L.state_size, np.float32)


def set_body(L, row, b, x, y, ang, vx, vy, w, mass, inertia, shape=0):
    o = L.bodies_off + b * BS
    row[o:o + 13] = [x, y, ang, vx, vy, w, 0, 0, 0, mass, 1.0 / mass if mass else 0,
                     1.0 / inertia if inertia else 0, shape]


def box_shape(hw, hh):
    s = np.zeros(20, np.float32)
    s[:10] = [0, 4, -hw, hh, -hw, -hh, hw, -hh, hw, hh]
    return s


def test_layout_offsets(orcmod, orc):
    L = orcmod.make_layout(orc, 3, 8, 2, 16, 8, 4, 3)
    assert (L.bodies_off, L.forces_off, L.joints_off, L.joint_count_off, L.edges_off,
            L.edge_count_off, L.meta_off, L.state_size) == (8, 47, 56, 90, 91, 187, 188, 192)
    L = orcmod.make_layout(orc, 5, 20, 4, 128, 24, 8, 5)
    assert L.state_size == 950
    L = orcmod.make_layout(orc, 7, 14, 6, 2, 17, 8, 7)
    assert L.state_size == 253


def test_free_fall_closed_form(orcmod, orc):
    L, row = make_row(orcmod, orc)
    set_body(L, row, 0, 1.0, 10.0, 0.0, 0.5, 0.0, 0.3, 2.0, 1.0)
    set_body(L, row, 1, 0.0, 0.0, 0.0, 1.0, 1.0, 1.0, 0.0, 0.0)  # static: must not move
    n, dt, g = 20, 0.02, -10.0
    for _ in range(n):
        orc.orc_integrate_velocities(C.byref(L), row, 0.0, g, dt)
        orc.orc_integrate_positions(C.byref(L), row, dt)
    b = row[L.bodies_off:L.bodies_off + 13]
    assert abs(b[4] - n * g * dt) < 1e-5                       # v = v0 + n g dt
    assert abs(b[1] - (10.0 + g * dt * dt * n * (n + 1) / 2)) < 1e-4  # semi-implicit sum
    assert abs(b[0] - (1.0 + 0.5 * n * dt)) < 1e-5 and abs(b[2] - 0.3 * n * dt) < 1e-6
    s = row[L.bodies_off + 13:L.bodies_off + 26]
    assert s[0] == 0 and s[1] == 0 and s[3] == 1.0


def test_force_and_torque_integration(orcmod, orc):
    L, row = make_row(orcmod, orc)
    set_body(L, row, 0, 0, 0, 0, 0, 0, 0, 4.0, 2.0)
    row[L.forces_off:L.forces_off + 3] = [8.0, -4.0, 6.0]
    orc.orc_integrate_velocities(C.byref(L), row, 0.0, 0.0, 0.5)
    b = row[L.bodies_off:L.bodies_off + 13]
    np.testing.assert_allclose(b[3:6], [1.0, -0.5, 1.5], rtol=1e-6)


def test_angle_wrap(orcmod, orc):
    L, row = make_row(orcmod, orc)
    for ang, w, want in [(3.0, 10.0, 3.2 - 2 * math.pi), (-3.0, -10.0, -3.2 + 2 * math.pi),
                         (99.0, 100.0, 0.0), (0.5, 1.0, 0.52)]:
        set_body(L, row, 0, 0, 0, ang, 0, 0, w, 1.0, 1.0)
        orc.orc_integrate_positions(C.byref(L), row, 0.02)
        assert abs(row[L.bodies_off + 2] - want) < 1e-5


def brute_edge_contacts(body, verts, edges, max_contacts):
    """float64 brute force of vertex-vs-segment penetration in (vertex, edge) order."""
    x, y, a = body
    out = []
    for vx, vy in verts:
        wx = x + vx * math.cos(a) - vy * math.sin(a)
        wy = y + vx * math.sin(a) + vy * math.cos(a)
        for (x0, y0, x1, y1, nx, ny) in edges:
            lo, hi = min(x0, x1) - 0.1, max(x0, x1) + 0.1
            if wx < lo or wx > hi:
                continue
            dx, dy = x1 - x0, y1 - y0
            t = max(0.0, min(1.0, ((wx - x0) * dx + (wy - y0) * dy) / (dx * dx + dy * dy)))
            pen = -((wx - x0 - t * dx) * nx + (wy - y0 - t * dy) * ny)
            if pen > 0 and len(out) < max_contacts:
                out.append((wx, wy, nx, ny, pen))
    return out


def test_edge_detect_brute_force(orcmod, orc):
    L, row = make_row(orcmod, orc, nb=1, mc=3, me=4)
    shapes = np.zeros(40, np.float32)
    shapes[:20] = box_shape(0.5, 0.25)
    heights = np.array([1.0, 1.0, 2.0, 1.5], np.float32)
    orc.orc_set_terrain_from_heights(C.byref(L), row, heights, 4, 0.0, 2.0)
    assert row[L.edge_count_off] == 3
    edges = row[L.edges_off:L.edges_off + 18].reshape(3, 6).astype(np.float64)
    for e in edges:                                  # unit, upward normals, perpendicular to edge
        assert abs(math.hypot(e[4], e[5]) - 1) < 1e-6 and e[5] > 0
        assert abs((e[2] - e[0]) * e[4] + (e[3] - e[1]) * e[5]) < 1e-6
    rng = np.random.default_rng(3)
    hits = 0
    for _ in range(300):
        bx, by, ba = rng.uniform(0, 6), rng.uniform(0.8, 2.3), rng.uniform(-1, 1)
        set_body(L, row, 0, bx, by, ba, 0, 0, 0, 1.0, 1.0)
        contacts = np.zeros(3 * CS, np.float32)
        n = orc.orc_edge_detect(C.byref(L), row, shapes, contacts)
        b32 = row[L.bodies_off:L.bodies_off + 3].astype(np.float64)
        want = brute_edge_contacts(b32, [(-.5, .25), (-.5, -.25), (.5, -.25), (.5, .25)],
                                   edges.tolist(), 3)
        if any(abs(w[4]) < 1e-5 for w in want) or n != len(want):
            # a penetration within rounding of zero may legitimately flip; everything else must agree
            assert any(abs(w[4]) < 1e-5 for w in brute_edge_contacts(
                b32, [(-.5, .25), (-.5, -.25), (.5, -.25), (.5, .25)], edges.tolist(), 99)), (n, want)
            continue
        hits += n
        assert n <= 3
        for k, w in enumerate(want):
            c = contacts[k * CS:(k + 1) * CS]
            assert c[0] == 0 and c[1] == -1 and c[7] == 0 and c[8] == 0
            np.testing.assert_allclose(c[2:7], w, rtol=1e-4, atol=2e-6)
    assert hits > 100


def test_vertex_on_joint_gives_two_contacts(orcmod, orc):
    # a vertex below the junction of two edges is reported against both (no dedup in the reference)
    L, row = make_row(orcmod, orc, nb=1, mc=8, me=4)
    shapes = np.zeros(40, np.float32)
    shapes[:6] = [0, 1, 0.0, 0.0, 0, 0]  # one-vertex polygon
    orc.orc_set_terrain_from_heights(C.byref(L), row, np.array([1, 1, 1], np.float32), 3, 0.0, 1.0)
    set_body(L, row, 0, 1.0, 0.9, 0, 0, 0, 0, 1.0, 1.0)
    contacts = np.zeros(8 * CS, np.float32)
    assert orc.orc_edge_detect(C.byref(L), row, shapes, contacts) == 2
    assert abs(contacts[6] - 0.1) < 1e-6 and abs(contacts[CS + 6] - 0.1) < 1e-6


def test_flat_detect(orcmod, orc):
    L, row = make_row(orcmod, orc, nb=2, mc=3)
    shapes = np.zeros(40, np.float32)
    shapes[:20] = box_shape(0.5, 0.5)
    shapes[20:24] = [1, 0.3, 0.0, 0.0]  # circle r = 0.3
    set_body(L, row, 0, 0.0, 0.4, 0.0, 0, 0, 0, 1, 1, shape=0)
    set_body(L, row, 1, 2.0, 0.2, 0.0, 0, 0, 0, 1, 1, shape=1)
    contacts = np.zeros(3 * CS, np.float32)
    n = orc.orc_flat_detect(C.byref(L), row, shapes, 0.0, contacts)
    assert n == 3  # two bottom vertices of the box, then the circle
    np.testing.assert_allclose(contacts[0:9], [0, -1, -.5, -.1, 0, 1, .1, 0, 0], atol=1e-6)
    np.testing.assert_allclose(contacts[9:18], [0, -1, .5, -.1, 0, 1, .1, 0, 0], atol=1e-6)
    np.testing.assert_allclose(contacts[18:27], [1, -1, 2.0, -.1, 0, 1, .1, 0, 0], atol=1e-6)


def test_contact_velocity_solve_single_contact(orcmod, orc):
    L, row = make_row(orcmod, orc, nb=1)
    set_body(L, row, 0, 0.0, 1.0, 0.0, 2.0, -3.0, 0.0, 2.0, 1e9)  # ~no rotation
    contact = np.array([0, -1, 0.0, 0.0, 0, 1, 0.05, 0, 0], np.float32)
    orc.orc_contact_solve_velocity(C.byref(L), row, contact, 1, 0.3, 0.0)
    b = row[L.bodies_off:L.bodies_off + 13]
    assert abs(b[4]) < 1e-6                               # normal velocity removed
    jn, jt = contact[7], contact[8]
    assert abs(jn - 3.0 * 2.0) < 1e-5                     # j = m * |v_n|
    assert abs(abs(jt) - 0.3 * jn) < 1e-5                 # sliding: friction saturates at mu * jn
    assert abs(b[3] - (2.0 - 0.3 * jn / 2.0)) < 1e-5      # opposes the slide
    before = row.copy()
    orc.orc_contact_solve_velocity(C.byref(L), row, contact, 1, 0.3, 0.0)
    np.testing.assert_array_equal(before, row)            # v_n == 0: a second sweep is a no-op
    # separating contact: untouched
    set_body(L, row, 0, 0, 1, 0, 0, 1.0, 0, 2.0, 1.0)
    c2 = np.array([0, -1, 0.0, 0.0, 0, 1, 0.05, 0, 0], np.float32)
    orc.orc_contact_solve_velocity(C.byref(L), row, c2, 1, 0.3, 0.0)
    assert row[L.bodies_off + 4] == 1.0 and c2[7] == 0


def test_contact_solve_with_rotation_conserves(orcmod, orc):
    # off-centre contact: the impulse applied to v and omega must be consistent (J = m dv, r x J = I dw)
    L, row = make_row(orcmod, orc, nb=1)
    m, I = 2.0, 0.5
    set_body(L, row, 0, 0.3, 1.0, 0.0, 0.0, -2.0, 0.4, m, I)
    contact = np.array([0, -1, 0.8, 0.0, 0, 1, 0.01, 0, 0], np.float32)
    v0 = row[L.bodies_off + 3:L.bodies_off + 6].copy()
    orc.orc_contact_solve_velocity(C.byref(L), row, contact, 1, 0.0, 0.0)
    v1 = row[L.bodies_off + 3:L.bodies_off + 6]
    Jx, Jy = m * (v1[0] - v0[0]), m * (v1[1] - v0[1])
    rx, ry = 0.8 - 0.3, 0.0 - 1.0
    assert abs(I * (v1[2] - v0[2]) - (rx * Jy - ry * Jx)) < 1e-5
    assert abs(Jx) < 1e-6 and abs(Jy - contact[7]) < 1e-5
    vn = v1[1] + v1[2] * rx
    assert abs(vn) < 1e-5


def test_contact_position_solve(orcmod, orc):
    L, row = make_row(orcmod, orc, nb=1)
    set_body(L, row, 0, 0.0, 1.0, 0, 0, 0, 0, 2.0, 1.0)
    c = np.array([0, -1, 0, 0, 0.6, 0.8, 0.105, 0, 0, 0, -1, 0, 0, 0, 1, 0.004, 0, 0], np.float32)
    orc.orc_contact_solve_position(C.byref(L), row, c, 2, 0.2, 0.005)
    np.testing.assert_allclose(row[L.bodies_off:L.bodies_off + 2], [0.6 * 0.02, 1 + 0.8 * 0.02], rtol=1e-5)


def two_body_joint(orcmod, orc, flags=0, lo=0, hi=0, stiff=0, damp=0, mt=0, ms=0):
    L, row = make_row(orcmod, orc, nb=2, mj=1)
    set_body(L, row, 0, 0.0, 0.0, 0.3, 0.5, -0.2, 0.7, 1.0, 0.5)
    set_body(L, row, 1, 1.0, 0.0, -0.2, -0.4, 0.3, -0.5, 1.0, 0.5)
    ca, sa, cb, sb = math.cos(0.3), math.sin(0.3), math.cos(-0.2), math.sin(-0.2)
    # anchor at world (0.5, 0): local = R(-angle) * (world - pos)
    ax, ay = ca * 0.5 + sa * 0.0, -sa * 0.5 + ca * 0.0
    bx, by = cb * -0.5 + sb * 0.0, -sb * -0.5 + cb * 0.0
    j = L.joints_off
    row[j:j + 17] = [0, 0, 1, ax, ay, bx, by, -0.5, lo, hi, mt, ms, stiff, damp, flags, 0, 0]
    row[L.joint_count_off] = 1
    return L, row


def anchor_vel(row, L, b, r):
    o = L.bodies_off + b * BS
    return row[o + 3] - row[o + 5] * r[1], row[o + 4] + row[o + 5] * r[0]


def test_joint_velocity_point_constraint(orcmod, orc):
    L, row = two_body_joint(orcmod, orc)
    p0 = row[L.bodies_off + 3:L.bodies_off + 5] + row[L.bodies_off + 16:L.bodies_off + 18]
    orc.orc_joint_solve_velocity(C.byref(L), row, 0.02)
    va = anchor_vel(row, L, 0, (0.5, 0.0))
    vb = anchor_vel(row, L, 1, (-0.5, 0.0))
    assert abs(va[0] - vb[0]) < 1e-5 and abs(va[1] - vb[1]) < 1e-5   # Cdot = 0 after one solve
    p1 = row[L.bodies_off + 3:L.bodies_off + 5] + row[L.bodies_off + 16:L.bodies_off + 18]
    np.testing.assert_allclose(p0, p1, atol=1e-6)                     # equal masses: momentum kept


def test_joint_motor_limit_spring(orcmod, orc):
    # motor, unclamped: relative omega reaches the target
    L, row = two_body_joint(orcmod, orc, flags=2, mt=1e6, ms=2.0)
    orc.orc_joint_solve_velocity(C.byref(L), row, 0.02)
    assert abs((row[L.bodies_off + 18] - row[L.bodies_off + 5]) - 2.0) < 1e-5
    # motor, clamped: impulse = max_torque * dt, split by inverse inertia
    L, row = two_body_joint(orcmod, orc, flags=0)
    orc.orc_joint_solve_velocity(C.byref(L), row, 0.02)
    base = row[L.bodies_off + 18] - row[L.bodies_off + 5]
    L, row = two_body_joint(orcmod, orc, flags=2, mt=0.5, ms=100.0)
    orc.orc_joint_solve_velocity(C.byref(L), row, 0.02)
    assert abs((row[L.bodies_off + 18] - row[L.bodies_off + 5]) - (base + 4.0 * 0.5 * 0.02)) < 1e-5
    # limit: rel angle = -0.2 - 0.3 + 0.5 = 0 <= lower(0.1) and rel omega < 0 -> killed
    L, row = two_body_joint(orcmod, orc, flags=1, lo=0.1, hi=0.5)
    orc.orc_joint_solve_velocity(C.byref(L), row, 0.02)
    assert base < 0 and abs(row[L.bodies_off + 18] - row[L.bodies_off + 5]) < 1e-6
    # limit not touched when moving away from it
    L, row = two_body_joint(orcmod, orc, flags=1, lo=-0.5, hi=-0.1)  # at/above upper, rel omega < 0
    orc.orc_joint_solve_velocity(C.byref(L), row, 0.02)
    assert abs((row[L.bodies_off + 18] - row[L.bodies_off + 5]) - base) < 1e-6
    # spring uses the PRE-impulse omegas: torque = -k*err - c*(wb - wa) with wb - wa = -1.2
    L, row = two_body_joint(orcmod, orc, flags=4, stiff=10.0, damp=2.0)
    orc.orc_joint_solve_velocity(C.byref(L), row, 0.02)
    imp = (-10.0 * 0.0 - 2.0 * (-1.2)) * 0.02
    assert abs((row[L.bodies_off + 18] - row[L.bodies_off + 5]) - (base + imp)) < 1e-5


def test_joint_position_solve(orcmod, orc):
    L, row = two_body_joint(orcmod, orc)
    row[L.bodies_off + 13] = 1.2     # pull body B away: anchor error 0.2 along x
    def err():
        a = row[L.bodies_off:L.bodies_off + 3]; b = row[L.bodies_off + 13:L.bodies_off + 16]
        j = row[L.joints_off:L.joints_off + 17]
        wa = (a[0] + j[3] * math.cos(a[2]) - j[4] * math.sin(a[2]), a[1] + j[3] * math.sin(a[2]) + j[4] * math.cos(a[2]))
        wb = (b[0] + j[5] * math.cos(b[2]) - j[6] * math.sin(b[2]), b[1] + j[5] * math.sin(b[2]) + j[6] * math.cos(b[2]))
        return math.hypot(wb[0] - wa[0], wb[1] - wa[1])
    e0 = err()
    orc.orc_joint_solve_position(C.byref(L), row, 0.2, 0.005)
    assert abs(err() - 0.8 * e0) < 2e-3          # |C| shrinks by (1 - beta) (linearised)
    # below slop: nothing moves, limit correction is skipped as well
    L, row = two_body_joint(orcmod, orc, flags=1, lo=0.3, hi=0.5)
    before = row.copy()
    orc.orc_joint_solve_position(C.byref(L), row, 0.2, 0.005)
    np.testing.assert_array_equal(before, row)
    # above slop with a violated lower limit: angles corrected by beta*(lo - rel), split by inv inertia
    row[L.bodies_off + 13] = 1.2
    orc.orc_joint_solve_position(C.byref(L), row, 0.2, 0.005)
    rel = row[L.bodies_off + 15] - row[L.bodies_off + 2] + 0.5
    assert rel > 0.0


def test_lidar_closed_form(orcmod, orc):
    L, row = make_row(orcmod, orc, nb=1, me=4)
    e = L.edges_off
    row[e:e + 12] = [0, 0, 10, 0, 0, 1, 10, 0, 10, 5, -1, 0]
    row[L.edge_count_off] = 2
    assert abs(orc.orc_lidar_ray(C.byref(L), row, 2.0, 3.0, 0.0, -6.0) - 0.5) < 1e-6       # straight down
    assert abs(orc.orc_lidar_ray(C.byref(L), row, 2.0, 3.0, 16.0, 0.0) - 0.5) < 1e-6       # wall at x=10
    assert orc.orc_lidar_ray(C.byref(L), row, 2.0, 3.0, 0.0, -2.0) == 1.0                  # too short
    assert orc.orc_lidar_ray(C.byref(L), row, 2.0, 3.0, 5.0, 0.0) == 1.0                   # parallel / miss
    assert abs(orc.orc_lidar_ray(C.byref(L), row, 2.0, 3.0, 6.0, -6.0) - 0.5) < 1e-6       # diagonal
