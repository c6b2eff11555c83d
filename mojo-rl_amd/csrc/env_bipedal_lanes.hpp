// BipedalWalker's physics step with one lane per BODY: eight lanes per env (five bodies, three idle).
//
// With one lane per env the solver is one long instruction stream: per sweep up to 20 contacts and
// four joints in turn, each body picked out of five with select chains, and the sines and cosines of
// both bodies of every joint taken again at every position correction.  Much of it is work on
// different bodies that does not interact:
//   * every contact is between one body and the terrain, so contacts of different bodies commute
//     exactly: a lane runs the contacts of its own body, in list order, where the one-lane form runs
//     the whole list;
//   * the joint sweep visits joints 0 .. 3 in order -- hull - upper leg 1, upper leg 1 - lower leg 1,
//     hull - upper leg 2, upper leg 2 - lower leg 2 -- and joints 1 and 2 have no body in common:
//     three joint slots per sweep instead of four.  In a slot the CHILD body's lane does the joint
//     (parent state fetched from the parent's lane, parent result handed back), so every lane holds its
//     body in plain registers and carries the sine / cosine of its own angle.
// Same operations on the same values in an order the arithmetic cannot tell from the one-lane form's:
// identical results bit for bit.
//
// The contacts are the env's merged list in LDS (the records the per-vertex detection tasks left, in
// (body, vertex) order, cut at MAX_CONTACTS); a lane owns the records whose body is its own and keeps
// their lever arms, effective masses and accumulated impulses in the record, like the one-lane form's
// LDS-resident list.  A row whose joint table differs from the walker's own is stepped by the one-lane
// form instead (lanes_row_ok, tested by the caller).
#pragma once
#include "env_walkers.hpp"

namespace mrl {
namespace bw {

constexpr int LANES_PER_ENV = 8;

// a single body behind the register-form contact functions of physics2d_reg.hpp
struct OneBody { static constexpr int NUM_BODIES = 1; };

// The exchanges of a joint slot as DPP row shifts (rows are 16 lanes: two groups shift side by side; a
// lane at a group's edge picks up a value that it never uses).
//   from_parent: the parent of body b is the body before it, except upper leg 2 (3), whose parent is
//                the hull three lanes down;
//   from_kid:    the parent's lane takes the result of its child in slot s -- the next lane, except the
//                hull in slot 1, whose child is upper leg 2 three lanes up.
MRL_DEV float lanes_shr1(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xF, 0xF, false)); }
MRL_DEV float lanes_shr3(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x113, 0xF, 0xF, false)); }
MRL_DEV float lanes_shl1(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x101, 0xF, 0xF, false)); }
MRL_DEV float lanes_shl3(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x103, 0xF, 0xF, false)); }
MRL_DEV float from_parent(float v, int b) {
    const float one = lanes_shr1(v), three = lanes_shr3(v);
    return b == 3 ? three : one;
}
MRL_DEV float from_kid(int s, float v, int b) {
    const float one = lanes_shl1(v), three = lanes_shl3(v);
    return (s == 1 && b == 0) ? three : one;
}

// true when the row has the wiring this form assumes
MRL_DEV bool lanes_row_ok(const float *row) {
    if ((int)row[L::JOINT_COUNT_OFF] != 4) return false;
    bool ok = true;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float *J = row + L::JOINTS_OFF + j * JOINT_SIZE;
        ok = ok && (int)J[J_TYPE] == 0 && (int)J[J_BODY_A] == Topology::a(j) && (int)J[J_BODY_B] == Topology::b(j);
    }
    return ok;
}

// The physics of bw::step_finish (one sub-step: 6 velocity and 2 position sweeps) by the eight lanes of
// an env's group; all lanes of the group call it together.  `lane` = lane in the wavefront, `row` = the
// group's env row in LDS (motors already set by step_motors), `contacts` = the env's merged contact list
// with n >= 0 records.  Leaves the bodies and the cleared forces in the row.
MRL_DEV void physics_lanes(float *row, float *contacts, int n, int lane) {
    const int b = lane & 7;
    const bool body = b < L::NUM_BODIES;
    // ---- wiring seen from this lane: the child of joint b - 1 (bodies 1 .. 4) ...
    const bool child = b >= 1 && b <= 4;
    const int j = child ? b - 1 : 0;
    const int myslot = b == 1 ? 0 : (b == 2 || b == 3) ? 1 : b == 4 ? 2 : -1;
    // ... and the parent of the joint that runs in slot s: bit s of kidmask
    const int kidmask = b == 0 ? 3 : b == 1 ? 2 : b == 3 ? 4 : 0;

    const float gx = (float)0.0, gy = (float)-10.0, dt = (float)(1.0 / FPS), friction = (float)2.5, restitution = (float)0.0;
    const float baumgarte = (float)0.2, slop = (float)0.005;

    const float *J = row + L::JOINTS_OFF + j * JOINT_SIZE;
    const float lax = J[J_AX], lay = J[J_AY], lbx = J[J_BX], lby = J[J_BY];
    const float jref = J[J_REF], jlo = J[J_LO], jhi = J[J_HI], jstiff = J[J_STIFF], jdamp = J[J_DAMP];
    const float motor_speed = J[J_MOTOR_SPEED], max_torque = J[J_MAX_TORQUE];
    const int jflags = (int)J[J_FLAGS];

    // ---- my body
    float *Bp = row + L::BODIES_OFF + (body ? b : 0) * BODY_SIZE;
    float x = Bp[IDX_X], y = Bp[IDX_Y], ang = Bp[IDX_ANGLE], vx = Bp[IDX_VX], vy = Bp[IDX_VY], w = Bp[IDX_OMEGA];
    const float im = Bp[IDX_INV_MASS], ii = Bp[IDX_INV_INERTIA];
    const float *F = row + L::FORCES_OFF + (body ? b : 0) * 3;
    const float fx = F[0], fy = F[1], tau = F[2];
    const float p_im = from_parent(im, b), p_ii = from_parent(ii, b);

    // my records of the list: bit c of `mine` (every slot is read, the count cuts afterwards)
    unsigned mine = 0;
#pragma unroll
    for (int c = 0; c < L::MAX_CONTACTS; ++c)
        mine |= (unsigned)((int)contacts[c * CONTACT_SIZE + C_BODY_A] == b) << c;
    mine &= n >= 32 ? 0xFFFFFFFFu : ((1u << n) - 1u);
    if (!body) mine = 0;

    // ---- integrate velocities (integrators/euler.mojo:82-130)
    if (im != 0.0f) {
        vx = vx + (fx * im + gx) * dt;
        vy = vy + (fy * im + gy) * dt;
        w = w + tau * ii * dt;
    }
    // ---- what stays fixed during the velocity phase: lever arms and effective masses of my contacts
    // (solvers/impulse.mojo:115-190), kept in the records ...
    RegBodies<OneBody> B1;
    B1.x[0] = x; B1.y[0] = y; B1.ang[0] = ang; B1.vx[0] = vx; B1.vy[0] = vy; B1.w[0] = w; B1.im[0] = im; B1.ii[0] = ii;
    for (unsigned m = mine; m; m &= m - 1) {
        const int c = __ffs((int)m) - 1;
        float *C = contacts + c * CONTACT_SIZE;
        const ContactFixed f = contact_prepare<OneBody>(B1, 0, C[C_PX], C[C_PY], C[C_NX], C[C_NY]);
        C[C_PX] = f.ra_x; C[C_PY] = f.ra_y;
        float *K = contacts + L::MAX_CONTACTS * CONTACT_SIZE + 4 * c;
        K[0] = f.k; K[1] = f.k_t; K[2] = f.rk; K[3] = f.rk_t;
    }
    // ... and the joint's lever arms, K^-1 and limit angle (joints/revolute.mojo:90-200), by the child
    float sin_a, cos_a;
    sincos32(ang, sin_a, cos_a);
    const float p_sin = from_parent(sin_a, b), p_cos = from_parent(cos_a, b), p_ang = from_parent(ang, b);
    const float rax = lax * p_cos - lay * p_sin, ray = lax * p_sin + lay * p_cos;
    const float rbx = lbx * cos_a - lby * sin_a, rby = lbx * sin_a + lby * cos_a;
    float inv_k11, inv_k12, inv_k22;
    {
        const float inv_ma = p_im, inv_ia = p_ii, inv_mb = im, inv_ib = ii;
        const float k11 = inv_ma + inv_mb + inv_ia * ray * ray + inv_ib * rby * rby;
        const float k12 = -inv_ia * rax * ray - inv_ib * rbx * rby;
        const float k22 = inv_ma + inv_mb + inv_ia * rax * rax + inv_ib * rbx * rbx;
        float det = k11 * k22 - k12 * k12;
        if (det < 1e-10f) det = 1e-10f;
        const float inv_det = 1.0f / det;
        inv_k11 = k22 * inv_det; inv_k12 = -k12 * inv_det; inv_k22 = k11 * inv_det;
    }
    const float eff = p_ii + ii;
    const float reff = 1.0f / eff;   // the limit and motor terms of every sweep divide by eff (div_by)
    const float angle_error = (ang - p_ang) - jref;
    const float spring_term = -jstiff * angle_error;
    const float rel_angle = ang - p_ang - jref;

    // ---- velocity iterations: my contacts in list order, then the joints slot by slot
    for (int it = 0; it < 6; ++it) {
        for (unsigned m = mine; m; m &= m - 1) {
            const int c = __ffs((int)m) - 1;
            float *C = contacts + c * CONTACT_SIZE;
            ContactFixed f;
            f.nx = C[C_NX]; f.ny = C[C_NY]; f.ra_x = C[C_PX]; f.ra_y = C[C_PY];
            f.inv_mass_a = im; f.inv_inertia_a = ii;
            const float *K = contacts + L::MAX_CONTACTS * CONTACT_SIZE + 4 * c;
            f.k = K[0]; f.k_t = K[1]; f.rk = K[2]; f.rk_t = K[3];
            float jn = C[C_JN], jt = C[C_JT];
            B1.vx[0] = vx; B1.vy[0] = vy; B1.w[0] = w;
            contact_velocity<OneBody>(B1, 0, f, jn, jt, friction, restitution);
            vx = B1.vx[0]; vy = B1.vy[0]; w = B1.w[0];
            C[C_JN] = jn; C[C_JT] = jt;
        }
#pragma unroll
        for (int s = 0; s < 3; ++s) {
            // joints/revolute.mojo:100-320 for the joint whose child I am, when its slot is s
            const float vxa = from_parent(vx, b), vya = from_parent(vy, b), wa = from_parent(w, b);
            const float inv_ma = p_im, inv_ia = p_ii, inv_mb = im, inv_ib = ii;
            const float vxb = vx, vyb = vy, wb = w;
            const float va_anchor_x = vxa - wa * ray, va_anchor_y = vya + wa * rax;
            const float vb_anchor_x = vxb - wb * rby, vb_anchor_y = vyb + wb * rbx;
            const float cdot_x = vb_anchor_x - va_anchor_x, cdot_y = vb_anchor_y - va_anchor_y;
            const float impulse_x = -(inv_k11 * cdot_x + inv_k12 * cdot_y);
            const float impulse_y = -(inv_k12 * cdot_x + inv_k22 * cdot_y);
            const float n_vxa = vxa - inv_ma * impulse_x, n_vya = vya - inv_ma * impulse_y;
            const float n_vxb = vxb + inv_mb * impulse_x, n_vyb = vyb + inv_mb * impulse_y;
            float cur_wa = wa - inv_ia * (rax * impulse_y - ray * impulse_x);
            float cur_wb = wb + inv_ib * (rbx * impulse_y - rby * impulse_x);
            const float e = eff;
            if (jflags & JF_SPRING) {
                const float rel_omega = wb - wa;
                const float spring_torque = spring_term - jdamp * rel_omega;
                const float angular_impulse = spring_torque * dt;
                if (e > 1e-10f) {
                    cur_wa = cur_wa - div_by(inv_ia * angular_impulse, e, reff);
                    cur_wb = cur_wb + div_by(inv_ib * angular_impulse, e, reff);
                }
            }
            if (jflags & JF_LIMIT) {
                const float rel_omega = cur_wb - cur_wa;
                if (e > 1e-10f) {
                    float limit_impulse = 0.0f;
                    const float stop = div_by(-rel_omega, e, reff);   // the same quotient on both sides of the test
                    if (rel_angle <= jlo) {
                        if (rel_omega < 0.0f) limit_impulse = stop;
                    } else if (rel_angle >= jhi) {
                        if (rel_omega > 0.0f) limit_impulse = stop;
                    }
                    if (limit_impulse != 0.0f) {
                        cur_wa = cur_wa - inv_ia * limit_impulse;
                        cur_wb = cur_wb + inv_ib * limit_impulse;
                    }
                }
            }
            if (jflags & JF_MOTOR) {
                const float rel_omega = cur_wb - cur_wa;
                const float speed_error = motor_speed - rel_omega;
                if (e > 1e-10f) {
                    float motor_impulse = div_by(speed_error, e, reff);
                    const float max_impulse = max_torque * dt;
                    if (motor_impulse > max_impulse) motor_impulse = max_impulse;
                    if (motor_impulse < -max_impulse) motor_impulse = -max_impulse;
                    cur_wa = cur_wa - inv_ia * motor_impulse;
                    cur_wb = cur_wb + inv_ib * motor_impulse;
                }
            }
            // the parent takes its new velocity from the child of this slot, the child keeps its own
            const float g_vx = from_kid(s, n_vxa, b), g_vy = from_kid(s, n_vya, b), g_w = from_kid(s, cur_wa, b);
            if ((kidmask >> s) & 1) { vx = g_vx; vy = g_vy; w = g_w; }
            if (myslot == s) { vx = n_vxb; vy = n_vyb; w = cur_wb; }
        }
    }
    // ---- integrate positions (integrators/euler.mojo:132-183)
    if (im != 0.0f) {
        const float pi_val = (float)3.14159265358979323846;
        const float two_pi = (float)(2.0 * 3.14159265358979323846);
        x = x + vx * dt;
        y = y + vy * dt;
        float angle = ang + w * dt;
        if (angle > 100.0f || angle < -100.0f) {
            angle = 0.0f;
        } else if (angle > pi_val) {
            angle = angle - two_pi;
            if (angle > pi_val) angle = angle - two_pi;
        } else if (angle < -pi_val) {
            angle = angle + two_pi;
            if (angle < -pi_val) angle = angle + two_pi;
        }
        ang = angle;
    }
    sincos32(ang, sin_a, cos_a);
    // ---- position iterations: my contacts (solvers/impulse.mojo:333-402), then the joints
    // (joints/revolute.mojo:323-495) slot by slot
    for (int it = 0; it < 2; ++it) {
        for (unsigned m = mine; m; m &= m - 1) {
            const int c = __ffs((int)m) - 1;
            const float *C = contacts + c * CONTACT_SIZE;
            B1.x[0] = x; B1.y[0] = y;
            contact_position<OneBody>(B1, 0, C[C_NX], C[C_NY], C[C_DEPTH], baumgarte, slop);
            x = B1.x[0]; y = B1.y[0];
        }
#pragma unroll
        for (int s = 0; s < 3; ++s) {
            const float xa = from_parent(x, b), ya = from_parent(y, b), angle_a = from_parent(ang, b);
            const float inv_ma = p_im, inv_ia = p_ii, inv_mb = im, inv_ib = ii;
            const float xb = x, yb = y, angle_b = ang;
            const float s_a = from_parent(sin_a, b), c_a = from_parent(cos_a, b);
            const float s_b = sin_a, c_b = cos_a;
            const float r_ax = lax * c_a - lay * s_a, r_ay = lax * s_a + lay * c_a;
            const float r_bx = lbx * c_b - lby * s_b, r_by = lbx * s_b + lby * c_b;
            const float anchor_ax = xa + r_ax, anchor_ay = ya + r_ay;
            const float anchor_bx = xb + r_bx, anchor_by = yb + r_by;
            const float cx = anchor_bx - anchor_ax, cy = anchor_by - anchor_ay;
            const float error = sqrtf(cx * cx + cy * cy);
            float n_xa = xa, n_ya = ya, n_aa = angle_a, n_xb = xb, n_yb = yb, n_ab = angle_b;
            if (!(error < slop)) {
                const float k11 = inv_ma + inv_mb + inv_ia * r_ay * r_ay + inv_ib * r_by * r_by;
                const float k12 = -inv_ia * r_ax * r_ay - inv_ib * r_bx * r_by;
                const float k22 = inv_ma + inv_mb + inv_ia * r_ax * r_ax + inv_ib * r_bx * r_bx;
                float det = k11 * k22 - k12 * k12;
                if (det < 1e-10f) det = 1e-10f;
                const float inv_det = 1.0f / det;
                const float ik11 = k22 * inv_det, ik12 = -k12 * inv_det, ik22 = k11 * inv_det;
                const float correction_x = -baumgarte * (ik11 * cx + ik12 * cy);
                const float correction_y = -baumgarte * (ik12 * cx + ik22 * cy);
                n_xa = xa - inv_ma * correction_x;
                n_ya = ya - inv_ma * correction_y;
                n_xb = xb + inv_mb * correction_x;
                n_yb = yb + inv_mb * correction_y;
                float cur_a = angle_a - inv_ia * (r_ax * correction_y - r_ay * correction_x);
                float cur_b = angle_b + inv_ib * (r_bx * correction_y - r_by * correction_x);
                if (jflags & JF_LIMIT) {
                    const float relative_angle = cur_b - cur_a - jref;
                    const float e = inv_ia + inv_ib;
                    if (e > 1e-10f) {
                        float angle_correction = 0.0f;
                        if (relative_angle < jlo) angle_correction = baumgarte * (jlo - relative_angle);
                        else if (relative_angle > jhi) angle_correction = baumgarte * (jhi - relative_angle);
                        if (angle_correction != 0.0f) {
                            cur_a = cur_a - div_by(inv_ia * angle_correction, e, reff);
                            cur_b = cur_b + div_by(inv_ib * angle_correction, e, reff);
                        }
                    }
                }
                n_aa = cur_a;
                n_ab = cur_b;
            }
            const float g_x = from_kid(s, n_xa, b), g_y = from_kid(s, n_ya, b), g_a = from_kid(s, n_aa, b);
            if ((kidmask >> s) & 1) { x = g_x; y = g_y; ang = g_a; }
            if (myslot == s) { x = n_xb; y = n_yb; ang = n_ab; }
            // (the last slot moves leg 2's segments only: the second iteration reads them in its last two slots,
            // behind another of these, and nothing reads them after the second iteration)
            if (s != 2) sincos32(ang, sin_a, cos_a);
        }
    }
    // ---- bodies and cleared forces back into the row
    if (body) {
        Bp[IDX_X] = x; Bp[IDX_Y] = y; Bp[IDX_ANGLE] = ang; Bp[IDX_VX] = vx; Bp[IDX_VY] = vy; Bp[IDX_OMEGA] = w;
        row[L::FORCES_OFF + b * 3] = 0.0f; row[L::FORCES_OFF + b * 3 + 1] = 0.0f; row[L::FORCES_OFF + b * 3 + 2] = 0.0f;
    }
    // ---- observation entries 0 .. 7 and 9 .. 12 (observe_state: the same expressions on the same values), every
    // body's lane its own: the hull 0 .. 3, a leg segment its angle and angular velocity against its parent's.
    // The contact flags (8, 13) and the lidar are left to what follows (step_tail<false, false>).
    {
        const double p_ang = (double)from_parent(ang, b), p_w = (double)from_parent(w, b);
        if (b == 0) {
            const double hull_angle = ang, hull_omega = w, hull_vx = vx, hull_vy = vy;
            row[0] = (float)hull_angle;
            row[1] = (float)(hull_omega / 5.0);
            row[2] = (float)(hull_vx * (600.0 / SCALE) / FPS);
            row[3] = (float)(hull_vy * (400.0 / SCALE) / FPS);
        } else if (b <= 4) {
            const int leg = (b - 1) >> 1, at = 4 + 5 * leg + (((b - 1) & 1) ? 2 : 0);
            row[at] = (float)(((double)ang - p_ang) / 1.0);
            row[at + 1] = (float)(((double)w - p_w) / 10.0);
        }
    }
}

}  // namespace bw
}  // namespace mrl
