// Register-resident form of the physics2d solver sweeps.
//
// The Gauss-Seidel sweeps touch the same few bodies over and over (6 velocity + 2 position
// iterations, each over every contact and joint).  Running them out of LDS makes every sweep a
// chain of dependent LDS round trips; here the dynamic body state, the contact list and the joint
// table are loaded into registers once per step, all sweeps run on registers, and the bodies are
// written back once.  A body is picked by its (runtime) index with a select chain over the
// NUM_BODIES register copies; contacts and joints are walked with fully unrolled, predicated
// loops so that every array index is a compile-time constant.
//
// The arithmetic is that of physics2d.hpp statement for statement (same operations, same order),
// so both forms give identical results.  Contacts are body-vs-ground only (body B = -1), which is
// all the terrain detectors ever emit.
#pragma once
#include "physics2d.hpp"

namespace mrl {

template <int N>
MRL_DEV float sel(const float (&a)[N], int i) {
    float r = a[0];
#pragma unroll
    for (int k = 1; k < N; ++k) r = (i == k) ? a[k] : r;
    return r;
}

template <int N>
MRL_DEV void put(float (&a)[N], int i, float v) {
#pragma unroll
    for (int k = 0; k < N; ++k) a[k] = (i == k) ? v : a[k];
}

template <class L>
struct RegBodies {
    static constexpr int NB = L::NUM_BODIES;
    float x[NB], y[NB], ang[NB], vx[NB], vy[NB], w[NB], im[NB], ii[NB];

    MRL_DEV void load(const float *row) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const float *B = row + L::BODIES_OFF + b * BODY_SIZE;
            x[b] = B[IDX_X]; y[b] = B[IDX_Y]; ang[b] = B[IDX_ANGLE];
            vx[b] = B[IDX_VX]; vy[b] = B[IDX_VY]; w[b] = B[IDX_OMEGA];
            im[b] = B[IDX_INV_MASS]; ii[b] = B[IDX_INV_INERTIA];
        }
    }
    MRL_DEV void store(float *row) const {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            float *B = row + L::BODIES_OFF + b * BODY_SIZE;
            B[IDX_X] = x[b]; B[IDX_Y] = y[b]; B[IDX_ANGLE] = ang[b];
            B[IDX_VX] = vx[b]; B[IDX_VY] = vy[b]; B[IDX_OMEGA] = w[b];
        }
    }
};

template <class L>
struct RegContacts {
    static constexpr int MC = L::MAX_CONTACTS;
    int n;
    int body[MC];
    float px[MC], py[MC], nx[MC], ny[MC], depth[MC], jn[MC], jt[MC];

    MRL_DEV void load(const float *contacts, int count) {
        n = count;
#pragma unroll
        for (int c = 0; c < MC; ++c) {
            body[c] = 0;
            px[c] = py[c] = nx[c] = ny[c] = depth[c] = jn[c] = jt[c] = 0.0f;
            if (c < count) {
                const float *C = contacts + c * CONTACT_SIZE;
                body[c] = (int)C[C_BODY_A];
                px[c] = C[C_PX]; py[c] = C[C_PY]; nx[c] = C[C_NX]; ny[c] = C[C_NY];
                depth[c] = C[C_DEPTH]; jn[c] = C[C_JN]; jt[c] = C[C_JT];
            }
        }
    }
};

template <class L>
struct RegJoints {
    static constexpr int MJ = L::MAX_JOINTS;
    int n;
    bool active[MJ];
    int ba[MJ], bb[MJ], flags[MJ];
    float lax[MJ], lay[MJ], lbx[MJ], lby[MJ], ref[MJ], lo[MJ], hi[MJ], max_torque[MJ], motor_speed[MJ],
        stiff[MJ], damp[MJ];
    float rax[MJ], ray[MJ], rbx[MJ], rby[MJ];  // world anchor offsets, valid while angles are fixed

    MRL_DEV void load(const float *row) {
        n = (int)row[L::JOINT_COUNT_OFF];
#pragma unroll
        for (int j = 0; j < MJ; ++j) {
            const float *J = row + L::JOINTS_OFF + j * JOINT_SIZE;
            active[j] = (j < n) && ((int)J[J_TYPE] == 0);
            ba[j] = (int)J[J_BODY_A]; bb[j] = (int)J[J_BODY_B]; flags[j] = (int)J[J_FLAGS];
            lax[j] = J[J_AX]; lay[j] = J[J_AY]; lbx[j] = J[J_BX]; lby[j] = J[J_BY];
            ref[j] = J[J_REF]; lo[j] = J[J_LO]; hi[j] = J[J_HI];
            max_torque[j] = J[J_MAX_TORQUE]; motor_speed[j] = J[J_MOTOR_SPEED];
            stiff[j] = J[J_STIFF]; damp[j] = J[J_DAMP];
            rax[j] = ray[j] = rbx[j] = rby[j] = 0.0f;
        }
    }
};

template <class L>
MRL_DEV void reg_integrate_velocities(RegBodies<L> &B, const float *row, float gx, float gy, float dt) {
#pragma unroll
    for (int b = 0; b < L::NUM_BODIES; ++b) {
        if (B.im[b] == 0.0f) continue;
        const float *F = row + L::FORCES_OFF + b * 3;
        B.vx[b] = B.vx[b] + (F[0] * B.im[b] + gx) * dt;
        B.vy[b] = B.vy[b] + (F[1] * B.im[b] + gy) * dt;
        B.w[b] = B.w[b] + F[2] * B.ii[b] * dt;
    }
}

template <class L>
MRL_DEV void reg_integrate_positions(RegBodies<L> &B, float dt) {
    const float pi_val = (float)3.14159265358979323846;
    const float two_pi = (float)(2.0 * 3.14159265358979323846);
#pragma unroll
    for (int b = 0; b < L::NUM_BODIES; ++b) {
        if (B.im[b] == 0.0f) continue;
        float x = B.x[b] + B.vx[b] * dt;
        float y = B.y[b] + B.vy[b] * dt;
        float angle = B.ang[b] + B.w[b] * dt;
        if (angle > 100.0f || angle < -100.0f) {
            angle = 0.0f;
        } else if (angle > pi_val) {
            angle = angle - two_pi;
            if (angle > pi_val) angle = angle - two_pi;
        } else if (angle < -pi_val) {
            angle = angle + two_pi;
            if (angle < -pi_val) angle = angle + two_pi;
        }
        B.x[b] = x; B.y[b] = y; B.ang[b] = angle;
    }
}

template <class L>
MRL_DEV void reg_contact_solve_velocity(RegBodies<L> &B, RegContacts<L> &C, float friction,
                                        float restitution) {
#pragma unroll
    for (int c = 0; c < L::MAX_CONTACTS; ++c) {
        if (c >= C.n) break;
        const int ia = C.body[c];
        const float point_x = C.px[c], point_y = C.py[c], normal_x = C.nx[c], normal_y = C.ny[c];
        const float pos_a_x = sel(B.x, ia), pos_a_y = sel(B.y, ia);
        float vel_a_x = sel(B.vx, ia), vel_a_y = sel(B.vy, ia), omega_a = sel(B.w, ia);
        const float inv_mass_a = sel(B.im, ia), inv_inertia_a = sel(B.ii, ia);
        const float inv_mass_b = 0.0f, inv_inertia_b = 0.0f, vel_b_x = 0.0f, vel_b_y = 0.0f, omega_b = 0.0f;
        const float ra_x = point_x - pos_a_x, ra_y = point_y - pos_a_y;
        const float rb_x = point_x - point_x, rb_y = point_y - point_y;
        float vel_at_a_x = vel_a_x - omega_a * ra_y, vel_at_a_y = vel_a_y + omega_a * ra_x;
        float vel_at_b_x = vel_b_x - omega_b * rb_y, vel_at_b_y = vel_b_y + omega_b * rb_x;
        float rel_vel_x = vel_at_a_x - vel_at_b_x, rel_vel_y = vel_at_a_y - vel_at_b_y;
        const float vel_normal = rel_vel_x * normal_x + rel_vel_y * normal_y;
        if (!(vel_normal < 0.0f)) continue;

        const float ra_cross_n = ra_x * normal_y - ra_y * normal_x;
        const float rb_cross_n = rb_x * normal_y - rb_y * normal_x;
        float k = inv_mass_a + inv_mass_b;
        k = k + inv_inertia_a * ra_cross_n * ra_cross_n;
        k = k + inv_inertia_b * rb_cross_n * rb_cross_n;
        float j_normal = -(1.0f + restitution) * vel_normal / k;
        const float old_impulse = C.jn[c];
        float new_impulse = old_impulse + j_normal;
        if (new_impulse < 0.0f) new_impulse = 0.0f;
        C.jn[c] = new_impulse;
        j_normal = new_impulse - old_impulse;
        const float impulse_x = j_normal * normal_x, impulse_y = j_normal * normal_y;
        vel_a_x = vel_a_x + impulse_x * inv_mass_a;
        vel_a_y = vel_a_y + impulse_y * inv_mass_a;
        omega_a = omega_a + (ra_x * impulse_y - ra_y * impulse_x) * inv_inertia_a;
        vel_at_a_x = vel_a_x - omega_a * ra_y; vel_at_a_y = vel_a_y + omega_a * ra_x;
        vel_at_b_x = vel_b_x - omega_b * rb_y; vel_at_b_y = vel_b_y + omega_b * rb_x;
        rel_vel_x = vel_at_a_x - vel_at_b_x; rel_vel_y = vel_at_a_y - vel_at_b_y;

        const float tangent_x = -normal_y, tangent_y = normal_x;
        const float vel_tangent = rel_vel_x * tangent_x + rel_vel_y * tangent_y;
        const float ra_cross_t = ra_x * tangent_y - ra_y * tangent_x;
        const float rb_cross_t = rb_x * tangent_y - rb_y * tangent_x;
        float k_t = inv_mass_a + inv_mass_b;
        k_t = k_t + inv_inertia_a * ra_cross_t * ra_cross_t;
        k_t = k_t + inv_inertia_b * rb_cross_t * rb_cross_t;
        float j_tangent = -vel_tangent / k_t;
        const float max_friction = friction * new_impulse;
        const float old_tangent = C.jt[c];
        float new_tangent = old_tangent + j_tangent;
        if (new_tangent > max_friction) new_tangent = max_friction;
        else if (new_tangent < -max_friction) new_tangent = -max_friction;
        C.jt[c] = new_tangent;
        j_tangent = new_tangent - old_tangent;
        const float friction_x = j_tangent * tangent_x, friction_y = j_tangent * tangent_y;
        put(B.vx, ia, vel_a_x + friction_x * inv_mass_a);
        put(B.vy, ia, vel_a_y + friction_y * inv_mass_a);
        put(B.w, ia, omega_a + (ra_x * friction_y - ra_y * friction_x) * inv_inertia_a);
    }
}

template <class L>
MRL_DEV void reg_contact_solve_position(RegBodies<L> &B, const RegContacts<L> &C, float baumgarte,
                                        float slop) {
#pragma unroll
    for (int c = 0; c < L::MAX_CONTACTS; ++c) {
        if (c >= C.n) break;
        float correction = C.depth[c] - slop;
        if (correction <= 0.0f) continue;
        correction = baumgarte * correction;
        const int ia = C.body[c];
        const float inv_mass_a = sel(B.im, ia);
        const float inv_mass_b = 0.0f;
        const float total = inv_mass_a + inv_mass_b;
        if (total == 0.0f) continue;
        const float correction_a = correction * inv_mass_a / total;
        put(B.x, ia, sel(B.x, ia) + C.nx[c] * correction_a);
        put(B.y, ia, sel(B.y, ia) + C.ny[c] * correction_a);
    }
}

template <class L>
MRL_DEV void reg_joint_anchor(const RegBodies<L> &B, const RegJoints<L> &J, int j, float &rax, float &ray,
                              float &rbx, float &rby) {
    float sin_a, cos_a, sin_b, cos_b;
    sincos32(sel(B.ang, J.ba[j]), sin_a, cos_a);
    sincos32(sel(B.ang, J.bb[j]), sin_b, cos_b);
    rax = J.lax[j] * cos_a - J.lay[j] * sin_a; ray = J.lax[j] * sin_a + J.lay[j] * cos_a;
    rbx = J.lbx[j] * cos_b - J.lby[j] * sin_b; rby = J.lbx[j] * sin_b + J.lby[j] * cos_b;
}

template <class L>
MRL_DEV void reg_joint_anchors_all(const RegBodies<L> &B, RegJoints<L> &J) {
#pragma unroll
    for (int j = 0; j < L::MAX_JOINTS; ++j)
        if (J.active[j]) reg_joint_anchor<L>(B, J, j, J.rax[j], J.ray[j], J.rbx[j], J.rby[j]);
}

template <class L>
MRL_DEV void reg_joint_solve_velocity(RegBodies<L> &B, const RegJoints<L> &J, float dt) {
#pragma unroll
    for (int j = 0; j < L::MAX_JOINTS; ++j) {
        if (!J.active[j]) continue;
        const int a = J.ba[j], b = J.bb[j];
        const float angle_a = sel(B.ang, a), vxa = sel(B.vx, a), vya = sel(B.vy, a), wa = sel(B.w, a);
        const float inv_ma = sel(B.im, a), inv_ia = sel(B.ii, a);
        const float angle_b = sel(B.ang, b), vxb = sel(B.vx, b), vyb = sel(B.vy, b), wb = sel(B.w, b);
        const float inv_mb = sel(B.im, b), inv_ib = sel(B.ii, b);
        const float rax = J.rax[j], ray = J.ray[j], rbx = J.rbx[j], rby = J.rby[j];
        const float va_anchor_x = vxa - wa * ray, va_anchor_y = vya + wa * rax;
        const float vb_anchor_x = vxb - wb * rby, vb_anchor_y = vyb + wb * rbx;
        const float cdot_x = vb_anchor_x - va_anchor_x, cdot_y = vb_anchor_y - va_anchor_y;
        const float k11 = inv_ma + inv_mb + inv_ia * ray * ray + inv_ib * rby * rby;
        const float k12 = -inv_ia * rax * ray - inv_ib * rbx * rby;
        const float k22 = inv_ma + inv_mb + inv_ia * rax * rax + inv_ib * rbx * rbx;
        float det = k11 * k22 - k12 * k12;
        if (det < 1e-10f) det = 1e-10f;
        const float inv_det = 1.0f / det;
        const float inv_k11 = k22 * inv_det, inv_k12 = -k12 * inv_det, inv_k22 = k11 * inv_det;
        const float impulse_x = -(inv_k11 * cdot_x + inv_k12 * cdot_y);
        const float impulse_y = -(inv_k12 * cdot_x + inv_k22 * cdot_y);
        put(B.vx, a, vxa - inv_ma * impulse_x);
        put(B.vy, a, vya - inv_ma * impulse_y);
        put(B.vx, b, vxb + inv_mb * impulse_x);
        put(B.vy, b, vyb + inv_mb * impulse_y);
        float cur_wa = wa - inv_ia * (rax * impulse_y - ray * impulse_x);
        float cur_wb = wb + inv_ib * (rbx * impulse_y - rby * impulse_x);

        const int flags = J.flags[j];
        const float eff = inv_ia + inv_ib;
        if (flags & JF_SPRING) {
            const float angle_error = (angle_b - angle_a) - J.ref[j];
            const float rel_omega = wb - wa;  // angular velocities from before the point impulse
            const float spring_torque = -J.stiff[j] * angle_error - J.damp[j] * rel_omega;
            const float angular_impulse = spring_torque * dt;
            if (eff > 1e-10f) {
                cur_wa = cur_wa - inv_ia * angular_impulse / eff;
                cur_wb = cur_wb + inv_ib * angular_impulse / eff;
            }
        }
        if (flags & JF_LIMIT) {
            const float relative_angle = angle_b - angle_a - J.ref[j];
            const float rel_omega = cur_wb - cur_wa;
            if (eff > 1e-10f) {
                float limit_impulse = 0.0f;
                if (relative_angle <= J.lo[j]) {
                    if (rel_omega < 0.0f) limit_impulse = -rel_omega / eff;
                } else if (relative_angle >= J.hi[j]) {
                    if (rel_omega > 0.0f) limit_impulse = -rel_omega / eff;
                }
                if (limit_impulse != 0.0f) {
                    cur_wa = cur_wa - inv_ia * limit_impulse;
                    cur_wb = cur_wb + inv_ib * limit_impulse;
                }
            }
        }
        if (flags & JF_MOTOR) {
            const float rel_omega = cur_wb - cur_wa;
            const float speed_error = J.motor_speed[j] - rel_omega;
            if (eff > 1e-10f) {
                float motor_impulse = speed_error / eff;
                const float max_impulse = J.max_torque[j] * dt;
                if (motor_impulse > max_impulse) motor_impulse = max_impulse;
                if (motor_impulse < -max_impulse) motor_impulse = -max_impulse;
                cur_wa = cur_wa - inv_ia * motor_impulse;
                cur_wb = cur_wb + inv_ib * motor_impulse;
            }
        }
        put(B.w, a, cur_wa);
        put(B.w, b, cur_wb);
    }
}

template <class L>
MRL_DEV void reg_joint_solve_position(RegBodies<L> &B, const RegJoints<L> &J, float baumgarte, float slop) {
#pragma unroll
    for (int j = 0; j < L::MAX_JOINTS; ++j) {
        if (!J.active[j]) continue;
        const int a = J.ba[j], b = J.bb[j];
        const float xa = sel(B.x, a), ya = sel(B.y, a), angle_a = sel(B.ang, a);
        const float inv_ma = sel(B.im, a), inv_ia = sel(B.ii, a);
        const float xb = sel(B.x, b), yb = sel(B.y, b), angle_b = sel(B.ang, b);
        const float inv_mb = sel(B.im, b), inv_ib = sel(B.ii, b);
        float rax, ray, rbx, rby;
        reg_joint_anchor<L>(B, J, j, rax, ray, rbx, rby);
        const float anchor_ax = xa + rax, anchor_ay = ya + ray;
        const float anchor_bx = xb + rbx, anchor_by = yb + rby;
        const float cx = anchor_bx - anchor_ax, cy = anchor_by - anchor_ay;
        const float error = sqrtf(cx * cx + cy * cy);
        if (error < slop) continue;
        const float k11 = inv_ma + inv_mb + inv_ia * ray * ray + inv_ib * rby * rby;
        const float k12 = -inv_ia * rax * ray - inv_ib * rbx * rby;
        const float k22 = inv_ma + inv_mb + inv_ia * rax * rax + inv_ib * rbx * rbx;
        float det = k11 * k22 - k12 * k12;
        if (det < 1e-10f) det = 1e-10f;
        const float inv_det = 1.0f / det;
        const float inv_k11 = k22 * inv_det, inv_k12 = -k12 * inv_det, inv_k22 = k11 * inv_det;
        const float correction_x = -baumgarte * (inv_k11 * cx + inv_k12 * cy);
        const float correction_y = -baumgarte * (inv_k12 * cx + inv_k22 * cy);
        put(B.x, a, xa - inv_ma * correction_x);
        put(B.y, a, ya - inv_ma * correction_y);
        put(B.x, b, xb + inv_mb * correction_x);
        put(B.y, b, yb + inv_mb * correction_y);
        float cur_a = angle_a - inv_ia * (rax * correction_y - ray * correction_x);
        float cur_b = angle_b + inv_ib * (rbx * correction_y - rby * correction_x);
        if (J.flags[j] & JF_LIMIT) {
            const float relative_angle = cur_b - cur_a - J.ref[j];
            const float eff = inv_ia + inv_ib;
            if (eff > 1e-10f) {
                float angle_correction = 0.0f;
                if (relative_angle < J.lo[j]) angle_correction = baumgarte * (J.lo[j] - relative_angle);
                else if (relative_angle > J.hi[j]) angle_correction = baumgarte * (J.hi[j] - relative_angle);
                if (angle_correction != 0.0f) {
                    cur_a = cur_a - inv_ia * angle_correction / eff;
                    cur_b = cur_b + inv_ib * angle_correction / eff;
                }
            }
        }
        put(B.ang, a, cur_a);
        put(B.ang, b, cur_b);
    }
}

// One physics step (or sub-step) of an env row with the sweeps on registers.  `row` must hold the
// current bodies / joints; contacts are detected into the LDS scratch (detection order and the
// MAX_CONTACTS cut-off unchanged), then everything iterative runs on registers.
template <class L, bool FLAT>
MRL_DEV int reg_physics_substep(float *row, const float *shapes, float *contacts, float gx, float gy,
                                float dt, float friction, float restitution, float baumgarte, float slop,
                                int vel_iters, int pos_iters) {
    RegBodies<L> B;
    B.load(row);
    reg_integrate_velocities<L>(B, row, gx, gy, dt);
    // the detectors read positions and angles only, which the velocity update has not touched
    const int n = FLAT ? flat_detect<L>(row, shapes, 0.0f, contacts) : edge_detect<L>(row, shapes, contacts);
    RegContacts<L> C;
    C.load(contacts, n);
    RegJoints<L> J;
    J.load(row);
    reg_joint_anchors_all<L>(B, J);
    for (int it = 0; it < vel_iters; ++it) {
        reg_contact_solve_velocity<L>(B, C, friction, restitution);
        reg_joint_solve_velocity<L>(B, J, dt);
    }
    reg_integrate_positions<L>(B, dt);
    for (int it = 0; it < pos_iters; ++it) {
        reg_contact_solve_position<L>(B, C, baumgarte, slop);
        reg_joint_solve_position<L>(B, J, baumgarte, slop);
    }
    B.store(row);
#pragma unroll
    for (int k = 0; k < L::NUM_BODIES * 3; ++k) row[L::FORCES_OFF + k] = 0.0f;
    return n;
}

}  // namespace mrl
