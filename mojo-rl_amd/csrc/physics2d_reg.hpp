// Register-resident form of the physics2d solver sweeps.
//
// The Gauss-Seidel sweeps touch the same few bodies over and over (4-6 velocity + 2 position
// iterations, each over every contact and joint).  Running them out of LDS makes every sweep a
// chain of dependent LDS round trips; here the dynamic body state and the joint table (and, for
// short contact lists, the contacts) are loaded into registers once per step, all sweeps run on
// registers, and the bodies are written back once.  A body is picked by its (runtime) index with
// a select chain over the NUM_BODIES register copies; joints (and register-resident contacts) are
// walked with fully unrolled, predicated loops so that every array index is a compile-time
// constant.
//
// Two further reductions, both value-preserving:
//   * whatever a velocity sweep recomputes from quantities that cannot change during the velocity
//     phase (positions, angles, masses: lever arms, effective masses, the joints' K^-1, spring
//     and limit terms) is computed once per step with the same expressions;
//   * an env whose joints always connect the same bodies passes that wiring as a compile-time
//     topology; the select chains then fold away.  The row's joint table is compared against it
//     first and the generic path is taken if any lane disagrees.
//
// The arithmetic is that of physics2d.hpp statement for statement (same operations, same order),
// so both forms give identical results.  Contacts are body-vs-ground only (body B = -1), which is
// all the terrain detectors ever emit.
#pragma once
#include <type_traits>
#include <utility>
#include "physics2d.hpp"

namespace mrl {

// floats of LDS scratch per contact: the 9-float record plus four slots for the two effective masses
// and their reciprocals
constexpr int CONTACT_SCRATCH = CONTACT_SIZE + 4;

// Per-body quantities of an env live in short vector values (ext_vector_type), not in arrays:
// reading or replacing one element of a vector is an operation on the whole value, so the
// compiler keeps it in registers from the first pass on.  (Arrays indexed inside a loop only get
// constant indices after unrolling; by then selects of loads have been merged into loads from a
// computed address, and the whole struct stays in memory.)
template <int N>
struct BodyVec {
    static constexpr int W = N <= 2 ? 2 : N <= 4 ? 4 : N <= 8 ? 8 : 16;
    typedef float type __attribute__((ext_vector_type(W)));
};

// element i (runtime) of the first N lanes of a body vector, as a select chain
template <int N, class V, int... K>
MRL_DEV float sel_impl(const V &a, int i, std::integer_sequence<int, K...>) {
    float r = a[0];
    ((r = (i == K + 1) ? a[K + 1] : r), ...);
    return r;
}
template <int N, class V>
MRL_DEV float sel(const V &a, int i) {
    return sel_impl<N>(a, i, std::make_integer_sequence<int, N - 1>{});
}

// a[i] = v for runtime i < N
template <int N, class V, int... K>
MRL_DEV void put_impl(V &a, int i, float v, std::integer_sequence<int, K...>) {
    ((a[K] = (i == K) ? v : a[K]), ...);
}
template <int N, class V>
MRL_DEV void put(V &a, int i, float v) {
    put_impl<N>(a, i, v, std::make_integer_sequence<int, N>{});
}

// joint j connects bodies a(j) -> b(j); DynamicTopology reads them from the row
struct DynamicTopology {
    static constexpr bool STATIC = false;
    static constexpr MRL_DEV int a(int) { return 0; }
    static constexpr MRL_DEV int b(int) { return 0; }
};

template <class L>
struct RegBodies {
    static constexpr int NB = L::NUM_BODIES;
    typename BodyVec<NB>::type x, y, ang, vx, vy, w, im, ii;

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

// ---------------------------------------------------------------- contacts

// Everything about one contact that stays fixed during the velocity phase.
struct ContactFixed {
    float nx, ny, ra_x, ra_y, inv_mass_a, inv_inertia_a, k, k_t;
    float rk, rk_t;   // 1 / k and 1 / k_t: every sweep divides by the effective masses (div_by)
};

template <class L>
MRL_DEV ContactFixed contact_prepare(const RegBodies<L> &B, int ia, float point_x, float point_y,
                                     float normal_x, float normal_y) {
    ContactFixed f;
    f.nx = normal_x; f.ny = normal_y;
    f.inv_mass_a = sel<L::NUM_BODIES>(B.im, ia); f.inv_inertia_a = sel<L::NUM_BODIES>(B.ii, ia);
    const float inv_mass_b = 0.0f, inv_inertia_b = 0.0f;
    f.ra_x = point_x - sel<L::NUM_BODIES>(B.x, ia); f.ra_y = point_y - sel<L::NUM_BODIES>(B.y, ia);
    const float rb_x = point_x - point_x, rb_y = point_y - point_y;
    const float ra_cross_n = f.ra_x * normal_y - f.ra_y * normal_x;
    const float rb_cross_n = rb_x * normal_y - rb_y * normal_x;
    float k = f.inv_mass_a + inv_mass_b;
    k = k + f.inv_inertia_a * ra_cross_n * ra_cross_n;
    k = k + inv_inertia_b * rb_cross_n * rb_cross_n;
    f.k = k;
    const float tangent_x = -normal_y, tangent_y = normal_x;
    const float ra_cross_t = f.ra_x * tangent_y - f.ra_y * tangent_x;
    const float rb_cross_t = rb_x * tangent_y - rb_y * tangent_x;
    float k_t = f.inv_mass_a + inv_mass_b;
    k_t = k_t + f.inv_inertia_a * ra_cross_t * ra_cross_t;
    k_t = k_t + inv_inertia_b * rb_cross_t * rb_cross_t;
    f.k_t = k_t;
    f.rk = 1.0f / k;
    f.rk_t = 1.0f / k_t;
    return f;
}

// one contact of one velocity sweep; jn / jt are the accumulated impulses
template <class L>
MRL_DEV void contact_velocity(RegBodies<L> &B, int ia, const ContactFixed &f, float &jn, float &jt,
                              float friction, float restitution) {
    const float normal_x = f.nx, normal_y = f.ny, ra_x = f.ra_x, ra_y = f.ra_y;
    const float inv_mass_a = f.inv_mass_a, inv_inertia_a = f.inv_inertia_a;
    float vel_a_x = sel<L::NUM_BODIES>(B.vx, ia), vel_a_y = sel<L::NUM_BODIES>(B.vy, ia), omega_a = sel<L::NUM_BODIES>(B.w, ia);
    const float vel_b_x = 0.0f, vel_b_y = 0.0f, omega_b = 0.0f, rb_x = 0.0f, rb_y = 0.0f;
    float vel_at_a_x = vel_a_x - omega_a * ra_y, vel_at_a_y = vel_a_y + omega_a * ra_x;
    float vel_at_b_x = vel_b_x - omega_b * rb_y, vel_at_b_y = vel_b_y + omega_b * rb_x;
    float rel_vel_x = vel_at_a_x - vel_at_b_x, rel_vel_y = vel_at_a_y - vel_at_b_y;
    const float vel_normal = rel_vel_x * normal_x + rel_vel_y * normal_y;
    if (!(vel_normal < 0.0f)) return;

    float j_normal = div_by(-(1.0f + restitution) * vel_normal, f.k, f.rk);
    const float old_impulse = jn;
    float new_impulse = old_impulse + j_normal;
    if (new_impulse < 0.0f) new_impulse = 0.0f;
    jn = new_impulse;
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
    float j_tangent = div_by(-vel_tangent, f.k_t, f.rk_t);
    const float max_friction = friction * new_impulse;
    const float old_tangent = jt;
    float new_tangent = old_tangent + j_tangent;
    if (new_tangent > max_friction) new_tangent = max_friction;
    else if (new_tangent < -max_friction) new_tangent = -max_friction;
    jt = new_tangent;
    j_tangent = new_tangent - old_tangent;
    const float friction_x = j_tangent * tangent_x, friction_y = j_tangent * tangent_y;
    put<L::NUM_BODIES>(B.vx, ia, vel_a_x + friction_x * inv_mass_a);
    put<L::NUM_BODIES>(B.vy, ia, vel_a_y + friction_y * inv_mass_a);
    put<L::NUM_BODIES>(B.w, ia, omega_a + (ra_x * friction_y - ra_y * friction_x) * inv_inertia_a);
}

template <class L>
MRL_DEV void contact_position(RegBodies<L> &B, int ia, float normal_x, float normal_y, float depth,
                              float baumgarte, float slop) {
    float correction = depth - slop;
    if (correction <= 0.0f) return;
    correction = baumgarte * correction;
    const float inv_mass_a = sel<L::NUM_BODIES>(B.im, ia);
    const float inv_mass_b = 0.0f;
    const float total = inv_mass_a + inv_mass_b;
    if (total == 0.0f) return;
    const float correction_a = correction * inv_mass_a / total;
    put<L::NUM_BODIES>(B.x, ia, sel<L::NUM_BODIES>(B.x, ia) + normal_x * correction_a);
    put<L::NUM_BODIES>(B.y, ia, sel<L::NUM_BODIES>(B.y, ia) + normal_y * correction_a);
}

// contact list held in registers (short MAX_CONTACTS)
template <class L>
struct RegContacts {
    static constexpr int MC = L::MAX_CONTACTS;
    int n;
    int body[MC];
    float depth[MC], jn[MC], jt[MC];
    ContactFixed f[MC];

    MRL_DEV void load(const RegBodies<L> &B, float *contacts, int count) {
        n = count;
#pragma unroll
        for (int c = 0; c < MC; ++c) {
            body[c] = 0;
            depth[c] = jn[c] = jt[c] = 0.0f;
            f[c] = ContactFixed{0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 1.0f, 1.0f, 1.0f, 1.0f};
            if (c < count) {
                const float *C = contacts + c * CONTACT_SIZE;
                body[c] = (int)C[C_BODY_A];
                depth[c] = C[C_DEPTH]; jn[c] = C[C_JN]; jt[c] = C[C_JT];
                f[c] = contact_prepare<L>(B, body[c], C[C_PX], C[C_PY], C[C_NX], C[C_NY]);
            }
        }
    }
    MRL_DEV void velocity_sweep(RegBodies<L> &B, float friction, float restitution) {
#pragma unroll
        for (int c = 0; c < MC; ++c) {
            if (c >= n) break;
            contact_velocity<L>(B, body[c], f[c], jn[c], jt[c], friction, restitution);
        }
    }
    MRL_DEV void position_sweep(RegBodies<L> &B, float baumgarte, float slop) const {
#pragma unroll
        for (int c = 0; c < MC; ++c) {
            if (c >= n) break;
            contact_position<L>(B, body[c], f[c].nx, f[c].ny, depth[c], baumgarte, slop);
        }
    }
};

// Contact list left in the lane's LDS scratch (long lists).  After load() the record's contact
// point slots hold the lever arm (the only way the point enters a sweep) and four slots behind
// the MAX_CONTACTS records hold each contact's effective masses and their reciprocals; body indices, normals, depth
// and accumulated impulses stay where the detector put them.
template <class L>
struct LdsContacts {
    int n;
    float *cts;

    MRL_DEV float &k_slot(int c, int which) { return cts[L::MAX_CONTACTS * CONTACT_SIZE + 4 * c + which]; }

    MRL_DEV void load(const RegBodies<L> &B, float *contacts, int count) {
        n = count;
        cts = contacts;
        for (int c = 0; c < n; ++c) {
            float *C = cts + c * CONTACT_SIZE;
            const ContactFixed f = contact_prepare<L>(B, (int)C[C_BODY_A], C[C_PX], C[C_PY], C[C_NX], C[C_NY]);
            C[C_PX] = f.ra_x; C[C_PY] = f.ra_y;
            k_slot(c, 0) = f.k;
            k_slot(c, 1) = f.k_t;
            k_slot(c, 2) = f.rk;
            k_slot(c, 3) = f.rk_t;
        }
    }
    MRL_DEV void velocity_sweep(RegBodies<L> &B, float friction, float restitution) {
        for (int c = 0; c < n; ++c) {
            float *C = cts + c * CONTACT_SIZE;
            const int ia = (int)C[C_BODY_A];
            ContactFixed f;
            f.nx = C[C_NX]; f.ny = C[C_NY]; f.ra_x = C[C_PX]; f.ra_y = C[C_PY];
            f.inv_mass_a = sel<L::NUM_BODIES>(B.im, ia); f.inv_inertia_a = sel<L::NUM_BODIES>(B.ii, ia);
            f.k = k_slot(c, 0); f.k_t = k_slot(c, 1); f.rk = k_slot(c, 2); f.rk_t = k_slot(c, 3);
            float jn = C[C_JN], jt = C[C_JT];
            contact_velocity<L>(B, ia, f, jn, jt, friction, restitution);
            C[C_JN] = jn; C[C_JT] = jt;
        }
    }
    MRL_DEV void position_sweep(RegBodies<L> &B, float baumgarte, float slop) const {
        for (int c = 0; c < n; ++c) {
            const float *C = cts + c * CONTACT_SIZE;
            contact_position<L>(B, (int)C[C_BODY_A], C[C_NX], C[C_NY], C[C_DEPTH], baumgarte, slop);
        }
    }
};

// ---------------------------------------------------------------- joints

// Joint table of one env.  Only what the velocity sweeps need is held in registers (filled by
// prepare_velocity); the two position sweeps read their few parameters from the row as they go.
template <class L, class T>
struct RegJoints {
    static constexpr int MJ = L::MAX_JOINTS;
    bool active[MJ];
    int ba_[MJ], bb_[MJ], flags[MJ];
    float lo[MJ], hi[MJ], max_torque[MJ], motor_speed[MJ], damp[MJ];
    // fixed during the velocity phase
    float rax[MJ], ray[MJ], rbx[MJ], rby[MJ], inv_k11[MJ], inv_k12[MJ], inv_k22[MJ], eff[MJ], reff[MJ],
        spring_term[MJ], rel_angle[MJ];   // reff = 1 / eff: the spring, limit and motor terms all divide by eff (div_by)

    MRL_DEV int ba(int j) const { return T::STATIC ? T::a(j) : ba_[j]; }
    MRL_DEV int bb(int j) const { return T::STATIC ? T::b(j) : bb_[j]; }

    static MRL_DEV void anchor(const RegBodies<L> &B, const float *J, int a, int b, float &ax, float &ay,
                               float &bx, float &by) {
        float sin_a, cos_a, sin_b, cos_b;
        sincos32(sel<L::NUM_BODIES>(B.ang, a), sin_a, cos_a);
        sincos32(sel<L::NUM_BODIES>(B.ang, b), sin_b, cos_b);
        const float lax = J[J_AX], lay = J[J_AY], lbx = J[J_BX], lby = J[J_BY];
        ax = lax * cos_a - lay * sin_a; ay = lax * sin_a + lay * cos_a;
        bx = lbx * cos_b - lby * sin_b; by = lbx * sin_b + lby * cos_b;
    }

    // lever arms, K^-1 and the angle-dependent spring / limit terms for the velocity phase
    MRL_DEV void prepare_velocity(const RegBodies<L> &B, const float *row) {
        const int n = (int)row[L::JOINT_COUNT_OFF];
#pragma unroll
        for (int j = 0; j < MJ; ++j) {
            const float *J = row + L::JOINTS_OFF + j * JOINT_SIZE;
            active[j] = (j < n) && ((int)J[J_TYPE] == 0);
            ba_[j] = (int)J[J_BODY_A]; bb_[j] = (int)J[J_BODY_B]; flags[j] = (int)J[J_FLAGS];
            lo[j] = J[J_LO]; hi[j] = J[J_HI];
            max_torque[j] = J[J_MAX_TORQUE]; motor_speed[j] = J[J_MOTOR_SPEED]; damp[j] = J[J_DAMP];
            rax[j] = ray[j] = rbx[j] = rby[j] = inv_k11[j] = inv_k12[j] = inv_k22[j] = 0.0f;
            eff[j] = spring_term[j] = rel_angle[j] = 0.0f;
            reff[j] = 1.0f;
            if (!active[j]) continue;
            const int a = ba(j), b = bb(j);
            anchor(B, J, a, b, rax[j], ray[j], rbx[j], rby[j]);
            const float inv_ma = sel<L::NUM_BODIES>(B.im, a), inv_ia = sel<L::NUM_BODIES>(B.ii, a);
            const float inv_mb = sel<L::NUM_BODIES>(B.im, b), inv_ib = sel<L::NUM_BODIES>(B.ii, b);
            const float k11 = inv_ma + inv_mb + inv_ia * ray[j] * ray[j] + inv_ib * rby[j] * rby[j];
            const float k12 = -inv_ia * rax[j] * ray[j] - inv_ib * rbx[j] * rby[j];
            const float k22 = inv_ma + inv_mb + inv_ia * rax[j] * rax[j] + inv_ib * rbx[j] * rbx[j];
            float det = k11 * k22 - k12 * k12;
            if (det < 1e-10f) det = 1e-10f;
            const float inv_det = 1.0f / det;
            inv_k11[j] = k22 * inv_det; inv_k12[j] = -k12 * inv_det; inv_k22[j] = k11 * inv_det;
            eff[j] = inv_ia + inv_ib;
            reff[j] = 1.0f / eff[j];
            const float angle_a = sel<L::NUM_BODIES>(B.ang, a), angle_b = sel<L::NUM_BODIES>(B.ang, b);
            const float ref = J[J_REF];
            const float angle_error = (angle_b - angle_a) - ref;
            spring_term[j] = -J[J_STIFF] * angle_error;
            rel_angle[j] = angle_b - angle_a - ref;
        }
    }

    MRL_DEV void velocity_sweep(RegBodies<L> &B, float dt) const {
#pragma unroll
        for (int j = 0; j < MJ; ++j) {
            if (!active[j]) continue;
            const int a = ba(j), b = bb(j);
            const float vxa = sel<L::NUM_BODIES>(B.vx, a), vya = sel<L::NUM_BODIES>(B.vy, a), wa = sel<L::NUM_BODIES>(B.w, a);
            const float inv_ma = sel<L::NUM_BODIES>(B.im, a), inv_ia = sel<L::NUM_BODIES>(B.ii, a);
            const float vxb = sel<L::NUM_BODIES>(B.vx, b), vyb = sel<L::NUM_BODIES>(B.vy, b), wb = sel<L::NUM_BODIES>(B.w, b);
            const float inv_mb = sel<L::NUM_BODIES>(B.im, b), inv_ib = sel<L::NUM_BODIES>(B.ii, b);
            const float r_ax = rax[j], r_ay = ray[j], r_bx = rbx[j], r_by = rby[j];
            const float va_anchor_x = vxa - wa * r_ay, va_anchor_y = vya + wa * r_ax;
            const float vb_anchor_x = vxb - wb * r_by, vb_anchor_y = vyb + wb * r_bx;
            const float cdot_x = vb_anchor_x - va_anchor_x, cdot_y = vb_anchor_y - va_anchor_y;
            const float impulse_x = -(inv_k11[j] * cdot_x + inv_k12[j] * cdot_y);
            const float impulse_y = -(inv_k12[j] * cdot_x + inv_k22[j] * cdot_y);
            put<L::NUM_BODIES>(B.vx, a, vxa - inv_ma * impulse_x);
            put<L::NUM_BODIES>(B.vy, a, vya - inv_ma * impulse_y);
            put<L::NUM_BODIES>(B.vx, b, vxb + inv_mb * impulse_x);
            put<L::NUM_BODIES>(B.vy, b, vyb + inv_mb * impulse_y);
            float cur_wa = wa - inv_ia * (r_ax * impulse_y - r_ay * impulse_x);
            float cur_wb = wb + inv_ib * (r_bx * impulse_y - r_by * impulse_x);

            const int fl = flags[j];
            const float e = eff[j], re = reff[j];
            if (fl & JF_SPRING) {
                const float rel_omega = wb - wa;  // angular velocities from before the point impulse
                const float spring_torque = spring_term[j] - damp[j] * rel_omega;
                const float angular_impulse = spring_torque * dt;
                if (e > 1e-10f) {
                    cur_wa = cur_wa - div_by(inv_ia * angular_impulse, e, re);
                    cur_wb = cur_wb + div_by(inv_ib * angular_impulse, e, re);
                }
            }
            if (fl & JF_LIMIT) {
                const float relative_angle = rel_angle[j];
                const float rel_omega = cur_wb - cur_wa;
                if (e > 1e-10f) {
                    float limit_impulse = 0.0f;
                    // (the same quotient on both sides of the test: taken once, used where the test says)
                    const float stop = div_by(-rel_omega, e, re);
                    if (relative_angle <= lo[j]) {
                        if (rel_omega < 0.0f) limit_impulse = stop;
                    } else if (relative_angle >= hi[j]) {
                        if (rel_omega > 0.0f) limit_impulse = stop;
                    }
                    if (limit_impulse != 0.0f) {
                        cur_wa = cur_wa - inv_ia * limit_impulse;
                        cur_wb = cur_wb + inv_ib * limit_impulse;
                    }
                }
            }
            if (fl & JF_MOTOR) {
                const float rel_omega = cur_wb - cur_wa;
                const float speed_error = motor_speed[j] - rel_omega;
                if (e > 1e-10f) {
                    float motor_impulse = div_by(speed_error, e, re);
                    const float max_impulse = max_torque[j] * dt;
                    if (motor_impulse > max_impulse) motor_impulse = max_impulse;
                    if (motor_impulse < -max_impulse) motor_impulse = -max_impulse;
                    cur_wa = cur_wa - inv_ia * motor_impulse;
                    cur_wb = cur_wb + inv_ib * motor_impulse;
                }
            }
            put<L::NUM_BODIES>(B.w, a, cur_wa);
            put<L::NUM_BODIES>(B.w, b, cur_wb);
        }
    }

    MRL_DEV void position_sweep(RegBodies<L> &B, const float *row, float baumgarte, float slop) const {
#pragma unroll
        for (int j = 0; j < MJ; ++j) {
            if (!active[j]) continue;
            const float *J = row + L::JOINTS_OFF + j * JOINT_SIZE;
            const int a = ba(j), b = bb(j);
            const float xa = sel<L::NUM_BODIES>(B.x, a), ya = sel<L::NUM_BODIES>(B.y, a), angle_a = sel<L::NUM_BODIES>(B.ang, a);
            const float inv_ma = sel<L::NUM_BODIES>(B.im, a), inv_ia = sel<L::NUM_BODIES>(B.ii, a);
            const float xb = sel<L::NUM_BODIES>(B.x, b), yb = sel<L::NUM_BODIES>(B.y, b), angle_b = sel<L::NUM_BODIES>(B.ang, b);
            const float inv_mb = sel<L::NUM_BODIES>(B.im, b), inv_ib = sel<L::NUM_BODIES>(B.ii, b);
            float r_ax, r_ay, r_bx, r_by;
            anchor(B, J, a, b, r_ax, r_ay, r_bx, r_by);
            const float anchor_ax = xa + r_ax, anchor_ay = ya + r_ay;
            const float anchor_bx = xb + r_bx, anchor_by = yb + r_by;
            const float cx = anchor_bx - anchor_ax, cy = anchor_by - anchor_ay;
            const float error = sqrtf(cx * cx + cy * cy);
            if (error < slop) continue;
            const float k11 = inv_ma + inv_mb + inv_ia * r_ay * r_ay + inv_ib * r_by * r_by;
            const float k12 = -inv_ia * r_ax * r_ay - inv_ib * r_bx * r_by;
            const float k22 = inv_ma + inv_mb + inv_ia * r_ax * r_ax + inv_ib * r_bx * r_bx;
            float det = k11 * k22 - k12 * k12;
            if (det < 1e-10f) det = 1e-10f;
            const float inv_det = 1.0f / det;
            const float ik11 = k22 * inv_det, ik12 = -k12 * inv_det, ik22 = k11 * inv_det;
            const float correction_x = -baumgarte * (ik11 * cx + ik12 * cy);
            const float correction_y = -baumgarte * (ik12 * cx + ik22 * cy);
            put<L::NUM_BODIES>(B.x, a, xa - inv_ma * correction_x);
            put<L::NUM_BODIES>(B.y, a, ya - inv_ma * correction_y);
            put<L::NUM_BODIES>(B.x, b, xb + inv_mb * correction_x);
            put<L::NUM_BODIES>(B.y, b, yb + inv_mb * correction_y);
            float cur_a = angle_a - inv_ia * (r_ax * correction_y - r_ay * correction_x);
            float cur_b = angle_b + inv_ib * (r_bx * correction_y - r_by * correction_x);
            if (flags[j] & JF_LIMIT) {
                const float relative_angle = cur_b - cur_a - J[J_REF];
                const float e = inv_ia + inv_ib;
                if (e > 1e-10f) {
                    float angle_correction = 0.0f;
                    if (relative_angle < lo[j]) angle_correction = baumgarte * (lo[j] - relative_angle);
                    else if (relative_angle > hi[j]) angle_correction = baumgarte * (hi[j] - relative_angle);
                    if (angle_correction != 0.0f) {
                        cur_a = cur_a - div_by(inv_ia * angle_correction, e, reff[j]);
                        cur_b = cur_b + div_by(inv_ib * angle_correction, e, reff[j]);
                    }
                }
            }
            put<L::NUM_BODIES>(B.ang, a, cur_a);
            put<L::NUM_BODIES>(B.ang, b, cur_b);
        }
    }
};

// true when every joint of the row connects the bodies that the static topology T names
template <class L, class T>
MRL_DEV bool topology_matches(const float *row) {
    bool ok = true;
    const int n = (int)row[L::JOINT_COUNT_OFF];
#pragma unroll
    for (int j = 0; j < L::MAX_JOINTS; ++j) {
        if (j >= n) break;
        const float *J = row + L::JOINTS_OFF + j * JOINT_SIZE;
        ok = ok && (int)J[J_BODY_A] == T::a(j) && (int)J[J_BODY_B] == T::b(j);
    }
    return ok;
}

template <class L, class T, bool FLAT, bool REG_CONTACTS>
MRL_DEV int reg_physics_substep_impl(float *row, const float *shapes, float *contacts, float gx, float gy,
                                     float dt, float friction, float restitution, float baumgarte,
                                     float slop, int vel_iters, int pos_iters, int n_given) {
    RegBodies<L> B;
    B.load(row);
    reg_integrate_velocities<L>(B, row, gx, gy, dt);
    // the detectors read positions and angles only, which the velocity update has not touched
    const int n = n_given >= 0 ? n_given
                  : (FLAT ? flat_detect<L>(row, shapes, 0.0f, contacts) : edge_detect<L>(row, shapes, contacts));
    typename std::conditional<REG_CONTACTS, RegContacts<L>, LdsContacts<L>>::type C;
    C.load(B, contacts, n);
    RegJoints<L, T> J;
    J.prepare_velocity(B, row);
    for (int it = 0; it < vel_iters; ++it) {
        C.velocity_sweep(B, friction, restitution);
        J.velocity_sweep(B, dt);
    }
    reg_integrate_positions<L>(B, dt);
    for (int it = 0; it < pos_iters; ++it) {
        C.position_sweep(B, baumgarte, slop);
        J.position_sweep(B, row, baumgarte, slop);
    }
    B.store(row);
#pragma unroll
    for (int k = 0; k < L::NUM_BODIES * 3; ++k) row[L::FORCES_OFF + k] = 0.0f;
    return n;
}

// One physics step (or sub-step) of an env row with the sweeps on registers.  `row` must hold the
// current bodies / joints; contacts are detected into the lane's LDS scratch, which holds
// MAX_CONTACTS * CONTACT_SCRATCH floats (detection order and the MAX_CONTACTS cut-off unchanged;
// afterwards the body indices of the contacts are still readable at
// contacts[c * CONTACT_SIZE + C_BODY_A / C_BODY_B], the contact-point slots are not), then
// everything iterative runs on registers.  n_given >= 0: `contacts` already holds that many
// contacts detected from the row's current positions (detection is skipped).
template <class L, class T, bool FLAT, bool REG_CONTACTS>
MRL_DEV int reg_physics_substep(float *row, const float *shapes, float *contacts, float gx, float gy,
                                float dt, float friction, float restitution, float baumgarte, float slop,
                                int vel_iters, int pos_iters, int n_given = -1) {
    if (T::STATIC && __all(topology_matches<L, T>(row) ? 1 : 0))
        return reg_physics_substep_impl<L, T, FLAT, REG_CONTACTS>(row, shapes, contacts, gx, gy, dt, friction,
                                                                  restitution, baumgarte, slop, vel_iters,
                                                                  pos_iters, n_given);
    return reg_physics_substep_impl<L, DynamicTopology, FLAT, REG_CONTACTS>(
        row, shapes, contacts, gx, gy, dt, friction, restitution, baumgarte, slop, vel_iters, pos_iters,
        n_given);
}

}  // namespace mrl
