// HalfCheetah's env step with one lane per BODY: eight lanes per env (seven bodies, one idle), eight
// envs per wavefront.
//
// With one lane per env the step is one long instruction stream per wavefront (5 sub-steps x 6
// Gauss-Seidel sweeps over 6 joints and up to 14 contacts, each body picked with a 7-way select
// chain).  Much of that stream is work on different bodies that does not interact:
//   * integration, ground detection and the contact sweeps touch only the contact's own body (the
//     ground is the other party), so contacts of different bodies commute exactly: every lane runs
//     the contacts of its own body, in vertex order, at the place in the sweep where the one-lane
//     form runs all contacts;
//   * the joint sweep visits joints 0 .. 5 in order, but after joint 0 (torso - back thigh) the back
//     leg's joints 1, 2 touch bodies 1, 2, 3 only and the front leg's joints 3, 4, 5 bodies 0, 4, 5, 6:
//     two chains without a body in common, which run side by side -- four joint slots per sweep
//     instead of six.  In a slot the CHILD body's lane does the joint (parent state fetched from the
//     parent's lane, parent result handed back), so every lane holds its body in plain registers.
// Same operations on the same values in an order the arithmetic cannot tell from the one-lane form's:
// the results are identical bit for bit (the parity tests compare both with the oracle).
//
// The wiring is HalfCheetah's (cheetah_planar_v2.mojo: torso 0; back thigh / shin / foot 1, 2, 3;
// front 4, 5, 6; joint j joins body j + 1 to its parent).  A row whose joint table or shapes differ
// from that is stepped by the one-lane form instead (lanes_row_ok, tested by the caller).
#pragma once
#include "env_walkers.hpp"

namespace mrl {
namespace hc {

constexpr int LANES_PER_ENV = 8;

// LDS writes of this wavefront's lanes become visible to its other lanes
MRL_DEV void wave_sync_lds() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// lanes of one env sit side by side: value of lane `src` of my group
template <class V>
MRL_DEV V group_get(V v, int base, int src) { return __shfl(v, base + src, 64); }

// The two exchanges of a joint slot as DPP row shifts (register to register, no trip through the LDS
// crossbar).  Rows are 16 lanes, so the two groups of a row shift side by side; a lane at a group's
// edge picks up a neighbour group's value that it never uses.
//   from_parent: every child's parent is the body before it, except the front thigh (4), whose
//                parent is the torso four lanes down;
//   from_kid<S>: the parent's lane takes the result of its child in slot S -- the next lane, except
//                the torso in slot 1, whose child is the front thigh four lanes up.
MRL_DEV float dpp_row_shr1(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xF, 0xF, false)); }
MRL_DEV float dpp_row_shr4(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x114, 0xF, 0xF, false)); }
MRL_DEV float dpp_row_shl1(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x101, 0xF, 0xF, false)); }
MRL_DEV float dpp_row_shl4(float v) { return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x104, 0xF, 0xF, false)); }
MRL_DEV float from_parent(float v, int b) {
    const float one = dpp_row_shr1(v), four = dpp_row_shr4(v);
    return b == 4 ? four : one;
}
template <int S>
MRL_DEV float from_kid(float v, int b) {
    const float one = dpp_row_shl1(v);
    if (S == 1) {
        const float four = dpp_row_shl4(v);
        return b == 0 ? four : one;
    }
    return one;
}

MRL_DEV float from_kid_slot(int s, float v, int b) {
    const float one = dpp_row_shl1(v), four = dpp_row_shl4(v);
    return (s == 1 && b == 0) ? four : one;
}

// true when the row has the wiring and shapes this form assumes
MRL_DEV bool lanes_row_ok(const float *row, const float *shapes) {
    if ((int)row[L::JOINT_COUNT_OFF] != 6) return false;
    bool ok = true;
    for (int j = 0; j < 6; ++j) {
        const float *J = row + L::JOINTS_OFF + j * JOINT_SIZE;
        ok = ok && (int)J[J_TYPE] == 0 && (int)J[J_BODY_A] == Topology::a(j) && (int)J[J_BODY_B] == Topology::b(j);
    }
    for (int b = 0; b < 7; ++b) {
        const float *S = shapes + (int)row[L::BODIES_OFF + b * BODY_SIZE + IDX_SHAPE] * SHAPE_SIZE;
        ok = ok && (int)S[0] == SHAPE_POLYGON && (int)S[1] <= 4;
    }
    return ok;
}

// everything after the physics of an env step but the observation (cheetah_planar_v2.mojo:790-846): reward
// and metadata; `a` = the clamped action, (x_after, torso_z) = the torso's position after the physics,
// `penalised` = ground contacts of the last sub-step on bodies other than the two feet
MRL_DEV void step_tail(float *row, const double *a, double x_before, double x_after, double torso_z, int penalised,
                       float &reward, float &done) {
    const double forward_velocity = (x_after - x_before) / (0.01 * (double)5);
    const double forward_reward = 1.0 * forward_velocity;
    double ctrl_cost = 0.0;
#pragma unroll
    for (int i = 0; i < ACT; ++i) {
        double c = a[i] < 1.0 ? a[i] : 1.0;
        c = c > -1.0 ? c : -1.0;
        ctrl_cost += c * c;
    }
    ctrl_cost *= 0.1;
    double height_bonus = 0.0;
    if (torso_z > 0.1) height_bonus = 1.0 * (torso_z < 0.5 ? torso_z : 0.5);
    const double penalty = 0.5 * (double)penalised;   // 0.5 per contact, summed in Float64: exact in any order
    const double r = forward_reward - ctrl_cost + height_bonus - penalty;
    float *M = row + L::META_OFF;
    const int step_count = (int)M[META_STEP] + 1;
    M[META_STEP] = (float)step_count;
    M[META_PREV_X] = (float)x_after;
    M[META_TOTAL] = (float)((double)M[META_TOTAL] + r);
    const bool d = step_count >= 1000;
    M[META_DONE] = d ? 1.0f : 0.0f;
    reward = (float)r;
    done = d ? 1.0f : 0.0f;
}

// The env step of hc::step_row by the eight lanes of an env's group (all lanes of the wavefront call
// it together; `lane` = lane in the wavefront, `row` = the group's env row in LDS, `action` = its six
// action components).  Lane 0 of the group returns reward / done.
MRL_DEV void step_lanes(float *row, const float *shapes, const float *action, int lane, float &reward, float &done) {
    const int b = lane & 7, base = lane & ~7;
    const bool body = b < 7;
    // ---- wiring seen from this lane: as the child of joint b - 1 (bodies 1 .. 6) ...
    const bool child = b >= 1 && b <= 6;
    const int j = child ? b - 1 : 0;
    const int par = (b == 1 || b == 4) ? 0 : (child ? b - 1 : 0);
    const int myslot = b == 1 ? 0 : (b == 2 || b == 4) ? 1 : (b == 3 || b == 5) ? 2 : b == 6 ? 3 : -1;
    // ... and as the parent of the joint that runs in slot s: bit s of kidmask (the torso has a child in
    // slots 0 and 1, the front thigh in slot 1 being the one that sits four lanes up)
    const int kidmask = b == 0 ? 3 : b == 1 ? 2 : (b == 2 || b == 4) ? 4 : b == 5 ? 8 : 0;

    const float gx = (float)0.0, gy = (float)-9.81, dt = (float)0.01, friction = (float)0.9, restitution = (float)0.0;
    const float baumgarte = (float)0.2, slop = (float)0.005;

    // ---- the action into the joint motors (child lane of joint j), as hc::step_row does
    float *J = row + L::JOINTS_OFF + j * JOINT_SIZE;
    float motor_speed = 0.0f, max_torque = 0.0f;
    if (child) {
        float v = action[j];
        v = v < 1.0f ? v : 1.0f;
        v = v > -1.0f ? v : -1.0f;
        const double av = (double)v;
        motor_speed = (av >= 0.0 ? 1.0f : -1.0f) * 1000.0f;
        max_torque = (float)(1.0 * ::fabs(av));
        J[J_MOTOR_SPEED] = motor_speed;
        J[J_MAX_TORQUE] = max_torque;
    }
    const float lax = J[J_AX], lay = J[J_AY], lbx = J[J_BX], lby = J[J_BY];
    const float jref = J[J_REF], jlo = J[J_LO], jhi = J[J_HI], jstiff = J[J_STIFF], jdamp = J[J_DAMP];
    const int jflags = (int)J[J_FLAGS];

    // ---- my body
    float *Bp = row + L::BODIES_OFF + (body ? b : 0) * BODY_SIZE;
    float x = Bp[IDX_X], y = Bp[IDX_Y], ang = Bp[IDX_ANGLE], vx = Bp[IDX_VX], vy = Bp[IDX_VY], w = Bp[IDX_OMEGA];
    const float im = Bp[IDX_INV_MASS], ii = Bp[IDX_INV_INERTIA];
    float fx = row[L::FORCES_OFF + (body ? b : 0) * 3], fy = row[L::FORCES_OFF + (body ? b : 0) * 3 + 1],
          tau = row[L::FORCES_OFF + (body ? b : 0) * 3 + 2];
    const float *S = shapes + (int)Bp[IDX_SHAPE] * SHAPE_SIZE;
    const int n_verts = (int)S[1];
    float lvx[4], lvy[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) { lvx[v] = S[2 + v * 2]; lvy[v] = S[3 + v * 2]; }
    const float p_im = from_parent(im, b), p_ii = from_parent(ii, b);
    const float eff = p_ii + ii;
    const float reff = 1.0f / eff;   // the limit and motor terms of every sweep divide by eff (div_by)
    const double x_before = (double)x;   // meaningful on lane 0 (the torso)

    // sine and cosine of my body's angle, kept in step with it (recomputed whenever the angle may have
    // changed): the same values that the one-lane form recomputes at every use
    float sin_a, cos_a;
    sincos32(ang, sin_a, cos_a);
    int kept = 0;   // my body's contacts of the current sub-step that made the list
    for (int sub = 0; sub < 5; ++sub) {
        // ---- integrate velocities (integrators/euler.mojo:82-130)
        if (im != 0.0f) {
            vx = vx + (fx * im + gx) * dt;
            vy = vy + (fy * im + gy) * dt;
            w = w + tau * ii * dt;
        }
        fx = fy = tau = 0.0f;   // the forces are cleared at the end of every sub-step
        // ---- ground contacts of my body, vertex order (collision/flat_terrain.mojo:69-204); the list
        // of an env is cut at MAX_CONTACTS in (body, vertex) order: contacts before mine are counted
        float cpx[4] = {0.0f, 0.0f, 0.0f, 0.0f}, cpy[4] = {0.0f, 0.0f, 0.0f, 0.0f}, cdepth[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        int found = 0;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float world_x = x + lvx[v] * cos_a - lvy[v] * sin_a;
            const float world_y = y + lvx[v] * sin_a + lvy[v] * cos_a;
            const float penetration = 0.0f - world_y;
            const bool hit = body && v < n_verts && penetration > 0.0f;
            // compacted in vertex order
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (hit && found == q) { cpx[q] = world_x; cpy[q] = world_y; cdepth[q] = penetration; }
            }
            found += hit ? 1 : 0;
        }
        int before = 0;   // contacts of the bodies before mine
#pragma unroll
        for (int o = 0; o < 7; ++o) {
            const int c = group_get(found, base, o);
            before += o < b ? c : 0;
        }
        kept = L::MAX_CONTACTS - before;
        kept = kept < 0 ? 0 : (kept > found ? found : kept);
        // ---- what stays fixed during the velocity phase: contact lever arms and effective masses
        // (solvers/impulse.mojo:115-190) ...
        const float nx = 0.0f, ny = 1.0f;
        ContactFixed cf[4];
        float jn[4], jt[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            jn[q] = jt[q] = 0.0f;
            ContactFixed f;
            f.nx = nx; f.ny = ny;
            f.inv_mass_a = im; f.inv_inertia_a = ii;
            const float inv_mass_b = 0.0f, inv_inertia_b = 0.0f;
            f.ra_x = cpx[q] - x; f.ra_y = cpy[q] - y;
            const float rb_x = cpx[q] - cpx[q], rb_y = cpy[q] - cpy[q];
            const float ra_cross_n = f.ra_x * ny - f.ra_y * nx;
            const float rb_cross_n = rb_x * ny - rb_y * nx;
            float k = f.inv_mass_a + inv_mass_b;
            k = k + f.inv_inertia_a * ra_cross_n * ra_cross_n;
            k = k + inv_inertia_b * rb_cross_n * rb_cross_n;
            f.k = k;
            const float tangent_x = -ny, tangent_y = nx;
            const float ra_cross_t = f.ra_x * tangent_y - f.ra_y * tangent_x;
            const float rb_cross_t = rb_x * tangent_y - rb_y * tangent_x;
            float k_t = f.inv_mass_a + inv_mass_b;
            k_t = k_t + f.inv_inertia_a * ra_cross_t * ra_cross_t;
            k_t = k_t + inv_inertia_b * rb_cross_t * rb_cross_t;
            f.k_t = k_t;
            f.rk = 1.0f / k;
            f.rk_t = 1.0f / k_t;
            cf[q] = f;
        }
        // ... and the joint's lever arms, K^-1 and limit angle (joints/revolute.mojo:90-200), by the child
        const float p_sin = from_parent(sin_a, b), p_cos = from_parent(cos_a, b);
        const float p_ang = from_parent(ang, b);
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
        const float angle_error = (ang - p_ang) - jref;
        const float spring_term = -jstiff * angle_error;
        const float rel_angle = ang - p_ang - jref;

        // ---- velocity iterations: my contacts, then the joints slot by slot
        for (int it = 0; it < 4; ++it) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (q >= kept) break;
                // one contact of solvers/impulse.mojo:192-331 on my body
                const ContactFixed &f = cf[q];
                float vel_a_x = vx, vel_a_y = vy, omega_a = w;
                const float vel_b_x = 0.0f, vel_b_y = 0.0f, omega_b = 0.0f, rb_x = 0.0f, rb_y = 0.0f;
                float vel_at_a_x = vel_a_x - omega_a * f.ra_y, vel_at_a_y = vel_a_y + omega_a * f.ra_x;
                float vel_at_b_x = vel_b_x - omega_b * rb_y, vel_at_b_y = vel_b_y + omega_b * rb_x;
                float rel_vel_x = vel_at_a_x - vel_at_b_x, rel_vel_y = vel_at_a_y - vel_at_b_y;
                const float vel_normal = rel_vel_x * f.nx + rel_vel_y * f.ny;
                if (!(vel_normal < 0.0f)) continue;
                float j_normal = div_by(-(1.0f + restitution) * vel_normal, f.k, f.rk);
                const float old_impulse = jn[q];
                float new_impulse = old_impulse + j_normal;
                if (new_impulse < 0.0f) new_impulse = 0.0f;
                jn[q] = new_impulse;
                j_normal = new_impulse - old_impulse;
                const float impulse_x = j_normal * f.nx, impulse_y = j_normal * f.ny;
                vel_a_x = vel_a_x + impulse_x * f.inv_mass_a;
                vel_a_y = vel_a_y + impulse_y * f.inv_mass_a;
                omega_a = omega_a + (f.ra_x * impulse_y - f.ra_y * impulse_x) * f.inv_inertia_a;
                vel_at_a_x = vel_a_x - omega_a * f.ra_y; vel_at_a_y = vel_a_y + omega_a * f.ra_x;
                vel_at_b_x = vel_b_x - omega_b * rb_y; vel_at_b_y = vel_b_y + omega_b * rb_x;
                rel_vel_x = vel_at_a_x - vel_at_b_x; rel_vel_y = vel_at_a_y - vel_at_b_y;
                const float tangent_x = -f.ny, tangent_y = f.nx;
                const float vel_tangent = rel_vel_x * tangent_x + rel_vel_y * tangent_y;
                float j_tangent = div_by(-vel_tangent, f.k_t, f.rk_t);
                const float max_friction = friction * new_impulse;
                const float old_tangent = jt[q];
                float new_tangent = old_tangent + j_tangent;
                if (new_tangent > max_friction) new_tangent = max_friction;
                else if (new_tangent < -max_friction) new_tangent = -max_friction;
                jt[q] = new_tangent;
                j_tangent = new_tangent - old_tangent;
                const float friction_x = j_tangent * tangent_x, friction_y = j_tangent * tangent_y;
                vx = vel_a_x + friction_x * f.inv_mass_a;
                vy = vel_a_y + friction_y * f.inv_mass_a;
                w = omega_a + (f.ra_x * friction_y - f.ra_y * friction_x) * f.inv_inertia_a;
            }
#pragma unroll
            for (int s = 0; s < 4; ++s) {
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
                const float g_vx = from_kid_slot(s, n_vxa, b), g_vy = from_kid_slot(s, n_vya, b);
                const float g_w = from_kid_slot(s, cur_wa, b);
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
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (q >= kept) break;
                float correction = cdepth[q] - slop;
                if (correction <= 0.0f) continue;
                correction = baumgarte * correction;
                const float inv_mass_a = im, inv_mass_b = 0.0f;
                const float total = inv_mass_a + inv_mass_b;
                if (total == 0.0f) continue;
                const float correction_a = correction * inv_mass_a / total;
                x = x + nx * correction_a;
                y = y + ny * correction_a;
            }
#pragma unroll
            for (int s = 0; s < 4; ++s) {
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
                const float g_x = from_kid_slot(s, n_xa, b), g_y = from_kid_slot(s, n_ya, b);
                const float g_a = from_kid_slot(s, n_aa, b);
                if ((kidmask >> s) & 1) { x = g_x; y = g_y; ang = g_a; }
                if (myslot == s) { x = n_xb; y = n_yb; ang = n_ab; }
                // (the last slot moves the front shin and foot only, which the second iteration reads in its
                // last two slots, behind two more of these; after the second iteration the next sub-step reads all)
                if (!(it == 0 && s == 3)) sincos32(ang, sin_a, cos_a);
            }
        }
    }
    // ---- bodies and forces back into the row, then the rest of the step on the torso's lane
    if (body) {
        Bp[IDX_X] = x; Bp[IDX_Y] = y; Bp[IDX_ANGLE] = ang; Bp[IDX_VX] = vx; Bp[IDX_VY] = vy; Bp[IDX_OMEGA] = w;
        row[L::FORCES_OFF + b * 3] = 0.0f; row[L::FORCES_OFF + b * 3 + 1] = 0.0f; row[L::FORCES_OFF + b * 3 + 2] = 0.0f;
    }
    int penalised = 0;   // contacts of the last sub-step on anything but the feet (bodies 3 and 6)
#pragma unroll
    for (int o = 0; o < 7; ++o) {
        const int c = group_get(kept, base, o);
        penalised += (o != 3 && o != 6) ? c : 0;
    }
    // ---- the observation (hc::observe: the same expressions on the same values), every body's lane its own
    // entries: the torso its height, angle and velocity, a leg segment its angle and angular velocity
    // against its parent's
    {
        const double p_ang = (double)from_parent(ang, b), p_w = (double)from_parent(w, b);
        if (b == 0) {
            row[0] = y; row[1] = ang; row[8] = vx; row[9] = vy; row[10] = w;
        } else if (child) {
            row[2 + j] = (float)((double)ang - p_ang);
            row[11 + j] = (float)((double)w - p_w);
        }
    }
    if (b == 0) {
        double a[ACT];
#pragma unroll
        for (int k = 0; k < ACT; ++k) {
            float v = action[k];
            v = v < 1.0f ? v : 1.0f;
            v = v > -1.0f ? v : -1.0f;
            a[k] = (double)v;
        }
        step_tail(row, a, x_before, (double)x, (double)y, penalised, reward, done);
    }
    wave_sync_lds();   // the row is complete for whoever reads it next
}

}  // namespace hc
}  // namespace mrl
