// HopperPlanar and Walker2dPlanar (envs/mujoco_planar/hopper_planar.mojo:162-614,
// walker_planar.mojo:168-639): the reference's two Float64 CPU envs with a simplified physics of their
// own -- joint velocities take the torque, joint angles are clamped to their limits, the torso falls
// under gravity, the leg segments are placed by forward kinematics, a foot below the ground pushes the
// torso up.  One lane per env; every arithmetic step is Float64 in the reference's order of operations.
//
// The reference has no batched form of these envs, so the row is this library's own:
//   floats [0, OBS)            the observation (get_observation cast to fp32)
//   float  [OBS]               padding (keeps the doubles 8-byte aligned: rows hold an even number of floats)
//   doubles from float OBS + 1 the struct's Float64 state, bit for bit, two floats each:
//       torso x, y, angle, vx, vy, omega | (x, y, angle) of every other body, in body order |
//       joint_angles | joint_velocities | step_count, done (0 / 1), total_reward, prev_x
//   Hopper: 12 + 2 * 25 = 62 floats; Walker2d: 18 + 2 * 40 = 98 floats.
// (Masses and inertias enter nothing in this physics.  vx, vy, omega of the leg bodies are written once,
// as 0, by _init_body; the one that is read -- the foot's vx in the hopper's ground contact,
// hopper_planar.mojo:600-602 -- enters as that 0.)
// Protocol of the batched form, as for the other envs: a row whose done flag is set returns (0, 1) untouched;
// the reset's draws of random_float64() (hopper_planar.mojo:318-322) are uniforms of Philox(combined seed, 0)
// in the order the loop consumes them.
#pragma once
#include "mrl_device.hpp"

namespace mrl {
namespace planar {

struct Hopper {
    static constexpr int LEGS = 1, OBS = 11, ACT = 3, STATE = 62;
    static constexpr double FOOT_LEN = 0.39, GEAR = 200.0, MIN_Z = 0.7, MAX_Z = -1.0, MAX_ANGLE = 0.2;
    static constexpr bool CHAIN_THROUGH_CENTRES = true, FOOT_FRICTION_TERM = true;
    static MRL_DEV double lim(int k, int side) {
        const double v[3][2] = {{-2.61799, 0.0}, {-2.61799, 0.0}, {-0.785398, 0.785398}};
        return v[k][side];
    }
    static MRL_DEV double hip_dx(int) { return 0.0; }
};
struct Walker2d {
    static constexpr int LEGS = 2, OBS = 17, ACT = 6, STATE = 98;
    static constexpr double FOOT_LEN = 0.2, GEAR = 100.0, MIN_Z = 0.8, MAX_Z = 2.0, MAX_ANGLE = 1.0;
    static constexpr bool CHAIN_THROUGH_CENTRES = false, FOOT_FRICTION_TERM = false;
    static MRL_DEV double lim(int k, int side) {
        const double v[3][2] = {{-1.0, 0.7}, {-1.2, 0.0}, {-0.5, 0.5}};
        return v[k][side];
    }
    static MRL_DEV double hip_dx(int l) { return l == 0 ? 0.1 : -0.1; }
};
constexpr double TORSO_LEN = 0.4, THIGH_LEN = 0.45, LEG_LEN = 0.5, FOOT_RADIUS = 0.06, INIT_HEIGHT = 1.25;
constexpr double DT = 0.008, GRAVITY = -9.81;
constexpr int FRAME_SKIP = 4;

// the Float64 state of one env in registers
template <class M>
struct State {
    static constexpr int NJ = 3 * M::LEGS, ND = 6 + 3 * NJ + 2 * NJ + 4;
    double torso[6], body[3 * NJ], ja[NJ], jv[NJ], meta[4];

    MRL_DEV void load(const float *row) {
        const double *d = reinterpret_cast<const double *>(row + M::OBS + 1);
#pragma unroll
        for (int k = 0; k < 6; ++k) torso[k] = d[k];
#pragma unroll
        for (int k = 0; k < 3 * NJ; ++k) body[k] = d[6 + k];
#pragma unroll
        for (int k = 0; k < NJ; ++k) { ja[k] = d[6 + 3 * NJ + k]; jv[k] = d[6 + 4 * NJ + k]; }
#pragma unroll
        for (int k = 0; k < 4; ++k) meta[k] = d[6 + 5 * NJ + k];
    }
    // the whole row: observation, padding, state
    MRL_DEV void store(float *row) const {
        row[0] = (float)torso[1];
        row[1] = (float)torso[2];
#pragma unroll
        for (int i = 0; i < NJ; ++i) row[2 + i] = (float)ja[i];
        row[2 + NJ] = (float)torso[3];
        row[3 + NJ] = (float)torso[4];
        row[4 + NJ] = (float)torso[5];
#pragma unroll
        for (int i = 0; i < NJ; ++i) row[5 + NJ + i] = (float)jv[i];
        row[M::OBS] = 0.0f;
        double *d = reinterpret_cast<double *>(row + M::OBS + 1);
#pragma unroll
        for (int k = 0; k < 6; ++k) d[k] = torso[k];
#pragma unroll
        for (int k = 0; k < 3 * NJ; ++k) d[6 + k] = body[k];
#pragma unroll
        for (int k = 0; k < NJ; ++k) { d[6 + 3 * NJ + k] = ja[k]; d[6 + 4 * NJ + k] = jv[k]; }
#pragma unroll
        for (int k = 0; k < 4; ++k) d[6 + 5 * NJ + k] = meta[k];
    }
    // get_observation (hopper_planar.mojo:324-375, walker_planar.mojo:339-403) into obs [OBS]
    MRL_DEV void observe(float *obs) const {
        obs[0] = (float)torso[1];
        obs[1] = (float)torso[2];
#pragma unroll
        for (int i = 0; i < NJ; ++i) obs[2 + i] = (float)ja[i];
        obs[2 + NJ] = (float)torso[3];
        obs[3 + NJ] = (float)torso[4];
        obs[4 + NJ] = (float)torso[5];
#pragma unroll
        for (int i = 0; i < NJ; ++i) obs[5 + NJ + i] = (float)jv[i];
    }
};

MRL_DEV uint64_t combined_seed(uint64_t seed, int env) {
    const int64_t seed_i = (int64_t)(float)seed;
    return (uint64_t)seed_i * 2654435761ull + (uint64_t)(env + 1) * 12345ull;
}

// _reset_state (hopper_planar.mojo:203-284, walker_planar.mojo:198-303) and the noise of reset() (:311-322)
template <class M>
MRL_DEV void reset(State<M> &s, uint64_t cseed) {
    constexpr int NJ = State<M>::NJ;
#pragma unroll
    for (int k = 0; k < 6; ++k) s.torso[k] = 0.0;
#pragma unroll
    for (int k = 0; k < 4; ++k) s.meta[k] = 0.0;
    const double torso_y = INIT_HEIGHT;
    s.torso[1] = torso_y;
    const double thigh_y = torso_y - TORSO_LEN / 2 - THIGH_LEN / 2;
    const double leg_y = thigh_y - THIGH_LEN / 2 - LEG_LEN / 2;
    const double foot_y = leg_y - LEG_LEN / 2 - M::FOOT_LEN / 2;
#pragma unroll
    for (int l = 0; l < M::LEGS; ++l) {
        s.body[9 * l + 0] = M::hip_dx(l); s.body[9 * l + 1] = thigh_y; s.body[9 * l + 2] = 0.0;
        s.body[9 * l + 3] = M::hip_dx(l); s.body[9 * l + 4] = leg_y; s.body[9 * l + 5] = 0.0;
        s.body[9 * l + 6] = M::hip_dx(l); s.body[9 * l + 7] = foot_y; s.body[9 * l + 8] = 0.0;
    }
    // draw n of the stream = lane (n % 4) of block (n / 4); joint i takes draws 2 i (angle) and 2 i + 1 (velocity)
    float u[2 * NJ];
#pragma unroll
    for (int q = 0; q < (2 * NJ + 3) / 4; ++q) {
        const Uniform4 rv = philox_uniform4(cseed, 0, (uint64_t)q);
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (4 * q + k < 2 * NJ) u[4 * q + k] = rv.v[k];
    }
#pragma unroll
    for (int i = 0; i < NJ; ++i) {
        s.ja[i] = ((double)u[2 * i] - 0.5) * 0.01;
        s.jv[i] = ((double)u[2 * i + 1] - 0.5) * 0.01;
    }
}

// one leg of _update_body_positions (hopper_planar.mojo:509-575, walker_planar.mojo:536-604)
// (the leg index is a template argument: every array index is a constant, the state stays in registers)
template <class M, int LEG>
MRL_DEV void place_leg(State<M> &s, double hip_x, double hip_y) {
    double b[9];
    const double joint_y = hip_y - TORSO_LEN / 2;
    const double hip_angle = s.ja[3 * LEG];
    double sn, cs;
    ::sincos(hip_angle, &sn, &cs);
    b[0] = hip_x + sn * THIGH_LEN / 2;
    b[1] = joint_y - cs * THIGH_LEN / 2;
    b[2] = hip_angle;
    double knee_x, knee_y;
    if (M::CHAIN_THROUGH_CENTRES) {
        knee_x = b[0] + sn * THIGH_LEN / 2;
        knee_y = b[1] - cs * THIGH_LEN / 2;
    } else {
        knee_x = hip_x + sn * THIGH_LEN;
        knee_y = joint_y - cs * THIGH_LEN;
    }
    const double total_angle = hip_angle + s.ja[3 * LEG + 1];
    ::sincos(total_angle, &sn, &cs);
    b[3] = knee_x + sn * LEG_LEN / 2;
    b[4] = knee_y - cs * LEG_LEN / 2;
    b[5] = total_angle;
    double ankle_x, ankle_y;
    if (M::CHAIN_THROUGH_CENTRES) {
        ankle_x = b[3] + sn * LEG_LEN / 2;
        ankle_y = b[4] - cs * LEG_LEN / 2;
    } else {
        ankle_x = knee_x + sn * LEG_LEN;
        ankle_y = knee_y - cs * LEG_LEN;
    }
    const double foot_angle = total_angle + s.ja[3 * LEG + 2];
    ::sincos(foot_angle, &sn, &cs);
    b[6] = ankle_x + sn * M::FOOT_LEN / 2;
    b[7] = ankle_y - cs * M::FOOT_LEN / 2;
    b[8] = foot_angle;
#pragma unroll
    for (int k = 0; k < 9; ++k) s.body[9 * LEG + k] = b[k];
}

// _physics_step (hopper_planar.mojo:444-507, walker_planar.mojo:462-534)
template <class M>
MRL_DEV void physics_step(State<M> &s, const double *torques) {
    constexpr int NJ = State<M>::NJ;
    const double dt = DT;
#pragma unroll
    for (int i = 0; i < NJ; ++i) s.jv[i] += torques[i] * dt * 0.01;
#pragma unroll
    for (int i = 0; i < NJ; ++i) {
        s.ja[i] += s.jv[i] * dt;
        const double low = M::lim(i % 3, 0), high = M::lim(i % 3, 1);
        if (s.ja[i] < low) { s.ja[i] = low; s.jv[i] = 0.0; }
        else if (s.ja[i] > high) { s.ja[i] = high; s.jv[i] = 0.0; }
    }
    s.torso[4] += GRAVITY * dt;
    double torso_x = s.torso[0], torso_y = s.torso[1];
    torso_x += s.torso[3] * DT;
    torso_y += s.torso[4] * DT;
    s.torso[0] = torso_x; s.torso[1] = torso_y;
    place_leg<M, 0>(s, torso_x + M::hip_dx(0), torso_y);
    if constexpr (M::LEGS == 2) place_leg<M, 1>(s, torso_x + M::hip_dx(1), torso_y);
    const double ground_y = 0.0;
#pragma unroll
    for (int l = 0; l < M::LEGS; ++l) {
        const double foot_y = s.body[9 * l + 7];
        if (foot_y - FOOT_RADIUS < ground_y) {
            const double penetration = ground_y - (foot_y - FOOT_RADIUS);
            s.torso[1] += penetration;
            if (s.torso[4] < 0) s.torso[4] = 0.0;
            if (M::FOOT_FRICTION_TERM) {
                const double foot_vx = 0.0;   // the foot body's vx slot: 0 since _init_body
                s.torso[3] += foot_vx * 0.1;
            }
        }
    }
}

// step (hopper_planar.mojo:377-442, walker_planar.mojo:405-460); action = ACT floats
template <class M>
MRL_DEV void step(State<M> &s, const float *action, float &reward, float &done) {
    constexpr int NJ = State<M>::NJ;
    if (s.meta[1] > 0.5) { reward = 0.0f; done = 1.0f; return; }
    double torques[NJ];
#pragma unroll
    for (int i = 0; i < NJ; ++i) {
        double a = (double)action[i];
        if (a > 1.0) a = 1.0;
        else if (a < -1.0) a = -1.0;
        torques[i] = a * M::GEAR;
    }
    const double x_before = s.torso[0];
    for (int k = 0; k < FRAME_SKIP; ++k) physics_step<M>(s, torques);
    const double x_after = s.torso[0], torso_y = s.torso[1], torso_angle = s.torso[2];
    const double forward_velocity = (x_after - x_before) / (DT * (double)FRAME_SKIP);
    const double forward_reward = 1.0 * forward_velocity;
    double ctrl_cost = 0.0;
#pragma unroll
    for (int i = 0; i < NJ; ++i) {
        const double ai = (double)action[i];
        const double a = (ai >= -1.0 && ai <= 1.0) ? ai : (ai > 0 ? 1.0 : -1.0);
        ctrl_cost += a * a;
    }
    ctrl_cost *= 0.001;
    bool is_healthy = torso_y >= M::MIN_Z && ::fabs(torso_angle) <= M::MAX_ANGLE;
    if (M::MAX_Z >= 0.0) is_healthy = is_healthy && torso_y <= M::MAX_Z;
    const double healthy_reward = is_healthy ? 1.0 : 0.0;
    const double rew = forward_reward + healthy_reward - ctrl_cost;
    s.meta[1] = is_healthy ? 0.0 : 1.0;
    s.meta[0] += 1.0;
    s.meta[2] += rew;
    reward = (float)rew;
    done = is_healthy ? 0.0f : 1.0f;
}

}  // namespace planar
}  // namespace mrl
