/*
 * CartPole and Pendulum: CPU restatement (test infrastructure, never shipped).
 *
 * CartPole step  : envs/cartpole.mojo:394-460 (CartPoleEnv.step_raw, the CPU path:
 *                  reward 0 on termination, truncation at 500 steps).
 * CartPole reset : envs/cartpole.mojo:784-905 (the seeded xorshift32 protocol of
 *                  reset_kernel / selective_reset_kernel; the CPU reset draws from the
 *                  unseedable global random_float64 stream and cannot be restated).
 * Pendulum step  : envs/pendulum/pendulum_v2.mojo:640-661 (action * max_torque),
 *                  :734-792 (_step_with_torque, _angle_normalize), :621-629 (obs through
 *                  Float64 cos/sin), laid out in the 8-float row of
 *                  envs/pendulum/constants.mojo (PendulumLayout).
 * Pendulum reset : pendulum_v2.mojo:294-331 (seed combination), :548-603 (row init),
 *                  :611-623 (CPU arithmetic of theta / theta_dot in Float64).
 */
#include <math.h>
#include "orc.h"

static inline float f32_sin(float x) { return (float)sin((double)x); }
static inline float f32_cos(float x) { return (float)cos((double)x); }

/* ---------------------------------------------------------------- CartPole */

void orc_cartpole_step(float s[4], int32_t *steps, int action, float *reward, float *done) {
    const float GRAVITY = (float)9.8, TOTAL_MASS = (float)(1.0 + 0.1), POLE_MASS = (float)0.1;
    const float POLE_HALF_LENGTH = (float)0.5, POLE_MASS_LENGTH = (float)(0.1 * 0.5);
    const float FORCE_MAG = (float)10.0, TAU = (float)0.02;
    const float X_THRESHOLD = (float)2.4, THETA_THRESHOLD = (float)0.2095;

    float x = s[0], x_dot = s[1], theta = s[2], theta_dot = s[3];
    float force = (action == 1) ? FORCE_MAG : -FORCE_MAG;
    float costheta = f32_cos(theta);
    float sintheta = f32_sin(theta);

    float temp = (force + POLE_MASS_LENGTH * theta_dot * theta_dot * sintheta) / TOTAL_MASS;
    float thetaacc = (GRAVITY * sintheta - costheta * temp) /
                     (POLE_HALF_LENGTH *
                      ((float)(4.0 / 3.0) - POLE_MASS * costheta * costheta / TOTAL_MASS));
    float xacc = temp - POLE_MASS_LENGTH * thetaacc * costheta / TOTAL_MASS;

    x = x + TAU * x_dot;
    x_dot = x_dot + TAU * xacc;
    theta = theta + TAU * theta_dot;
    theta_dot = theta_dot + TAU * thetaacc;
    s[0] = x; s[1] = x_dot; s[2] = theta; s[3] = theta_dot;

    *steps += 1;
    int terminated = (x < -X_THRESHOLD) || (x > X_THRESHOLD) || (theta < -THETA_THRESHOLD) ||
                     (theta > THETA_THRESHOLD);
    int truncated = *steps >= 500;
    *done = (terminated || truncated) ? 1.0f : 0.0f;
    *reward = terminated ? 0.0f : 1.0f;
}

void orc_cartpole_reset(float s[4], int32_t *steps, int env, uint32_t seed) {
    /* Scalar[uint32](i * 2654435761 + seed): 64-bit product truncated to 32 bits */
    uint32_t rng = orc_xorshift32((uint32_t)((uint64_t)env * 2654435761ull + (uint64_t)seed));
    for (int k = 0; k < 4; ++k) s[k] = orc_random_range(&rng, -0.05f, 0.05f);
    *steps = 0;
}

void orc_cartpole_step_batch(float *states, int32_t *steps, const float *actions, float *rewards,
                             float *dones, float *obs, int batch) {
    for (int i = 0; i < batch; ++i) {
        orc_cartpole_step(states + 4 * i, steps + i, (int)actions[i], rewards + i, dones + i);
        for (int k = 0; k < 4; ++k) obs[4 * i + k] = states[4 * i + k];
    }
}

void orc_cartpole_reset_batch(float *states, int32_t *steps, int batch, uint32_t seed) {
    for (int i = 0; i < batch; ++i) orc_cartpole_reset(states + 4 * i, steps + i, i, seed);
}

void orc_cartpole_selective_reset_batch(float *states, int32_t *steps, float *dones, int batch,
                                        uint32_t seed) {
    for (int i = 0; i < batch; ++i) {
        if (dones[i] < 0.5f) continue;
        orc_cartpole_reset(states + 4 * i, steps + i, i, seed);
        dones[i] = 0.0f;
    }
}

/* ---------------------------------------------------------------- Pendulum */
/* row: [cos, sin, theta_dot, theta, step_count, done, total_reward, last_torque] */

void orc_pendulum_step(float s[8], float action, float *reward, float *done) {
    const float max_speed = (float)8.0, max_torque = (float)2.0, dt = (float)0.05;
    const float g = (float)10.0, m = (float)1.0, l = (float)1.0;
    float theta = s[3], theta_dot = s[2];

    float u = action * max_torque;
    if (u > max_torque) u = max_torque;
    else if (u < -max_torque) u = -max_torque;

    float sin_theta = f32_sin(theta);
    float theta_acc = (3.0f * g) / (2.0f * l) * sin_theta + (3.0f / (m * l * l)) * u;

    theta_dot = theta_dot + theta_acc * dt;
    theta = theta + theta_dot * dt;
    if (theta_dot > max_speed) theta_dot = max_speed;
    else if (theta_dot < -max_speed) theta_dot = -max_speed;

    const float pi_val = (float)3.14159265358979323846;
    const float two_pi = (float)(2.0 * 3.14159265358979323846);
    while (theta > pi_val) theta -= two_pi;
    while (theta < -pi_val) theta += two_pi;

    float steps = s[4] + 1.0f;
    float r = -(theta * theta + 0.1f * theta_dot * theta_dot + 0.001f * u * u);
    float d = (steps >= 200.0f) ? 1.0f : 0.0f;

    s[0] = f32_cos(theta);
    s[1] = f32_sin(theta);
    s[2] = theta_dot;
    s[3] = theta;
    s[4] = steps;
    s[5] = d;
    s[6] = s[6] + r;
    s[7] = u;
    *reward = r;
    *done = d;
}

void orc_pendulum_reset(float s[8], int env, uint64_t seed) {
    /* seed travels through a Scalar[float32] kernel argument, then Int(seed) */
    int64_t seed_i = (int64_t)(float)seed;
    uint64_t combined = (uint64_t)seed_i * 2654435761ull + (uint64_t)env * 12345ull;
    float u[4];
    orc_philox_uniform4(combined, 0, 0, u);
    float theta = (float)(((double)u[0] * 2.0 - 1.0) * 3.14159265358979323846);
    float theta_dot = (float)((double)u[1] * 2.0 - 1.0);
    for (int k = 0; k < 8; ++k) s[k] = 0.0f;
    s[0] = f32_cos(theta);
    s[1] = f32_sin(theta);
    s[2] = theta_dot;
    s[3] = theta;
}

void orc_pendulum_step_batch(float *states, const float *actions, float *rewards, float *dones,
                             float *obs, int batch) {
    for (int i = 0; i < batch; ++i) {
        float *s = states + 8 * i;
        orc_pendulum_step(s, actions[i], rewards + i, dones + i);
        obs[3 * i + 0] = s[0]; obs[3 * i + 1] = s[1]; obs[3 * i + 2] = s[2];
    }
}

void orc_pendulum_reset_batch(float *states, int batch, uint64_t seed) {
    for (int i = 0; i < batch; ++i) orc_pendulum_reset(states + 8 * i, i, seed);
}

void orc_pendulum_selective_reset_batch(float *states, float *dones, int batch, uint64_t seed) {
    for (int i = 0; i < batch; ++i) {
        if (dones[i] > 0.5f) {
            orc_pendulum_reset(states + 8 * i, i, seed);
            dones[i] = 0.0f;
        }
    }
}
