// CartPole and Pendulum, one lane per environment.
//
// CartPole step : envs/cartpole.mojo:394-460 (CPU step_raw: reward 0 on termination,
//                 truncation at 500 steps).  The [B,4] state row of the batched trait has
//                 no step counter, so the counter lives in a per-env int32 side array
//                 owned by the library context.
// CartPole reset: envs/cartpole.mojo:784-905 (xorshift32(i*2654435761 + seed), four
//                 random_range(-0.05, 0.05) draws; selective reset clears dones[i]).
// Pendulum      : envs/pendulum/pendulum_v2.mojo:640-661, :734-792 (CPU arithmetic) on the
//                 8-float row [cos, sin, theta_dot, theta, step, done, total_reward, last_u]
//                 of envs/pendulum/constants.mojo; reset :294-399, :548-623.
#pragma once
#include "mrl_device.hpp"

namespace mrl {
namespace cartpole {

constexpr int STATE = 4, OBS = 4;

MRL_DEV void step(float s[4], int32_t &steps, int action, float &reward, float &done) {
    const float GRAVITY = (float)9.8, TOTAL_MASS = (float)(1.0 + 0.1), POLE_MASS = (float)0.1;
    const float POLE_HALF_LENGTH = (float)0.5, POLE_MASS_LENGTH = (float)(0.1 * 0.5);
    const float FORCE_MAG = (float)10.0, TAU = (float)0.02;
    const float X_THRESHOLD = (float)2.4, THETA_THRESHOLD = (float)0.2095;
    float x = s[0], x_dot = s[1], theta = s[2], theta_dot = s[3];
    float force = (action == 1) ? FORCE_MAG : -FORCE_MAG;
    float sintheta, costheta;
    sincos32(theta, sintheta, costheta);
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
    steps += 1;
    bool terminated = (x < -X_THRESHOLD) || (x > X_THRESHOLD) || (theta < -THETA_THRESHOLD) ||
                      (theta > THETA_THRESHOLD);
    bool truncated = steps >= 500;
    done = (terminated || truncated) ? 1.0f : 0.0f;
    reward = terminated ? 0.0f : 1.0f;
}

MRL_DEV void reset(float s[4], int32_t &steps, int env, uint32_t seed) {
    uint32_t rng = xorshift32((uint32_t)((uint64_t)env * 2654435761ull + (uint64_t)seed));
#pragma unroll
    for (int k = 0; k < 4; ++k) s[k] = random_range(rng, -0.05f, 0.05f);
    steps = 0;
}

}  // namespace cartpole

namespace pendulum {

constexpr int STATE = 8, OBS = 3;

MRL_DEV void step(float s[8], float action, float &reward, float &done) {
    const float max_speed = (float)8.0, max_torque = (float)2.0, dt = (float)0.05;
    const float g = (float)10.0, m = (float)1.0, l = (float)1.0;
    float theta = s[3], theta_dot = s[2];
    float u = action * max_torque;
    if (u > max_torque) u = max_torque;
    else if (u < -max_torque) u = -max_torque;
    float sin_theta = sin32(theta);
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
    float sn, cs;
    sincos32(theta, sn, cs);
    s[0] = cs; s[1] = sn; s[2] = theta_dot; s[3] = theta;
    s[4] = steps; s[5] = d; s[6] = s[6] + r; s[7] = u;
    reward = r;
    done = d;
}

MRL_DEV void reset(float s[8], int env, uint64_t seed) {
    int64_t seed_i = (int64_t)(float)seed;
    uint64_t combined = (uint64_t)seed_i * 2654435761ull + (uint64_t)env * 12345ull;
    Uniform4 u = philox_uniform4(combined, 0, 0);
    float theta = (float)(((double)u.v[0] * 2.0 - 1.0) * 3.14159265358979323846);
    float theta_dot = (float)((double)u.v[1] * 2.0 - 1.0);
    float sn, cs;
    sincos32(theta, sn, cs);
    s[0] = cs; s[1] = sn; s[2] = theta_dot; s[3] = theta;
    s[4] = 0.0f; s[5] = 0.0f; s[6] = 0.0f; s[7] = 0.0f;
}

}  // namespace pendulum
}  // namespace mrl
