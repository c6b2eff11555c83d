// LunarLanderV2 on one env row (one lane per env, row resident in LDS).
//
// Arithmetic: the reference's CPU path -- engines in fp64
// (envs/lunar_lander/lunar_lander_v2.mojo:1025-1095), physics step order :1097-1168,
// observation normalised in fp64 and rounded to fp32 (:699-775,
// envs/lunar_lander/helpers.mojo:10-64), reward and terminations :1192-1255 +
// helpers.mojo:92-133, reset :443-634.
// Buffer protocol: the batched trait's (:1453-1517, :1591-1966, :2109-2482) -- obs at
// row[0:8], metadata [step_count, total_reward, prev_shaping, done], a finished row
// reports (reward 0, done 1) until it is reset, engine dispersion drawn from
// Philox(seed = env + 12345, offset = step_count), reset seed
// Int(f32(seed)) * 2654435761 + (env + 1) * 12345.
#pragma once
#include "physics2d_reg.hpp"

namespace mrl {
namespace ll {

// joint j hangs leg j + 1 on the lander body (reset_row below, lunar_lander_v2.mojo:560-634)
struct Topology {
    static constexpr bool STATIC = true;
    static constexpr MRL_DEV int a(int) { return 0; }
    static constexpr MRL_DEV int b(int j) { return j + 1; }
};

using L = LunarLanderLayout;
constexpr int STATE = L::STATE_SIZE;  // 192
constexpr int OBS = 8;
enum { META_STEP = 0, META_TOTAL_REWARD = 1, META_PREV_SHAPING = 2, META_DONE = 3 };

constexpr double SCALE = 30.0;
constexpr double LEG_AWAY = 20.0 / SCALE;
constexpr double LEG_DOWN = 18.0 / SCALE;
constexpr double LEG_W = 2.0 / SCALE;
constexpr double LEG_H = 8.0 / SCALE;
constexpr double LANDER_MASS = 5.0;
constexpr double LANDER_INERTIA = 2.0;
constexpr double LEG_MASS = 0.2;
constexpr double LEG_INERTIA = 0.02;
constexpr double MAIN_ENGINE_POWER = 13.0;
constexpr double SIDE_ENGINE_POWER = 0.6;
constexpr double W_UNITS = 600.0 / SCALE;
constexpr double H_UNITS = 400.0 / SCALE;
constexpr double HELIPAD_Y = H_UNITS / 4.0;
constexpr double HELIPAD_X = W_UNITS / 2.0;
constexpr double FPS = 50.0;
constexpr double DT = 0.02;
constexpr int TERRAIN_CHUNKS = 11;

// polygon table shared by all envs: hull (6 vertices) and two identical legs (4 vertices); behind it
// the wind setting of the context [on (0 / 1), wind power, turbulence power, unused], off by default
constexpr int WIND_OFF = 3 * SHAPE_SIZE, NSHAPE_FLOATS = WIND_OFF + 4;
struct Shapes { float v[NSHAPE_FLOATS]; };
inline Shapes make_shapes() {
    Shapes s{};
    const double lv[6][2] = {{-14.0, 17.0}, {-17.0, 0.0}, {-17.0, -10.0},
                             {17.0, -10.0}, {17.0, 0.0},  {14.0, 17.0}};
    s.v[0] = 0.0f; s.v[1] = 6.0f;
    for (int i = 0; i < 6; ++i) {
        s.v[2 + 2 * i] = (float)(lv[i][0] / SCALE);
        s.v[3 + 2 * i] = (float)(lv[i][1] / SCALE);
    }
    const double gv[4][2] = {{-LEG_W, LEG_H}, {-LEG_W, -LEG_H}, {LEG_W, -LEG_H}, {LEG_W, LEG_H}};
    for (int k = 1; k <= 2; ++k) {
        float *S = s.v + SHAPE_SIZE * k;
        S[0] = 0.0f; S[1] = 4.0f;
        for (int i = 0; i < 4; ++i) { S[2 + 2 * i] = (float)gv[i][0]; S[3 + 2 * i] = (float)gv[i][1]; }
    }
    return s;
}

MRL_DEV double terrain_height(const float *row, double x) {
    const double chunk_width = W_UNITS / (double)(TERRAIN_CHUNKS - 1);
    int idx = (int)(x / chunk_width);
    if (idx < 0) idx = 0;
    if (idx >= TERRAIN_CHUNKS) idx = TERRAIN_CHUNKS - 1;
    const float *E = row + L::EDGES_OFF;
    return (idx < TERRAIN_CHUNKS - 1) ? (double)E[idx * 6 + 1] : (double)E[(TERRAIN_CHUNKS - 2) * 6 + 3];
}

MRL_DEV void observe(const float *row, float obs[8]) {
    const float *B0 = row + L::BODIES_OFF;
    const float *B1 = B0 + BODY_SIZE, *B2 = B0 + 2 * BODY_SIZE;
    double x = B0[IDX_X], y = B0[IDX_Y], vx = B0[IDX_VX], vy = B0[IDX_VY];
    double omega = B0[IDX_OMEGA];
    obs[0] = (float)((x - HELIPAD_X) / (W_UNITS / 2.0));
    obs[1] = (float)((y - (HELIPAD_Y + LEG_DOWN / SCALE)) / (H_UNITS / 2.0));
    obs[2] = (float)(vx * (W_UNITS / 2.0) / FPS);
    obs[3] = (float)(vy * (H_UNITS / 2.0) / FPS);
    obs[4] = B0[IDX_ANGLE];
    obs[5] = (float)(20.0 * omega / FPS);
    double left_y = B1[IDX_Y], left_x = B1[IDX_X], right_y = B2[IDX_Y], right_x = B2[IDX_X];
    obs[6] = (left_y - LEG_H <= terrain_height(row, left_x) + 0.01) ? 1.0f : 0.0f;
    obs[7] = (right_y - LEG_H <= terrain_height(row, right_x) + 0.01) ? 1.0f : 0.0f;
}

MRL_DEV float shaping(const float o[8]) {
    float dist = sqrtf(o[0] * o[0] + o[1] * o[1]);
    float speed = sqrtf(o[2] * o[2] + o[3] * o[3]);
    float abs_angle = (o[4] >= 0.0f) ? o[4] : -o[4];
    return -100.0f * dist - 100.0f * speed - 100.0f * abs_angle + 10.0f * o[6] + 10.0f * o[7];
}

MRL_DEV void set_body(float *B, double x, double y, double vx, double vy, double mass,
                      double inertia, int shape) {
    B[IDX_X] = (float)x; B[IDX_Y] = (float)y; B[IDX_ANGLE] = 0.0f;
    B[IDX_VX] = (float)vx; B[IDX_VY] = (float)vy; B[IDX_OMEGA] = 0.0f;
    B[IDX_FX] = 0.0f; B[IDX_FY] = 0.0f; B[IDX_TAU] = 0.0f;
    B[IDX_MASS] = (float)mass;
    B[IDX_INV_MASS] = (float)(1.0 / mass);
    B[IDX_INV_INERTIA] = (float)(1.0 / inertia);
    B[IDX_SHAPE] = (float)shape;
}

MRL_DEV void set_joint(float *J, int body_b, double ax, double ay, double bx, double by, double lo,
                       double hi) {
    for (int k = 0; k < JOINT_SIZE; ++k) J[k] = 0.0f;
    J[J_BODY_B] = (float)body_b;
    J[J_AX] = (float)ax; J[J_AY] = (float)ay; J[J_BX] = (float)bx; J[J_BY] = (float)by;
    J[J_LO] = (float)lo; J[J_HI] = (float)hi;
    J[J_STIFF] = (float)400.0; J[J_DAMP] = (float)40.0;
    J[J_FLAGS] = (float)(JF_SPRING | JF_LIMIT);
}

MRL_DEV uint64_t combined_seed(uint64_t seed, int env) {
    int64_t seed_i = (int64_t)(float)seed;
    return (uint64_t)seed_i * 2654435761ull + (uint64_t)(env + 1) * 12345ull;
}

// writes every float of the row
MRL_DEV void reset_row(float *row, uint64_t cseed) {
    for (int k = 0; k < STATE; ++k) row[k] = 0.0f;
    Uniform4 rv = philox_uniform4(cseed, 0, 0);

    double raw[TERRAIN_CHUNKS + 1];
#pragma unroll
    for (int c = 0; c < TERRAIN_CHUNKS + 1; ++c)
        raw[c] = (double)philox_uniform4(cseed + 1000ull, 0, (uint64_t)c).v[0] * (H_UNITS / 2.0);
    float heights[TERRAIN_CHUNKS];
#pragma unroll
    for (int c = 0; c < TERRAIN_CHUNKS; ++c) {
        double s;
        if (c == 0) s = (raw[0] + raw[0] + raw[1]) / 3.0;
        else if (c == TERRAIN_CHUNKS - 1) s = (raw[c - 1] + raw[c] + raw[c]) / 3.0;
        else s = (raw[c - 1] + raw[c] + raw[c + 1]) / 3.0;
        heights[c] = (float)s;
        if (c >= TERRAIN_CHUNKS / 2 - 2 && c < TERRAIN_CHUNKS / 2 + 3) heights[c] = (float)HELIPAD_Y;
    }
    // physics2d/collision/edge_terrain.mojo:93-147, fp64
    const double x_spacing = W_UNITS / (double)(TERRAIN_CHUNKS - 1);
#pragma unroll
    for (int i = 0; i < TERRAIN_CHUNKS - 1; ++i) {
        double x0 = 0.0 + (double)i * x_spacing, y0 = (double)heights[i];
        double x1 = 0.0 + (double)(i + 1) * x_spacing, y1 = (double)heights[i + 1];
        double dx = x1 - x0, dy = y1 - y0;
        double length = ::sqrt(dx * dx + dy * dy);
        double nx = -dy / length, ny = dx / length;
        if (ny < 0) { nx = -nx; ny = -ny; }
        float *E = row + L::EDGES_OFF + i * 6;
        E[0] = (float)x0; E[1] = (float)y0; E[2] = (float)x1; E[3] = (float)y1;
        E[4] = (float)nx; E[5] = (float)ny;
    }
    row[L::EDGE_COUNT_OFF] = (float)(TERRAIN_CHUNKS - 1);

    double init_x = HELIPAD_X, init_y = H_UNITS;
    double init_fx = ((double)rv.v[0] * 2.0 - 1.0) * 1000.0;
    double init_fy = ((double)rv.v[1] * 2.0 - 1.0) * 1000.0;
    double init_vx = init_fx * DT / LANDER_MASS;
    double init_vy = init_fy * DT / LANDER_MASS;
    float *B = row + L::BODIES_OFF;
    set_body(B, init_x, init_y, init_vx, init_vy, LANDER_MASS, LANDER_INERTIA, 0);
    double leg_y = init_y - (10.0 / SCALE) - LEG_DOWN;
    set_body(B + BODY_SIZE, init_x - LEG_AWAY, leg_y, init_vx, init_vy, LEG_MASS, LEG_INERTIA, 1);
    set_body(B + 2 * BODY_SIZE, init_x + LEG_AWAY, leg_y, init_vx, init_vy, LEG_MASS, LEG_INERTIA, 2);
    float *J = row + L::JOINTS_OFF;
    set_joint(J, 1, -LEG_AWAY, -10.0 / SCALE, 0.0, LEG_H, 0.4, 0.9);
    set_joint(J + JOINT_SIZE, 2, LEG_AWAY, -10.0 / SCALE, 0.0, LEG_H, -0.9, -0.4);
    row[L::JOINT_COUNT_OFF] = 2.0f;

    float obs[8];
    observe(row, obs);
#pragma unroll
    for (int k = 0; k < 8; ++k) row[k] = obs[k];
    row[L::META_OFF + META_PREV_SHAPING] = shaping(obs);
}

// Same row as reset_row, written by the 64 lanes of one wavefront together: the 13 Philox draws,
// the 11 smoothed heights and the 10 edges each go to their own lane, the row is zero-filled in
// stripes, and bodies / joints / counters are set by separate lanes.  Every value is computed by
// the same expressions as in reset_row, so the result is bit-identical; only who computes it
// differs.  All lanes of the wavefront must call this with the same `row`.
MRL_DEV void reset_row_wave(float *row, uint64_t cseed, int lane) {
    for (int k = lane; k < STATE; k += 64) row[k] = 0.0f;
    // lane 0: velocity draw; lanes 1..12: terrain draws 0..11 of the second stream
    Uniform4 u = philox_uniform4(lane == 0 ? cseed : cseed + 1000ull, 0,
                                 lane == 0 ? 0ull : (uint64_t)((lane - 1) & 15));
    const double raw = (double)u.v[0] * (H_UNITS / 2.0);       // lanes 1..12: raw[lane - 1]
    const double raw_m = __shfl(raw, (lane + 63) & 63, 64);     // raw[lane - 2]
    const double raw_p = __shfl(raw, (lane + 1) & 63, 64);      // raw[lane]
    const int c = lane - 1;                                      // chunk index on lanes 1..11
    double sm;
    if (c == 0) sm = (raw + raw + raw_p) / 3.0;
    else if (c == TERRAIN_CHUNKS - 1) sm = (raw_m + raw + raw) / 3.0;
    else sm = (raw_m + raw + raw_p) / 3.0;
    float h = (float)sm;
    if (c >= TERRAIN_CHUNKS / 2 - 2 && c < TERRAIN_CHUNKS / 2 + 3) h = (float)HELIPAD_Y;
    const float h_next = __shfl(h, (lane + 1) & 63, 64);
    if (c >= 0 && c < TERRAIN_CHUNKS - 1) {                      // edge c from heights c, c + 1
        const double x_spacing = W_UNITS / (double)(TERRAIN_CHUNKS - 1);
        double x0 = 0.0 + (double)c * x_spacing, y0 = (double)h;
        double x1 = 0.0 + (double)(c + 1) * x_spacing, y1 = (double)h_next;
        double dx = x1 - x0, dy = y1 - y0;
        double length = ::sqrt(dx * dx + dy * dy);
        double nx = -dy / length, ny = dx / length;
        if (ny < 0) { nx = -nx; ny = -ny; }
        float *E = row + L::EDGES_OFF + c * 6;
        E[0] = (float)x0; E[1] = (float)y0; E[2] = (float)x1; E[3] = (float)y1;
        E[4] = (float)nx; E[5] = (float)ny;
    }
    const float u0 = __shfl(u.v[0], 0, 64), u1 = __shfl(u.v[1], 0, 64);
    const double init_x = HELIPAD_X, init_y = H_UNITS;
    const double init_vx = (((double)u0 * 2.0 - 1.0) * 1000.0) * DT / LANDER_MASS;
    const double init_vy = (((double)u1 * 2.0 - 1.0) * 1000.0) * DT / LANDER_MASS;
    const double leg_y = init_y - (10.0 / SCALE) - LEG_DOWN;
    float *B = row + L::BODIES_OFF;
    float *J = row + L::JOINTS_OFF;
    if (lane == 16) set_body(B, init_x, init_y, init_vx, init_vy, LANDER_MASS, LANDER_INERTIA, 0);
    if (lane == 17) set_body(B + BODY_SIZE, init_x - LEG_AWAY, leg_y, init_vx, init_vy, LEG_MASS, LEG_INERTIA, 1);
    if (lane == 18) set_body(B + 2 * BODY_SIZE, init_x + LEG_AWAY, leg_y, init_vx, init_vy, LEG_MASS, LEG_INERTIA, 2);
    if (lane == 19) set_joint(J, 1, -LEG_AWAY, -10.0 / SCALE, 0.0, LEG_H, 0.4, 0.9);
    if (lane == 20) set_joint(J + JOINT_SIZE, 2, LEG_AWAY, -10.0 / SCALE, 0.0, LEG_H, -0.9, -0.4);
    if (lane == 21) {
        row[L::EDGE_COUNT_OFF] = (float)(TERRAIN_CHUNKS - 1);
        row[L::JOINT_COUNT_OFF] = 2.0f;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (lane == 0) {
        float obs[8];
        observe(row, obs);
#pragma unroll
        for (int k = 0; k < 8; ++k) row[k] = obs[k];
        row[L::META_OFF + META_PREV_SHAPING] = shaping(obs);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

MRL_DEV void apply_engines(float *row, int env, int step_count, double m_power, double s_power,
                           double direction) {
    if (m_power == 0.0 && s_power == 0.0) return;
    float *B = row + L::BODIES_OFF;
    double angle = B[IDX_ANGLE], vx = B[IDX_VX], vy = B[IDX_VY], omega = B[IDX_OMEGA];
    double tip_x, tip_y;
    ::sincos(angle, &tip_x, &tip_y);
    double side_x = -tip_y, side_y = tip_x;
    Uniform4 rv = philox_uniform4((uint64_t)((int64_t)env + 12345), (uint64_t)step_count, 0);
    double dispersion_x = ((double)rv.v[0] * 2.0 - 1.0) / SCALE;
    double dispersion_y = ((double)rv.v[1] * 2.0 - 1.0) / SCALE;
    double dvx = 0.0, dvy = 0.0, domega = 0.0;
    if (m_power > 0.0) {
        double main_y_offset = 4.0 / SCALE;
        double ox = tip_x * (main_y_offset + 2.0 * dispersion_x) + side_x * dispersion_y;
        double oy = -tip_y * (main_y_offset + 2.0 * dispersion_x) - side_y * dispersion_y;
        double impulse_x = -ox * MAIN_ENGINE_POWER * m_power;
        double impulse_y = -oy * MAIN_ENGINE_POWER * m_power;
        dvx += impulse_x / LANDER_MASS;
        dvy += impulse_y / LANDER_MASS;
        double torque = ox * impulse_y - oy * impulse_x;
        domega += torque / LANDER_INERTIA;
    }
    if (s_power > 0.0) {
        double side_away = 12.0 / SCALE;
        double ox = tip_x * dispersion_x + side_x * (3.0 * dispersion_y + direction * side_away);
        double oy = -tip_y * dispersion_x - side_y * (3.0 * dispersion_y + direction * side_away);
        double impulse_x = -ox * SIDE_ENGINE_POWER * s_power;
        double impulse_y = -oy * SIDE_ENGINE_POWER * s_power;
        dvx += impulse_x / LANDER_MASS;
        dvy += impulse_y / LANDER_MASS;
        double side_height = 14.0 / SCALE;
        double r_x = ox - tip_x * 17.0 / SCALE;
        double r_y = oy + tip_y * side_height;
        double torque = r_x * impulse_y - r_y * impulse_x;
        domega += torque / LANDER_INERTIA;
    }
    B[IDX_VX] = (float)(vx + dvx);
    B[IDX_VY] = (float)(vy + dvy);
    B[IDX_OMEGA] = (float)(omega + domega);
}

// An env step in two halves, so that contact detection -- which reads positions only -- can run
// on other wavefronts while this one applies the engines (which write velocities only):
//   step_begin   already-finished short-circuit, engine impulses;
//   step_finish  physics with the `n` contacts given in `contacts` (n < 0: detect here),
//                observation, reward, termination.
struct StepCarry {
    int step_count;
    double m_power, s_power;
    bool skip;   // the row was already finished: reward 0, done 1, nothing moves
};

// Wind and turbulence (struct parameters ENABLE_WIND / WIND_POWER / TURBULENCE_POWER of the reference,
// lunar_lander_v2.mojo:123-127; _apply_wind, :983-1023): skipped while a leg touches the ground;
// otherwise tanh(sin(0.02 t) + sin(pi 0.01 t)) times the power as an impulse on the lander's vx and
// omega, in Float64, before the engines.  t is the row's step count, as in the GPU trait (:2041-2105):
// the row has no slot for the CPU env's two running indices.
MRL_DEV void apply_wind(float *row, int step_count, const float *shapes) {
    if (!(shapes[WIND_OFF] > 0.5f)) return;
    if (row[6] > 0.5f || row[7] > 0.5f) return;
    const double k = 0.01, t = (double)step_count, pi = 3.14159265358979323846;
    const double wind_mag = ::tanh(::sin(0.02 * t) + ::sin(pi * k * t)) * (double)shapes[WIND_OFF + 1];
    const double torque_mag = ::tanh(::sin(0.02 * t) + ::sin(pi * k * t)) * (double)shapes[WIND_OFF + 2];
    float *B = row + L::BODIES_OFF;
    const double vx = (double)B[IDX_VX], omega = (double)B[IDX_OMEGA];
    const double dvx = wind_mag * DT / LANDER_MASS;
    const double domega = torque_mag * DT / LANDER_INERTIA;
    B[IDX_VX] = (float)(vx + dvx);
    B[IDX_OMEGA] = (float)(omega + domega);
}

MRL_DEV StepCarry step_begin(float *row, int env, int action, const float *shapes) {
    StepCarry c;
    c.skip = row[L::META_OFF + META_DONE] > 0.5f;
    c.step_count = (int)row[L::META_OFF + META_STEP];
    c.m_power = 0.0; c.s_power = 0.0;
    double direction = 0.0;
    if (action == 2) c.m_power = 1.0;
    else if (action == 1) { c.s_power = 1.0; direction = -1.0; }
    else if (action == 3) { c.s_power = 1.0; direction = 1.0; }
    if (!c.skip) {
        apply_wind(row, c.step_count, shapes);
        apply_engines(row, env, c.step_count, c.m_power, c.s_power, direction);
    }
    return c;
}

// The continuous-action overload (step_continuous_vec, lunar_lander_v2.mojo:1329-1383, decoded in
// fp64 like the rest of the engine arithmetic): a[0] in [-1, 1] is the main throttle, remapped to
// (a0 + 1) / 2 and clipped to [0, 1]; a[1] clipped to [-1, 1] fires the left (< -0.5) or right
// (> 0.5) engine with power (|a1| - 0.5) * 2.  Both engines can fire in one step.
MRL_DEV StepCarry step_begin_continuous(float *row, int env, const float *a, const float *shapes) {
    StepCarry c;
    c.skip = row[L::META_OFF + META_DONE] > 0.5f;
    c.step_count = (int)row[L::META_OFF + META_STEP];
    double m_power = ((double)a[0] + 1.0) * 0.5;
    if (m_power < 0.0) m_power = 0.0;
    if (m_power > 1.0) m_power = 1.0;
    double side_action = (double)a[1], s_power = 0.0, direction = 0.0;
    if (side_action < -1.0) side_action = -1.0;
    if (side_action > 1.0) side_action = 1.0;
    if (side_action < -0.5) { direction = -1.0; s_power = (-side_action - 0.5) * 2.0; }
    else if (side_action > 0.5) { direction = 1.0; s_power = (side_action - 0.5) * 2.0; }
    c.m_power = m_power; c.s_power = s_power;
    if (!c.skip) {
        apply_wind(row, c.step_count, shapes);
        apply_engines(row, env, c.step_count, m_power, s_power, direction);
    }
    return c;
}

MRL_DEV void step_finish(float *row, float *contacts, int n_given, const float *shapes, const StepCarry &c,
                         float &reward, float &done) {
    if (c.skip) {
        reward = 0.0f;
        done = 1.0f;
        return;
    }
    const double m_power = c.m_power, s_power = c.s_power;
    int step_count = c.step_count;
    const float gx = (float)0.0, gy = (float)-10.0, dt = (float)DT;
    const float friction = (float)0.1, restitution = (float)0.0;
    const float baumgarte = (float)0.2, slop = (float)0.005;
    const int n = reg_physics_substep<L, Topology, false, true>(row, shapes, contacts, gx, gy, dt, friction,
                                                                restitution, baumgarte, slop, 6, 2, n_given);

    step_count += 1;
    float obs[8];
    observe(row, obs);
    const float *B = row + L::BODIES_OFF;
    double vx = B[IDX_VX], vy = B[IDX_VY], omega = B[IDX_OMEGA];
    float new_shaping = shaping(obs);
    float r = new_shaping - row[L::META_OFF + META_PREV_SHAPING];
    r = r - (float)(m_power * 0.30);
    r = r - (float)(s_power * 0.03);
    bool terminated = false;
    if (obs[0] >= 1.0f || obs[0] <= -1.0f) { terminated = true; r = -100.0f; }
    bool both_legs = obs[6] > 0.5f && obs[7] > 0.5f;
    double speed = ::sqrt(vx * vx + vy * vy);
    // every slot is read (one round trip to the lane's scratch for all of them), the count cuts afterwards
    bool lander_contact = false;
#pragma unroll
    for (int k = 0; k < L::MAX_CONTACTS; ++k) {
        const int body = (int)contacts[k * CONTACT_SIZE + C_BODY_A];
        lander_contact = lander_contact || (k < n && body == 0);
    }
    if (lander_contact) { terminated = true; r = -100.0f; }
    if (speed < 0.01 && ::fabs(omega) < 0.01 && both_legs) { terminated = true; r = r + 100.0f; }
    if (step_count >= 1000) terminated = true;

#pragma unroll
    for (int k = 0; k < 8; ++k) row[k] = obs[k];
    row[L::META_OFF + META_STEP] = (float)step_count;
    row[L::META_OFF + META_PREV_SHAPING] = new_shaping;
    row[L::META_OFF + META_DONE] = terminated ? 1.0f : 0.0f;
    reward = r;
    done = terminated ? 1.0f : 0.0f;
}

// one env step on an LDS-resident row by one lane; `contacts` = this lane's contact scratch
MRL_DEV void step_row(float *row, float *contacts, const float *shapes, int env, int action,
                      float &reward, float &done) {
    const StepCarry c = step_begin(row, env, action, shapes);
    step_finish(row, contacts, -1, shapes, c, reward, done);
}

}  // namespace ll
}  // namespace mrl
