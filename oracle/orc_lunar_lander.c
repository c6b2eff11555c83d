/*
 * LunarLanderV2: CPU restatement (test infrastructure, never shipped).
 *
 * Arithmetic follows the reference's CPU path, on the flat 192-float row that its
 * CPU and GPU paths share (physics2d/layout.mojo:247-255):
 *   constants            envs/lunar_lander/constants.mojo:9-130
 *   shapes               envs/lunar_lander/lunar_lander_v2.mojo:259-289
 *   reset                lunar_lander_v2.mojo:443-634 (_reset_cpu), row writes as
 *                        :1709-1966 (_reset_env_gpu), seed combination :1618-1638
 *   engines              lunar_lander_v2.mojo:1025-1095 (_apply_engines, Float64)
 *   continuous actions   lunar_lander_v2.mojo:1329-1383 (step_continuous_vec: throttle and side
 *                        control decoded in Float64) + :1385-1436 (_step_cpu_continuous)
 *   physics step         lunar_lander_v2.mojo:1097-1168 (_step_physics_cpu)
 *   observation          lunar_lander_v2.mojo:699-775 + envs/lunar_lander/helpers.mojo:10-64
 *   reward / termination lunar_lander_v2.mojo:1192-1255 + helpers.mojo:92-133
 *
 * Buffer protocol of the batched trait (what a row holds between calls, the
 * done-row short circuit "reward 0, done 1", obs copied out of row[0:8], dispersion
 * stream Philox(seed = env + 12345, offset = step_count)) follows
 * lunar_lander_v2.mojo:2109-2262, :2266-2482, :2624-2750.  The CPU struct is the
 * env = 0 instance of that protocol (its comment at :1040-1044 says so).
 * The CPU struct keeps terrain heights in a side list; here they are read back from
 * the row's edges (edge i holds heights i and i+1), which hold the same fp32 values.
 */
#include <math.h>
#include <string.h>
#include "orc.h"

#define SCALE 30.0
#define LEG_AWAY (20.0 / SCALE)
#define LEG_DOWN (18.0 / SCALE)
#define LEG_W (2.0 / SCALE)
#define LEG_H (8.0 / SCALE)
#define LANDER_MASS 5.0
#define LANDER_INERTIA 2.0
#define LEG_MASS 0.2
#define LEG_INERTIA 0.02
#define MAIN_ENGINE_POWER 13.0
#define SIDE_ENGINE_POWER 0.6
#define W_UNITS (600.0 / SCALE)
#define H_UNITS (400.0 / SCALE)
#define HELIPAD_Y (H_UNITS / 4.0)
#define HELIPAD_X (W_UNITS / 2.0)
#define FPS 50.0
#define DT 0.02
#define TERRAIN_CHUNKS 11

enum { META_STEP = 0, META_TOTAL_REWARD = 1, META_PREV_SHAPING = 2, META_DONE = 3 };

void orc_ll_layout(orc_layout *L) { orc_layout_make(L, 3, 8, 2, 16, 8, 4, 3); }

void orc_ll_shapes(float shapes[3 * 20]) {
    memset(shapes, 0, sizeof(float) * 60);
    const double lv[6][2] = {{-14.0, 17.0}, {-17.0, 0.0}, {-17.0, -10.0},
                             {17.0, -10.0}, {17.0, 0.0},  {14.0, 17.0}};
    shapes[0] = 0.0f; shapes[1] = 6.0f;
    for (int i = 0; i < 6; ++i) {
        shapes[2 + 2 * i] = (float)(lv[i][0] / SCALE);
        shapes[3 + 2 * i] = (float)(lv[i][1] / SCALE);
    }
    const double gv[4][2] = {{-LEG_W, LEG_H}, {-LEG_W, -LEG_H}, {LEG_W, -LEG_H}, {LEG_W, LEG_H}};
    for (int s = 1; s <= 2; ++s) {
        float *S = shapes + 20 * s;
        S[0] = 0.0f; S[1] = 4.0f;
        for (int i = 0; i < 4; ++i) { S[2 + 2 * i] = (float)gv[i][0]; S[3 + 2 * i] = (float)gv[i][1]; }
    }
}

uint64_t orc_ll_combined_seed(uint64_t seed, int env) {
    int64_t seed_i = (int64_t)(float)seed; /* Scalar[float32](rng_seed) then Int(seed) */
    return (uint64_t)seed_i * 2654435761ull + (uint64_t)(env + 1) * 12345ull;
}

static double terrain_height(const orc_layout *L, const float *row, double x) {
    double chunk_width = W_UNITS / (double)(TERRAIN_CHUNKS - 1);
    int idx = (int)(x / chunk_width);
    if (idx < 0) idx = 0;
    if (idx >= TERRAIN_CHUNKS) idx = TERRAIN_CHUNKS - 1;
    const float *E = row + L->edges_off;
    return (idx < TERRAIN_CHUNKS - 1) ? (double)E[idx * 6 + 1] : (double)E[(TERRAIN_CHUNKS - 2) * 6 + 3];
}

/* get_observation: Float64 normalisation, cast to fp32 */
static void observe(const orc_layout *L, const float *row, float obs[8]) {
    const float *B0 = row + L->bodies_off;
    const float *B1 = B0 + ORC_BODY_SIZE, *B2 = B0 + 2 * ORC_BODY_SIZE;
    double x = B0[ORC_IDX_X], y = B0[ORC_IDX_Y], vx = B0[ORC_IDX_VX], vy = B0[ORC_IDX_VY];
    double angle = B0[ORC_IDX_ANGLE], omega = B0[ORC_IDX_OMEGA];
    double x_norm = (x - HELIPAD_X) / (W_UNITS / 2.0);
    double y_norm = (y - (HELIPAD_Y + LEG_DOWN / SCALE)) / (H_UNITS / 2.0);
    double vx_norm = vx * (W_UNITS / 2.0) / FPS;
    double vy_norm = vy * (H_UNITS / 2.0) / FPS;
    double omega_norm = 20.0 * omega / FPS;
    double left_y = B1[ORC_IDX_Y], left_x = B1[ORC_IDX_X];
    double right_y = B2[ORC_IDX_Y], right_x = B2[ORC_IDX_X];
    double left_terrain = terrain_height(L, row, left_x);
    double right_terrain = terrain_height(L, row, right_x);
    obs[0] = (float)x_norm; obs[1] = (float)y_norm; obs[2] = (float)vx_norm; obs[3] = (float)vy_norm;
    obs[4] = (float)angle; obs[5] = (float)omega_norm;
    obs[6] = (left_y - LEG_H <= left_terrain + 0.01) ? 1.0f : 0.0f;
    obs[7] = (right_y - LEG_H <= right_terrain + 0.01) ? 1.0f : 0.0f;
}

static float shaping(const float o[8]) {
    float dist = sqrtf(o[0] * o[0] + o[1] * o[1]);
    float speed = sqrtf(o[2] * o[2] + o[3] * o[3]);
    float abs_angle = (o[4] >= 0.0f) ? o[4] : -o[4];
    return -100.0f * dist - 100.0f * speed - 100.0f * abs_angle + 10.0f * o[6] + 10.0f * o[7];
}

static void set_body(float *B, double x, double y, double vx, double vy, double mass, double inertia,
                     int shape) {
    memset(B, 0, sizeof(float) * ORC_BODY_SIZE);
    B[ORC_IDX_X] = (float)x; B[ORC_IDX_Y] = (float)y; B[ORC_IDX_ANGLE] = 0.0f;
    B[ORC_IDX_VX] = (float)vx; B[ORC_IDX_VY] = (float)vy; B[ORC_IDX_OMEGA] = 0.0f;
    B[ORC_IDX_MASS] = (float)mass;
    B[ORC_IDX_INV_MASS] = (float)(1.0 / mass);
    B[ORC_IDX_INV_INERTIA] = (float)(1.0 / inertia);
    B[ORC_IDX_SHAPE] = (float)shape;
}

static void set_joint(float *J, int body_b, double ax, double ay, double bx, double by, double lo,
                      double hi) {
    memset(J, 0, sizeof(float) * ORC_JOINT_SIZE);
    J[ORC_J_TYPE] = 0.0f; J[ORC_J_BODY_A] = 0.0f; J[ORC_J_BODY_B] = (float)body_b;
    J[ORC_J_AX] = (float)ax; J[ORC_J_AY] = (float)ay; J[ORC_J_BX] = (float)bx; J[ORC_J_BY] = (float)by;
    J[ORC_J_REF] = 0.0f; /* angle_b - angle_a at creation, both 0 */
    J[ORC_J_LO] = (float)lo; J[ORC_J_HI] = (float)hi;
    J[ORC_J_STIFF] = (float)400.0; J[ORC_J_DAMP] = (float)40.0;
    J[ORC_J_FLAGS] = (float)(ORC_JF_SPRING | ORC_JF_LIMIT);
}

void orc_ll_reset(float *row, uint64_t combined_seed) {
    orc_layout L; orc_ll_layout(&L);
    memset(row, 0, sizeof(float) * ORC_LL_STATE);

    float rv[4];
    orc_philox_uniform4(combined_seed, 0, 0, rv);

    double raw[TERRAIN_CHUNKS + 1];
    for (int c = 0; c < TERRAIN_CHUNKS + 1; ++c) {
        float t[4];
        orc_philox_uniform4(combined_seed + 1000ull, 0, (uint64_t)c, t);
        raw[c] = (double)t[0] * (H_UNITS / 2.0);
    }
    float heights[TERRAIN_CHUNKS];
    for (int c = 0; c < TERRAIN_CHUNKS; ++c) {
        double s;
        if (c == 0) s = (raw[0] + raw[0] + raw[1]) / 3.0;
        else if (c == TERRAIN_CHUNKS - 1) s = (raw[c - 1] + raw[c] + raw[c]) / 3.0;
        else s = (raw[c - 1] + raw[c] + raw[c + 1]) / 3.0;
        heights[c] = (float)s;
    }
    for (int c = TERRAIN_CHUNKS / 2 - 2; c < TERRAIN_CHUNKS / 2 + 3; ++c)
        if (c >= 0 && c < TERRAIN_CHUNKS) heights[c] = (float)HELIPAD_Y;
    orc_set_terrain_from_heights(&L, row, heights, TERRAIN_CHUNKS, 0.0,
                                 W_UNITS / (double)(TERRAIN_CHUNKS - 1));

    double init_x = HELIPAD_X, init_y = H_UNITS;
    double init_fx = ((double)rv[0] * 2.0 - 1.0) * 1000.0;
    double init_fy = ((double)rv[1] * 2.0 - 1.0) * 1000.0;
    double init_vx = init_fx * DT / LANDER_MASS;
    double init_vy = init_fy * DT / LANDER_MASS;

    float *B = row + L.bodies_off;
    set_body(B, init_x, init_y, init_vx, init_vy, LANDER_MASS, LANDER_INERTIA, 0);
    double leg_y = init_y - (10.0 / SCALE) - LEG_DOWN;
    set_body(B + ORC_BODY_SIZE, init_x - LEG_AWAY, leg_y, init_vx, init_vy, LEG_MASS, LEG_INERTIA, 1);
    set_body(B + 2 * ORC_BODY_SIZE, init_x + LEG_AWAY, leg_y, init_vx, init_vy, LEG_MASS, LEG_INERTIA, 2);

    float *J = row + L.joints_off;
    set_joint(J, 1, -LEG_AWAY, -10.0 / SCALE, 0.0, LEG_H, 0.4, 0.9);
    set_joint(J + ORC_JOINT_SIZE, 2, LEG_AWAY, -10.0 / SCALE, 0.0, LEG_H, -0.9, -0.4);
    row[L.joint_count_off] = 2.0f;

    float obs[8];
    observe(&L, row, obs);
    memcpy(row, obs, sizeof(obs));
    row[L.meta_off + META_STEP] = 0.0f;
    row[L.meta_off + META_TOTAL_REWARD] = 0.0f;
    row[L.meta_off + META_PREV_SHAPING] = shaping(obs);
    row[L.meta_off + META_DONE] = 0.0f;
}

static void apply_engines(const orc_layout *L, float *row, int env, int step_count, double m_power,
                          double s_power, double direction) {
    if (m_power == 0.0 && s_power == 0.0) return;
    float *B = row + L->bodies_off;
    double angle = B[ORC_IDX_ANGLE], vx = B[ORC_IDX_VX], vy = B[ORC_IDX_VY], omega = B[ORC_IDX_OMEGA];
    /* sin/cos of a Float64 that holds an fp32 angle */
    double tip_x = sin(angle), tip_y = cos(angle);
    double side_x = -tip_y, side_y = tip_x;
    float rv[4];
    orc_philox_uniform4((uint64_t)((int64_t)env + 12345), (uint64_t)step_count, 0, rv);
    double dispersion_x = ((double)rv[0] * 2.0 - 1.0) / SCALE;
    double dispersion_y = ((double)rv[1] * 2.0 - 1.0) / SCALE;
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
    B[ORC_IDX_VX] = (float)(vx + dvx);
    B[ORC_IDX_VY] = (float)(vy + dvy);
    B[ORC_IDX_OMEGA] = (float)(omega + domega);
}

static void step_powers(float *row, int env, double m_power, double s_power, double direction, float *reward,
                        float *done, float *contacts_out, int *n_contacts_out);

/* Wind and turbulence, the struct parameters ENABLE_WIND / WIND_POWER / TURBULENCE_POWER of the
 * reference (lunar_lander_v2.mojo:123-127), off by default: one setting for all rows stepped after
 * the call.  _apply_wind (CPU, :983-1023): skipped while a leg touches the ground; otherwise
 * tanh(sin(0.02 t) + sin(pi 0.01 t)) times the power, as an impulse on the lander's vx and omega, in
 * Float64, before the engines.  The CPU env keeps two running indices that start at random values of
 * its own generator; the GPU row has no slot for them and the GPU trait uses the step count of the row
 * for both (:2041-2105): that protocol is followed here, with the CPU's Float64 arithmetic. */
static int g_wind_on = 0;
static double g_wind_power = 15.0, g_turbulence_power = 1.5;
void orc_ll_set_wind(int enable, double wind_power, double turbulence_power) {
    g_wind_on = enable;
    g_wind_power = wind_power;
    g_turbulence_power = turbulence_power;
}
static void apply_wind(const orc_layout *L, float *row, int step_count) {
    if (!g_wind_on) return;
    if (row[6] > 0.5f || row[7] > 0.5f) return;
    const double k = 0.01, t = (double)step_count, pi = 3.14159265358979323846;
    const double wind_mag = tanh(sin(0.02 * t) + sin(pi * k * t)) * g_wind_power;
    const double torque_mag = tanh(sin(0.02 * t) + sin(pi * k * t)) * g_turbulence_power;
    float *B = row + L->bodies_off;
    const double vx = (double)B[ORC_IDX_VX], omega = (double)B[ORC_IDX_OMEGA];
    const double dvx = wind_mag * DT / LANDER_MASS;
    const double domega = torque_mag * DT / LANDER_INERTIA;
    B[ORC_IDX_VX] = (float)(vx + dvx);
    B[ORC_IDX_OMEGA] = (float)(omega + domega);
}

void orc_ll_step(float *row, int env, int action, float *reward, float *done, float *contacts_out,
                 int *n_contacts_out) {
    double m_power = 0.0, s_power = 0.0, direction = 0.0;
    if (action == 2) m_power = 1.0;
    else if (action == 1) { s_power = 1.0; direction = -1.0; }
    else if (action == 3) { s_power = 1.0; direction = 1.0; }
    step_powers(row, env, m_power, s_power, direction, reward, done, contacts_out, n_contacts_out);
}

/* step_continuous_vec, lunar_lander_v2.mojo:1329-1383: a0 in [-1, 1] -> throttle (a0 + 1) / 2
 * clipped to [0, 1]; a1 clipped to [-1, 1], the side engine fires beyond +-0.5 with power
 * (|a1| - 0.5) * 2 */
void orc_ll_step_continuous(float *row, int env, float a0, float a1, float *reward, float *done,
                            float *contacts_out, int *n_contacts_out) {
    double m_power = ((double)a0 + 1.0) * 0.5;
    if (m_power < 0.0) m_power = 0.0;
    if (m_power > 1.0) m_power = 1.0;
    double side_action = (double)a1, s_power = 0.0, direction = 0.0;
    if (side_action < -1.0) side_action = -1.0;
    if (side_action > 1.0) side_action = 1.0;
    if (side_action < -0.5) { direction = -1.0; s_power = (-side_action - 0.5) * 2.0; }
    else if (side_action > 0.5) { direction = 1.0; s_power = (side_action - 0.5) * 2.0; }
    step_powers(row, env, m_power, s_power, direction, reward, done, contacts_out, n_contacts_out);
}

static void step_powers(float *row, int env, double m_power, double s_power, double direction, float *reward,
                        float *done, float *contacts_out, int *n_contacts_out) {
    orc_layout L; orc_ll_layout(&L);
    float shapes[60]; orc_ll_shapes(shapes);
    float contacts[8 * ORC_CONTACT_SIZE];
    memset(contacts, 0, sizeof(contacts));

    if (row[L.meta_off + META_DONE] > 0.5f) { /* finished rows are frozen until reset */
        *reward = 0.0f; *done = 1.0f;
        if (n_contacts_out) *n_contacts_out = 0;
        return;
    }

    int step_count = (int)row[L.meta_off + META_STEP];

    apply_wind(&L, row, step_count);
    apply_engines(&L, row, env, step_count, m_power, s_power, direction);

    const float gx = (float)0.0, gy = (float)-10.0, dt = (float)DT;
    const float friction = (float)0.1, restitution = (float)0.0;
    const float baumgarte = (float)0.2, slop = (float)0.005;
    orc_integrate_velocities(&L, row, gx, gy, dt);
    int n = orc_edge_detect(&L, row, shapes, contacts);
    for (int it = 0; it < 6; ++it) {
        orc_contact_solve_velocity(&L, row, contacts, n, friction, restitution);
        orc_joint_solve_velocity(&L, row, dt);
    }
    orc_integrate_positions(&L, row, dt);
    for (int it = 0; it < 2; ++it) {
        orc_contact_solve_position(&L, row, contacts, n, baumgarte, slop);
        orc_joint_solve_position(&L, row, baumgarte, slop);
    }
    for (int k = 0; k < 9; ++k) row[L.forces_off + k] = 0.0f;

    /* _compute_step_result */
    step_count += 1;
    float obs[8];
    observe(&L, row, obs);
    const float *B = row + L.bodies_off;
    double vx = B[ORC_IDX_VX], vy = B[ORC_IDX_VY], omega = B[ORC_IDX_OMEGA];
    float new_shaping = shaping(obs);
    float r = new_shaping - row[L.meta_off + META_PREV_SHAPING];
    r = r - (float)(m_power * 0.30);
    r = r - (float)(s_power * 0.03);
    int terminated = 0;
    if (obs[0] >= 1.0f || obs[0] <= -1.0f) { terminated = 1; r = -100.0f; }
    int both_legs = obs[6] > 0.5f && obs[7] > 0.5f;
    double speed = sqrt(vx * vx + vy * vy);
    int lander_contact = 0;
    for (int c = 0; c < n; ++c)
        if ((int)contacts[c * ORC_CONTACT_SIZE + ORC_C_BODY_A] == 0) { lander_contact = 1; break; }
    if (lander_contact) { terminated = 1; r = -100.0f; }
    if (speed < 0.01 && fabs(omega) < 0.01 && both_legs) { terminated = 1; r = r + 100.0f; }
    if (step_count >= 1000) terminated = 1;

    memcpy(row, obs, sizeof(obs));
    row[L.meta_off + META_STEP] = (float)step_count;
    row[L.meta_off + META_PREV_SHAPING] = new_shaping;
    row[L.meta_off + META_DONE] = terminated ? 1.0f : 0.0f;
    *reward = r;
    *done = terminated ? 1.0f : 0.0f;
    if (contacts_out) memcpy(contacts_out, contacts, sizeof(contacts));
    if (n_contacts_out) *n_contacts_out = n;
}

void orc_ll_reset_batch(float *states, int batch, uint64_t seed) {
    for (int i = 0; i < batch; ++i) orc_ll_reset(states + (long)i * ORC_LL_STATE, orc_ll_combined_seed(seed, i));
}

void orc_ll_selective_reset_batch(float *states, const float *dones, int batch, uint64_t seed) {
    for (int i = 0; i < batch; ++i)
        if (dones[i] > 0.5f) orc_ll_reset(states + (long)i * ORC_LL_STATE, orc_ll_combined_seed(seed, i));
}

void orc_ll_step_continuous_batch(float *states, const float *actions, float *rewards, float *dones,
                                  float *obs, int batch) {
    /* rows are independent; the thread count is the OpenMP default (OMP_NUM_THREADS) */
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int i = 0; i < batch; ++i) {
        float *row = states + (long)i * ORC_LL_STATE;
        orc_ll_step_continuous(row, i, actions[2 * i], actions[2 * i + 1], rewards + i, dones + i, 0, 0);
        memcpy(obs + (long)i * 8, row, sizeof(float) * 8);
    }
}

void orc_ll_step_batch(float *states, const float *actions, float *rewards, float *dones,
                       float *obs, int batch, int n_threads) {
    (void)n_threads;
#ifdef _OPENMP
#pragma omp parallel for num_threads(n_threads > 0 ? n_threads : 1) schedule(static)
#endif
    for (int i = 0; i < batch; ++i) {
        float *row = states + (long)i * ORC_LL_STATE;
        orc_ll_step(row, i, (int)actions[i], rewards + i, dones + i, 0, 0);
        memcpy(obs + (long)i * 8, row, sizeof(float) * 8);
    }
}
