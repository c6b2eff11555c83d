/*
 * HopperPlanar and Walker2dPlanar: CPU restatement (test infrastructure, never shipped).
 *
 * The reference's two planar MuJoCo-style envs are Float64 CPU structs with a simplified physics of their
 * own (no constraint solver): joint velocities take the torque, joint angles are clamped to their limits,
 * the torso falls under gravity, the leg segments are placed by forward kinematics and a foot below the
 * ground pushes the torso up.
 *   envs/mujoco_planar/hopper_planar.mojo:162-614   HopperPlanar    (4 bodies, 3 joints, obs 11, action 3)
 *   envs/mujoco_planar/walker_planar.mojo:168-639   Walker2dPlanar  (7 bodies, 6 joints, obs 17, action 6)
 * Every arithmetic step below is Float64 in the reference's order of operations.
 *
 * The reference has no batched (GPU) form of these envs, hence no row layout to follow; the row used
 * here and by the library is:
 *   floats [0, OBS)            the observation, fp32 (get_observation cast to fp32)
 *   float  [OBS]               padding (keeps the doubles 8-byte aligned)
 *   doubles from float OBS + 1 the struct's Float64 state, bit for bit, two floats each:
 *       torso x, y, angle, vx, vy, omega                               6
 *       x, y, angle of every other body, in body order                 3 * (NB - 1)
 *       joint_angles, joint_velocities                                 2 * NJ
 *       step_count, done (0 / 1), total_reward, prev_x                 4
 *   Hopper: 12 + 2 * 25 = 62 floats; Walker2d: 18 + 2 * 40 = 98 floats.
 * (The bodies' masses and inertias enter nothing: the simplified physics never reads them.  vx, vy, omega
 * of the leg bodies are written once, as 0, by _init_body and never again; the one that is
 * read -- the foot's vx in the hopper's ground contact, hopper_planar.mojo:600-602 -- enters as that 0.)
 *
 * Protocol of the batched form (as for the other envs of this library): a row whose done flag is set
 * returns (reward 0, done 1) and is left untouched until it is reset; the reset's six (twelve) draws
 * `random_float64()` (hopper_planar.mojo:318-322) come from Philox(combined seed, 0), one uniform per
 * draw in the order the loop consumes them.
 */
#include <math.h>
#include <string.h>
#include "orc.h"

typedef struct {
    int legs, obs, state;                 /* 1 / 2 legs; observation width; floats per row */
    double torso_len, thigh_len, leg_len, foot_len, foot_radius, init_height;
    double gear, lim[3][2];               /* hip, knee, ankle */
    double min_z, max_z, max_angle;       /* max_z < 0: no upper bound (hopper) */
    double hip_dx[2];                     /* x offset of each leg's hip from the torso */
    int chain_through_centres;            /* hopper: a joint is found from the segment's centre (+ half a length) */
    int foot_friction_term;               /* hopper: torso vx += foot vx * 0.1 at a ground contact */
} planar_model;

static const planar_model HOPPER = {
    1, 11, 62, 0.4, 0.45, 0.5, 0.39, 0.06, 1.25,
    200.0, {{-2.61799, 0.0}, {-2.61799, 0.0}, {-0.785398, 0.785398}},
    0.7, -1.0, 0.2, {0.0, 0.0}, 1, 1};
static const planar_model WALKER = {
    2, 17, 98, 0.4, 0.45, 0.5, 0.2, 0.06, 1.25,
    100.0, {{-1.0, 0.7}, {-1.2, 0.0}, {-0.5, 0.5}},
    0.8, 2.0, 1.0, {0.1, -0.1}, 0, 0};

#define DT 0.008
#define FRAME_SKIP 4
#define GRAVITY (-9.81)

/* views into a row */
typedef struct {
    float *obs;
    double *torso;    /* x, y, angle, vx, vy, omega */
    double *body;     /* (x, y, angle) of bodies 1 .. */
    double *ja, *jv;  /* joint angles, velocities */
    double *meta;     /* step_count, done, total_reward, prev_x */
} planar_row;

static planar_row view(const planar_model *m, float *row) {
    planar_row r;
    const int nj = 3 * m->legs;
    double *d = (double *)(row + m->obs + 1);
    r.obs = row; r.torso = d; r.body = d + 6; r.ja = d + 6 + 3 * nj; r.jv = r.ja + nj; r.meta = r.jv + nj;
    return r;
}

/* get_observation, hopper_planar.mojo:324-375 / walker_planar.mojo:339-403 */
static void observe(const planar_model *m, planar_row r) {
    const int nj = 3 * m->legs;
    r.obs[0] = (float)r.torso[1];
    r.obs[1] = (float)r.torso[2];
    for (int i = 0; i < nj; ++i) r.obs[2 + i] = (float)r.ja[i];
    r.obs[2 + nj] = (float)r.torso[3];
    r.obs[3 + nj] = (float)r.torso[4];
    r.obs[4 + nj] = (float)r.torso[5];
    for (int i = 0; i < nj; ++i) r.obs[5 + nj + i] = (float)r.jv[i];
}

/* _reset_state (hopper_planar.mojo:203-284, walker_planar.mojo:198-303) + the noise of reset() (:311-322) */
static void planar_reset(const planar_model *m, float *row, uint64_t cseed) {
    memset(row, 0, sizeof(float) * m->state);
    planar_row r = view(m, row);
    const double torso_y = m->init_height;
    r.torso[0] = 0.0; r.torso[1] = torso_y;
    const double thigh_y = torso_y - m->torso_len / 2 - m->thigh_len / 2;
    const double leg_y = thigh_y - m->thigh_len / 2 - m->leg_len / 2;
    const double foot_y = leg_y - m->leg_len / 2 - m->foot_len / 2;
    for (int l = 0; l < m->legs; ++l) {
        double *b = r.body + 9 * l;
        b[0] = m->hip_dx[l]; b[1] = thigh_y; b[2] = 0.0;
        b[3] = m->hip_dx[l]; b[4] = leg_y; b[5] = 0.0;
        b[6] = m->hip_dx[l]; b[7] = foot_y; b[8] = 0.0;
    }
    const int nj = 3 * m->legs;
    for (int i = 0; i < nj; ++i) {
        float u[4];
        /* draws 2 i and 2 i + 1 of the stream: lane (n % 4) of block (n / 4) */
        orc_philox_uniform4(cseed, 0, (uint64_t)((2 * i) / 4), u);
        const double ua = (double)u[(2 * i) % 4];
        orc_philox_uniform4(cseed, 0, (uint64_t)((2 * i + 1) / 4), u);
        const double uv = (double)u[(2 * i + 1) % 4];
        r.ja[i] = (ua - 0.5) * 0.01;
        r.jv[i] = (uv - 0.5) * 0.01;
    }
    observe(m, r);
}

/* one leg of _update_body_positions: hopper_planar.mojo:509-575, walker_planar.mojo:536-604 */
static void place_leg(const planar_model *m, planar_row r, int l, double hip_x, double hip_y) {
    double *b = r.body + 9 * l;
    const double *ja = r.ja + 3 * l;
    const double joint_y = hip_y - m->torso_len / 2;
    const double hip_angle = ja[0];
    b[0] = hip_x + sin(hip_angle) * m->thigh_len / 2;
    b[1] = joint_y - cos(hip_angle) * m->thigh_len / 2;
    b[2] = hip_angle;
    double knee_x, knee_y;
    if (m->chain_through_centres) {
        knee_x = b[0] + sin(hip_angle) * m->thigh_len / 2;
        knee_y = b[1] - cos(hip_angle) * m->thigh_len / 2;
    } else {
        knee_x = hip_x + sin(hip_angle) * m->thigh_len;
        knee_y = joint_y - cos(hip_angle) * m->thigh_len;
    }
    const double total_angle = hip_angle + ja[1];
    b[3] = knee_x + sin(total_angle) * m->leg_len / 2;
    b[4] = knee_y - cos(total_angle) * m->leg_len / 2;
    b[5] = total_angle;
    double ankle_x, ankle_y;
    if (m->chain_through_centres) {
        ankle_x = b[3] + sin(total_angle) * m->leg_len / 2;
        ankle_y = b[4] - cos(total_angle) * m->leg_len / 2;
    } else {
        ankle_x = knee_x + sin(total_angle) * m->leg_len;
        ankle_y = knee_y - cos(total_angle) * m->leg_len;
    }
    const double foot_angle = total_angle + ja[2];
    b[6] = ankle_x + sin(foot_angle) * m->foot_len / 2;
    b[7] = ankle_y - cos(foot_angle) * m->foot_len / 2;
    b[8] = foot_angle;
}

/* _physics_step, hopper_planar.mojo:444-507 / walker_planar.mojo:462-534 */
static void physics_step(const planar_model *m, planar_row r, const double *torques) {
    const double dt = DT;
    const int nj = 3 * m->legs;
    for (int i = 0; i < nj; ++i) r.jv[i] += torques[i] * dt * 0.01;
    for (int i = 0; i < nj; ++i) {
        r.ja[i] += r.jv[i] * dt;
        const double low = m->lim[i % 3][0], high = m->lim[i % 3][1];
        if (r.ja[i] < low) { r.ja[i] = low; r.jv[i] = 0.0; }
        else if (r.ja[i] > high) { r.ja[i] = high; r.jv[i] = 0.0; }
    }
    r.torso[4] += GRAVITY * dt;
    /* _update_body_positions */
    double torso_x = r.torso[0], torso_y = r.torso[1];
    torso_x += r.torso[3] * DT;
    torso_y += r.torso[4] * DT;
    r.torso[0] = torso_x; r.torso[1] = torso_y;
    for (int l = 0; l < m->legs; ++l) place_leg(m, r, l, torso_x + m->hip_dx[l], torso_y);
    /* _handle_ground_collision: each foot in turn */
    const double ground_y = 0.0;
    for (int l = 0; l < m->legs; ++l) {
        const double foot_y = r.body[9 * l + 7];
        if (foot_y - m->foot_radius < ground_y) {
            const double penetration = ground_y - (foot_y - m->foot_radius);
            r.torso[1] += penetration;
            if (r.torso[4] < 0) r.torso[4] = 0.0;
            if (m->foot_friction_term) {
                const double foot_vx = 0.0;   /* the foot body's vx slot: 0 since _init_body */
                r.torso[3] += foot_vx * 0.1;
            }
        }
    }
}

/* step, hopper_planar.mojo:377-442 / walker_planar.mojo:405-460 */
static void planar_step(const planar_model *m, float *row, const float *action, float *reward, float *done) {
    planar_row r = view(m, row);
    if (r.meta[1] > 0.5) { *reward = 0.0f; *done = 1.0f; return; }
    const int nj = 3 * m->legs;
    double torques[6];
    for (int i = 0; i < nj; ++i) {
        double a = (double)action[i];
        if (a > 1.0) a = 1.0;
        else if (a < -1.0) a = -1.0;
        torques[i] = a * m->gear;
    }
    const double x_before = r.torso[0];
    for (int k = 0; k < FRAME_SKIP; ++k) physics_step(m, r, torques);
    const double x_after = r.torso[0], torso_y = r.torso[1], torso_angle = r.torso[2];
    const double forward_velocity = (x_after - x_before) / (DT * (double)FRAME_SKIP);
    const double forward_reward = 1.0 * forward_velocity;
    double ctrl_cost = 0.0;
    for (int i = 0; i < nj; ++i) {
        const double ai = (double)action[i];
        const double a = (ai >= -1.0 && ai <= 1.0) ? ai : (ai > 0 ? 1.0 : -1.0);
        ctrl_cost += a * a;
    }
    ctrl_cost *= 0.001;
    int is_healthy = torso_y >= m->min_z && fabs(torso_angle) <= m->max_angle;
    if (m->max_z >= 0.0) is_healthy = is_healthy && torso_y <= m->max_z;
    const double healthy_reward = is_healthy ? 1.0 : 0.0;
    const double rew = forward_reward + healthy_reward - ctrl_cost;
    r.meta[1] = is_healthy ? 0.0 : 1.0;
    r.meta[0] += 1.0;
    r.meta[2] += rew;
    observe(m, r);
    *reward = (float)rew;
    *done = is_healthy ? 0.0f : 1.0f;
}

static uint64_t planar_seed(uint64_t seed, int env) {
    int64_t seed_i = (int64_t)(float)seed;
    return (uint64_t)seed_i * 2654435761ull + (uint64_t)(env + 1) * 12345ull;
}

static const planar_model *model_of(int which) { return which == 0 ? &HOPPER : &WALKER; }

int orc_planar_state_size(int which) { return model_of(which)->state; }
void orc_planar_reset(int which, float *row, uint64_t combined_seed) { planar_reset(model_of(which), row, combined_seed); }
void orc_planar_step(int which, float *row, const float *action, float *reward, float *done) {
    planar_step(model_of(which), row, action, reward, done);
}
void orc_planar_reset_batch(int which, float *states, const float *dones, int batch, uint64_t seed) {
    const planar_model *m = model_of(which);
    for (int i = 0; i < batch; ++i)
        if (!dones || dones[i] > 0.5f) planar_reset(m, states + (long)i * m->state, planar_seed(seed, i));
}
void orc_planar_step_batch(int which, float *states, const float *actions, float *rewards, float *dones, float *obs,
                           int batch, int n_threads) {
    const planar_model *m = model_of(which);
    const int aw = 3 * m->legs;
    (void)n_threads;
#ifdef _OPENMP
#pragma omp parallel for num_threads(n_threads > 0 ? n_threads : 1) schedule(static)
#endif
    for (int i = 0; i < batch; ++i) {
        float *row = states + (long)i * m->state;
        planar_step(m, row, actions + (long)i * aw, rewards + i, dones + i);
        memcpy(obs + (long)i * m->obs, row, sizeof(float) * m->obs);
    }
}
