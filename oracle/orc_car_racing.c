/*
 * CarRacingV2: CPU restatement (test infrastructure, never shipped).
 *
 * Row layout (physics2d/car/layout.mojo:42-110, envs/car_racing/constants.mojo:95-130), 3040 floats:
 *   [obs 13 | hull 6 (x, y, angle, vx, vy, omega) | wheels 4 x 3 (omega, joint angle, phase) |
 *    controls 3 (steering, gas, brake) | metadata 6 (step_count, total_reward, done, truncated,
 *    tiles_visited, num_tiles) | track 300 x 9 (four vertices, friction) | visited 300]
 *
 * Step: the CPU env's step (envs/car_racing/car_racing_v2.mojo:258-287) on the GPU trait's
 * row (track tiles and visited flags embedded in the row, tile count in the metadata):
 *   action decoding in Float64                       car_racing_v2.mojo:262-268
 *   CarDynamics.step_with_obs                        physics2d/car/car_dynamics.mojo (update_steering,
 *                                                    step_single_env, integrate_hull, update_observation)
 *   WheelFriction.compute_wheel_forces / _all_       physics2d/car/wheel_friction.mojo
 *   TileCollision.point_in_quad / get_friction_at /
 *   check_tile_visited                               physics2d/car/tile_collision.mojo
 *   reward -0.1 (+ 100 / track_length for a new tile), Float64       car_racing_v2.mojo:781-809
 *   termination: playfield, lap fraction, step limit                  car_racing_v2.mojo:811-846
 * From the GPU trait's protocol: a row whose done flag is set returns (0, done) untouched, and a
 * tile count <= 0 is read as 100 (car_racing_v2.mojo:1564-1581).
 * (The reference's GPU step computes another reward, 0.5 * forward speed - 0.01 + tile reward, in
 * fp32: car_racing_v2.mojo:1636-1666.  The CPU statement is the default; orc_cr_set_step_form(1)
 * selects the trait's.)
 *
 * Reset: the GPU trait's _reset_env_gpu / _generate_random_track_gpu (car_racing_v2.mojo:1155-1485),
 * the only code of the reference that fills the embedded-track row (the CPU env builds its track with
 * another, Float64 generator into a separate structure).  All fp32, Philox(seed, 0) successive draws.
 */
#include <math.h>
#include <string.h>
#include "orc.h"

#define CR_STATE 3040
#define CR_OBS 13
#define CR_HULL 13
#define CR_WHEELS 19
#define CR_CTRL 31
#define CR_META 34
#define CR_TRACK 40
#define CR_VISITED 2740
#define CR_MAX_TILES 300
#define CR_TILE 9
enum { H_X, H_Y, H_ANGLE, H_VX, H_VY, H_OMEGA };
enum { W_OMEGA, W_JOINT, W_PHASE, W_SIZE };
enum { M_STEP, M_TOTAL, M_DONE, M_TRUNC, M_VISITED, M_NUM_TILES };

static const double SIZE_ = 0.02, SCALE_ = 6.0, PI_ = 3.14159265358979323846;

static inline float f32_sin(float x) { return (float)sin((double)x); }
static inline float f32_cos(float x) { return (float)cos((double)x); }

/* TileCollision.point_in_quad, tile_collision.mojo:52-90 */
static int point_in_quad(float px, float py, const float *t) {
    float v0x = t[0], v0y = t[1], v1x = t[2], v1y = t[3], v2x = t[4], v2y = t[5], v3x = t[6], v3y = t[7];
    float c0 = (v1x - v0x) * (py - v0y) - (v1y - v0y) * (px - v0x);
    float c1 = (v2x - v1x) * (py - v1y) - (v2y - v1y) * (px - v1x);
    float c2 = (v3x - v2x) * (py - v2y) - (v3y - v2y) * (px - v2x);
    float c3 = (v0x - v3x) * (py - v3y) - (v0y - v3y) * (px - v3x);
    int all_positive = c0 >= 0.0f && c1 >= 0.0f && c2 >= 0.0f && c3 >= 0.0f;
    int all_negative = c0 <= 0.0f && c1 <= 0.0f && c2 <= 0.0f && c3 <= 0.0f;
    return all_positive || all_negative;
}

/* first tile that holds the point, -1 if none (check_tile_visited, tile_collision.mojo:232-262) */
int orc_cr_tile_at(const float *row, float x, float y, int num_tiles) {
    for (int i = 0; i < num_tiles; ++i)
        if (point_in_quad(x, y, row + CR_TRACK + i * CR_TILE)) return i;
    return -1;
}

static float friction_limit_at(const float *row, float x, float y, int num_tiles) {
    int i = orc_cr_tile_at(row, x, y, num_tiles);
    float surface = i >= 0 ? row[CR_TRACK + i * CR_TILE + 8] : (float)0.6;
    return (float)(1000000.0 * SIZE_ * SIZE_) * surface;
}

/* CarDynamics._update_steering_angle, car_dynamics.mojo:118-150 */
static float update_steering_angle(float current, float target, float dt) {
    float diff = target - current;
    float gain = (float)50.0, max_speed = (float)3.0;
    float speed = diff * gain;
    if (speed > max_speed) speed = max_speed;
    else if (speed < -max_speed) speed = -max_speed;
    float new_angle = current + speed * dt;
    float limit = (float)0.4;
    if (new_angle > limit) new_angle = limit;
    else if (new_angle < -limit) new_angle = -limit;
    return new_angle;
}

/* WheelFriction.compute_wheel_forces, wheel_friction.mojo:100-215 */
static void wheel_forces(float wheel_omega, float joint_angle, float hull_angle, float hull_vx, float hull_vy,
                         float hull_omega, float lx, float ly, float gas, float brake, int is_rear,
                         float friction_limit, float dt, float *fx_o, float *fy_o, float *tq_o, float *omega_o) {
    float omega = wheel_omega;
    const float wheel_rad = (float)(27.0 * SIZE_), moment = (float)(4000.0 * SIZE_ * SIZE_);
    const float engine_power = (float)(100000000.0 * SIZE_ * SIZE_), brake_force = (float)15.0;
    const float friction_coef = (float)(205000.0 * SIZE_ * SIZE_);
    const float zero = 0.0f, one = 1.0f;
    if (is_rear && gas > zero) {
        float omega_abs = omega >= zero ? omega : -omega;
        float denom = moment * (omega_abs + (float)5.0);
        omega = omega + (dt * engine_power * gas) / denom;
    }
    if (brake >= (float)0.9) {
        omega = zero;
    } else if (brake > zero) {
        float dir = omega > zero ? -one : one;
        float val = brake_force * brake;
        float omega_abs = omega >= zero ? omega : -omega;
        if (val > omega_abs) val = omega_abs;
        omega = omega + dir * val;
    }
    float cos_hull = f32_cos(hull_angle), sin_hull = f32_sin(hull_angle);
    float wheel_world_x = lx * cos_hull - ly * sin_hull;
    float wheel_world_y = lx * sin_hull + ly * cos_hull;
    float vx_wheel = hull_vx - hull_omega * wheel_world_y;
    float vy_wheel = hull_vy + hull_omega * wheel_world_x;
    float wheel_angle = hull_angle + joint_angle;
    float cos_wheel = f32_cos(wheel_angle), sin_wheel = f32_sin(wheel_angle);
    float forw_x = -sin_wheel, forw_y = cos_wheel, side_x = cos_wheel, side_y = sin_wheel;
    float vf = forw_x * vx_wheel + forw_y * vy_wheel;
    float vs = side_x * vx_wheel + side_y * vy_wheel;
    float vr = omega * wheel_rad;
    float f_force = (-vf + vr) * friction_coef;
    float p_force = -vs * friction_coef;
    float force_sq = f_force * f_force + p_force * p_force;
    if (force_sq < zero) force_sq = zero;
    float force_mag = sqrtf(force_sq);
    if (force_mag > friction_limit && force_mag > (float)1e-8) {
        float scale = friction_limit / force_mag;
        f_force = f_force * scale;
        p_force = p_force * scale;
    }
    if (f_force != f_force) f_force = zero;
    if (p_force != p_force) p_force = zero;
    if (moment > (float)1e-8) omega = omega - dt * f_force * wheel_rad / moment;
    const float max_wheel_omega = (float)200.0;
    if (omega > max_wheel_omega) omega = max_wheel_omega;
    else if (omega < -max_wheel_omega) omega = -max_wheel_omega;
    if (omega != omega) omega = zero;
    float fx = p_force * side_x + f_force * forw_x;
    float fy = p_force * side_y + f_force * forw_y;
    *fx_o = fx; *fy_o = fy;
    *tq_o = wheel_world_x * fy - wheel_world_y * fx;
    *omega_o = omega;
}

static const double WHEEL_LX[4] = {-55.0, 55.0, -55.0, 55.0}, WHEEL_LY[4] = {80.0, 80.0, -82.0, -82.0};

/* CarDynamics.update_observation, car_dynamics.mojo:292-350 */
static void update_observation(float *row) {
    const float *Hl = row + CR_HULL;
    for (int k = 0; k < 6; ++k) row[k] = Hl[k];
    row[6] = row[CR_WHEELS + 0 * W_SIZE + W_JOINT];
    row[7] = row[CR_WHEELS + 1 * W_SIZE + W_JOINT];
    for (int w = 0; w < 4; ++w) row[8 + w] = row[CR_WHEELS + w * W_SIZE + W_OMEGA];
    float vx = Hl[H_VX], vy = Hl[H_VY];
    float speed_sq = vx * vx + vy * vy;
    if (speed_sq < 0.0f) speed_sq = 0.0f;
    float speed = sqrtf(speed_sq);
    if (speed != speed) speed = 0.0f;
    row[12] = speed;
}

/* CarDynamics.step_with_obs, car_dynamics.mojo:226-420 */
static void physics_step(float *row, int num_tiles, float dt) {
    float *Hl = row + CR_HULL, *Wh = row + CR_WHEELS, *C = row + CR_CTRL;
    /* update_steering */
    float target_angle = C[0] * (float)0.4;
    Wh[0 * W_SIZE + W_JOINT] = update_steering_angle(Wh[0 * W_SIZE + W_JOINT], target_angle, dt);
    Wh[1 * W_SIZE + W_JOINT] = update_steering_angle(Wh[1 * W_SIZE + W_JOINT], target_angle, dt);
    /* friction limits under the four wheels (get_wheel_friction_limits, tile_collision.mojo:160-230) */
    float hull_x = Hl[H_X], hull_y = Hl[H_Y], hull_angle = Hl[H_ANGLE];
    float cos_a = f32_cos(hull_angle), sin_a = f32_sin(hull_angle);
    float limits[4];
    for (int w = 0; w < 4; ++w) {
        float lx = (float)(WHEEL_LX[w] * SIZE_), ly = (float)(WHEEL_LY[w] * SIZE_);
        float wx = hull_x + lx * cos_a - ly * sin_a;
        float wy = hull_y + lx * sin_a + ly * cos_a;
        limits[w] = friction_limit_at(row, wx, wy, num_tiles);
    }
    /* compute_all_wheels_forces, wheel_friction.mojo:218-300 */
    float total_fx = 0.0f, total_fy = 0.0f, total_torque = 0.0f;
    float hull_vx = Hl[H_VX], hull_vy = Hl[H_VY], hull_omega = Hl[H_OMEGA];
    float steering = C[0], gas = C[1], brake = C[2];
    for (int w = 0; w < 4; ++w) {
        float lx = (float)(WHEEL_LX[w] * SIZE_), ly = (float)(WHEEL_LY[w] * SIZE_);
        int is_front = w < 2, is_rear = w >= 2;
        float steer_angle = is_front ? steering : 0.0f;   /* the steering INPUT, as the reference passes it */
        float fx, fy, tq, om;
        wheel_forces(Wh[w * W_SIZE + W_OMEGA], steer_angle, hull_angle, hull_vx, hull_vy, hull_omega, lx, ly, gas,
                     brake, is_rear, limits[w], dt, &fx, &fy, &tq, &om);
        total_fx = total_fx + fx;
        total_fy = total_fy + fy;
        total_torque = total_torque + tq;
        Wh[w * W_SIZE + W_OMEGA] = om;
        Wh[w * W_SIZE + W_PHASE] = Wh[w * W_SIZE + W_PHASE] + om * dt;
    }
    /* integrate_hull, car_dynamics.mojo:152-224 */
    float x = Hl[H_X], y = Hl[H_Y], angle = Hl[H_ANGLE], vx = Hl[H_VX], vy = Hl[H_VY], omega = Hl[H_OMEGA];
    const float inv_mass = (float)(1.0 / 10.0), inv_inertia = (float)(1.0 / 10.0);
    vx = vx + total_fx * inv_mass * dt;
    vy = vy + total_fy * inv_mass * dt;
    omega = omega + total_torque * inv_inertia * dt;
    const float max_vel = (float)500.0, max_omega = (float)50.0;
    if (vx > max_vel) vx = max_vel; else if (vx < -max_vel) vx = -max_vel;
    if (vy > max_vel) vy = max_vel; else if (vy < -max_vel) vy = -max_vel;
    if (omega > max_omega) omega = max_omega; else if (omega < -max_omega) omega = -max_omega;
    if (vx != vx) vx = 0.0f;
    if (vy != vy) vy = 0.0f;
    if (omega != omega) omega = 0.0f;
    x = x + vx * dt;
    y = y + vy * dt;
    angle = angle + omega * dt;
    if (x != x) x = 0.0f;
    if (y != y) y = 0.0f;
    if (angle != angle) angle = 0.0f;
    const float pi_val = (float)PI_, two_pi = (float)(2.0 * PI_);
    if (angle > (float)100.0 || angle < (float)-100.0) {
        angle = 0.0f;
    } else if (angle > pi_val) {
        angle = angle - two_pi;
        if (angle > pi_val) angle = angle - two_pi;
    } else if (angle < -pi_val) {
        angle = angle + two_pi;
        if (angle < -pi_val) angle = angle + two_pi;
    }
    Hl[H_X] = x; Hl[H_Y] = y; Hl[H_ANGLE] = angle; Hl[H_VX] = vx; Hl[H_VY] = vy; Hl[H_OMEGA] = omega;
    update_observation(row);
}

/* 0: the CPU env's step (car_racing_v2.mojo:258-287, the default); 1: the GPU trait's step_kernel_gpu
 * (car_racing_v2.mojo:1556-1716): same dynamics, reward 0.5 * forward speed - 0.01 (+ 100 / tiles for a new
 * tile) in fp32 from the hull state after the physics, fp32 playfield and lap tests, the episode total taken
 * after the playfield penalty, and the observation left as the dynamics wrote it. */
static int cr_step_form = 0;
void orc_cr_set_step_form(int form) { cr_step_form = form; }

void orc_cr_step(float *row, const float *action, float *reward, float *done) {
    float *M = row + CR_META;
    if (M[M_DONE] > 0.5f) { *reward = 0.0f; *done = 1.0f; return; }
    int num_tiles = (int)M[M_NUM_TILES];
    if (num_tiles <= 0) num_tiles = 100;
    /* car_racing_v2.mojo:262-268: Float64 clamp and remap, stored as fp32 controls.  (The trait's fp32
     * decoding, :1583-1603, gives the same controls: the halving is exact, so both round a + 1 once.) */
    double steering = (double)action[0];
    steering = steering < -1.0 ? -1.0 : (steering > 1.0 ? 1.0 : steering);
    double gas = ((double)action[1] + 1.0) * 0.5;
    gas = gas < 0.0 ? 0.0 : (gas > 1.0 ? 1.0 : gas);
    double brake = ((double)action[2] + 1.0) * 0.5;
    brake = brake < 0.0 ? 0.0 : (brake > 1.0 ? 1.0 : brake);
    row[CR_CTRL + 0] = (float)steering; row[CR_CTRL + 1] = (float)gas; row[CR_CTRL + 2] = (float)brake;
    physics_step(row, num_tiles, (float)0.02);
    float hull_x = row[CR_HULL + H_X], hull_y = row[CR_HULL + H_Y];
    if (cr_step_form == 1) {
        /* step_kernel_gpu, :1622-1710 */
        float hull_vx = row[CR_HULL + H_VX], hull_vy = row[CR_HULL + H_VY], hull_angle = row[CR_HULL + H_ANGLE];
        float cos_angle = f32_cos(hull_angle), sin_angle = f32_sin(hull_angle);
        float forward_vel = hull_vx * cos_angle + hull_vy * sin_angle;
        float step_reward = forward_vel * (float)0.5 - (float)0.01;
        int tile_idx = orc_cr_tile_at(row, hull_x, hull_y, num_tiles);
        float tiles_visited = M[M_VISITED];
        if (tile_idx >= 0 && !(row[CR_VISITED + tile_idx] > 0.5f)) {
            row[CR_VISITED + tile_idx] = 1.0f;
            float tile_reward = (float)100.0 / (float)num_tiles;
            step_reward = step_reward + tile_reward;
            tiles_visited = tiles_visited + 1.0f;
            M[M_VISITED] = tiles_visited;
        }
        float is_done = 0.0f;
        const float playfield = (float)(2000.0 / SCALE_);
        float abs_x = hull_x >= 0.0f ? hull_x : -hull_x, abs_y = hull_y >= 0.0f ? hull_y : -hull_y;
        if (abs_x > playfield || abs_y > playfield) { is_done = 1.0f; step_reward = (float)-100.0; }
        float num_tiles_f = (float)(num_tiles > 1 ? num_tiles : 1);
        float progress = tiles_visited / num_tiles_f;
        if (progress >= (float)0.95) is_done = 1.0f;
        float step_count = M[M_STEP] + 1.0f;
        M[M_STEP] = step_count;
        if (step_count >= (float)500.0) { is_done = 1.0f; M[M_TRUNC] = 1.0f; }
        M[M_TOTAL] = M[M_TOTAL] + step_reward;
        M[M_DONE] = is_done;
        *reward = step_reward;
        *done = is_done;
        return;
    }
    /* _check_tiles_and_reward, :781-809 */
    int tile_idx = orc_cr_tile_at(row, hull_x, hull_y, num_tiles);
    double step_reward = -0.1;
    float tiles_visited = M[M_VISITED];
    if (tile_idx >= 0 && !(row[CR_VISITED + tile_idx] > 0.5f)) {
        row[CR_VISITED + tile_idx] = 1.0f;
        tiles_visited = tiles_visited + 1.0f;
        M[M_VISITED] = tiles_visited;
        step_reward += 100.0 / (double)num_tiles;
    }
    M[M_TOTAL] = (float)((double)M[M_TOTAL] + step_reward);
    float step_count = M[M_STEP] + 1.0f;
    M[M_STEP] = step_count;
    /* _check_termination, :811-846 */
    int is_done = 0;
    const double playfield = 2000.0 / SCALE_;
    double hx = (double)hull_x, hy = (double)hull_y;
    double abs_x = hx >= 0.0 ? hx : -hx, abs_y = hy >= 0.0 ? hy : -hy;
    if (abs_x > playfield || abs_y > playfield) { is_done = 1; step_reward = -100.0; }
    double progress = (double)tiles_visited / (double)(num_tiles > 1 ? num_tiles : 1);
    if (progress >= 0.95) is_done = 1;
    if (step_count >= (float)500.0) { is_done = 1; M[M_TRUNC] = 1.0f; }
    /* _update_observation, :848-898 (same copies; the speed without the guards) */
    update_observation(row);
    {
        float vx = row[CR_HULL + H_VX], vy = row[CR_HULL + H_VY];
        row[12] = sqrtf(vx * vx + vy * vy);
    }
    M[M_DONE] = is_done ? 1.0f : 0.0f;
    *reward = (float)step_reward;
    *done = is_done ? 1.0f : 0.0f;
}

/* the arctangent stand-in of the track generator (car_racing_v2.mojo:1203-1243, :1389-1430):
 * angle of (dx, dy) from a three-term series of the smaller ratio, clamped to +-0.8 */
static float track_angle(float dx, float dy) {
    const float pi_f = (float)PI_;
    float abs_dx = dx >= 0.0f ? dx : -dx, abs_dy = dy >= 0.0f ? dy : -dy;
    float out;
    if (abs_dx > abs_dy) {
        float t = dy / dx;
        float t2 = t * t, t3 = t2 * t, t5 = t3 * t2;
        float atan_val = t - t3 / (float)3.0 + t5 / (float)5.0;
        if (atan_val > (float)0.8) atan_val = (float)0.8;
        else if (atan_val < (float)-0.8) atan_val = (float)-0.8;
        out = atan_val;
        if (dx < 0.0f) {
            if (dy >= 0.0f) out = out + pi_f;
            else out = out - pi_f;
        }
    } else {
        float t = dx / dy;
        float t2 = t * t, t3 = t2 * t, t5 = t3 * t2;
        float atan_val = t - t3 / (float)3.0 + t5 / (float)5.0;
        if (atan_val > (float)0.8) atan_val = (float)0.8;
        else if (atan_val < (float)-0.8) atan_val = (float)-0.8;
        out = (float)(PI_ / 2.0) - atan_val;
        if (dy < 0.0f) out = -out;
    }
    return out;
}

/* _generate_random_track_gpu, car_racing_v2.mojo:1302-1485 */
static int generate_track(float *row, uint64_t seed) {
    const float track_rad = (float)(900.0 / SCALE_), track_width = (float)(40.0 / SCALE_);
    const float detail_step = (float)(21.0 / SCALE_), turn_rate = (float)0.31;
    const float two_pi = (float)(2.0 * PI_), pi_f = (float)PI_;
    const int num_checkpoints = 12;
    float cx[12], cy[12];
    for (int c = 0; c < num_checkpoints; ++c) {
        float rv[4];
        orc_philox_uniform4(seed, 0, (uint64_t)c, rv);
        float noise = (rv[0] - (float)0.5) * two_pi / (float)num_checkpoints * (float)0.5;
        float alpha = two_pi * (float)c / (float)num_checkpoints + noise;
        float rad = track_rad * ((float)0.5 + rv[1] * (float)0.5);
        if (c == 0) { alpha = 0.0f; rad = track_rad; }
        cx[c] = rad * f32_cos(alpha);
        cy[c] = rad * f32_sin(alpha);
    }
    float x = cx[0], y = cy[0];
    float beta = (float)(PI_ / 2.0);
    int num_tiles = 0, dest_i = 1;
    float prev_x = x, prev_y = y;
    for (int it = 0; it < 500; ++it) {
        if (num_tiles >= CR_MAX_TILES - 1) break;
        float dest_x = cx[dest_i % num_checkpoints], dest_y = cy[dest_i % num_checkpoints];
        float dx = dest_x - x, dy = dest_y - y;
        float dist = sqrtf(dx * dx + dy * dy);
        float angle_to_dest = 0.0f;
        if (dist > (float)0.001) angle_to_dest = track_angle(dx, dy);
        float angle_diff = angle_to_dest - beta;
        while (angle_diff > pi_f) angle_diff = angle_diff - two_pi;
        while (angle_diff < -pi_f) angle_diff = angle_diff + two_pi;
        float steer = turn_rate;
        if (angle_diff < 0.0f) steer = -turn_rate;
        if (angle_diff > (float)-0.1 && angle_diff < (float)0.1) steer = angle_diff;
        beta = beta + steer;
        x = x + detail_step * f32_cos(beta);
        y = y + detail_step * f32_sin(beta);
        if (dist < track_rad * (float)0.3) dest_i += 1;
        float perp_x = -f32_sin(beta) * track_width / (float)2.0;
        float perp_y = f32_cos(beta) * track_width / (float)2.0;
        float *t = row + CR_TRACK + num_tiles * CR_TILE;
        t[0] = prev_x - perp_x; t[1] = prev_y - perp_y;
        t[2] = x - perp_x;      t[3] = y - perp_y;
        t[4] = x + perp_x;      t[5] = y + perp_y;
        t[6] = prev_x + perp_x; t[7] = prev_y + perp_y;
        t[8] = 1.0f;
        num_tiles += 1;
        prev_x = x; prev_y = y;
        if (dest_i >= num_checkpoints + 1) break;
    }
    return num_tiles;
}

/* _reset_env_gpu, car_racing_v2.mojo:1155-1300 */
void orc_cr_reset(float *row, uint64_t combined_seed) {
    memset(row, 0, sizeof(float) * CR_STATE);
    int num_tiles = generate_track(row, combined_seed);
    row[CR_META + M_NUM_TILES] = (float)num_tiles;
    const float *t0 = row + CR_TRACK;
    float start_x = (t0[0] + t0[6]) / (float)2.0;
    float start_y = (t0[1] + t0[7]) / (float)2.0;
    float dx = t0[2] - t0[0], dy = t0[3] - t0[1];
    float start_angle = 0.0f;
    float dist_sq = dx * dx + dy * dy;
    if (dist_sq > (float)0.0001) start_angle = track_angle(dx, dy);
    row[CR_HULL + H_X] = start_x; row[CR_HULL + H_Y] = start_y; row[CR_HULL + H_ANGLE] = start_angle;
    row[0] = start_x; row[1] = start_y; row[2] = start_angle;
}

/* reset_wrapper / selective_reset_wrapper, car_racing_v2.mojo:1062-1150: the seed goes through fp32 */
uint64_t orc_cr_combined_seed(uint64_t seed, int env) {
    int64_t s = (int64_t)(float)seed;
    return (uint64_t)s * 2654435761ull + (uint64_t)((int64_t)env * 12345);
}

void orc_cr_reset_batch(float *states, float *dones, int batch, uint64_t seed) {
#pragma omp parallel for schedule(dynamic, 8)
    for (int i = 0; i < batch; ++i) {
        if (dones != NULL) {
            if (!(dones[i] > 0.5f)) continue;
            dones[i] = 0.0f;
        }
        orc_cr_reset(states + (long)i * CR_STATE, orc_cr_combined_seed(seed, i));
    }
}

void orc_cr_step_batch(float *states, const float *actions, float *rewards, float *dones, float *obs, int batch,
                       int n_threads) {
#pragma omp parallel for schedule(static) num_threads(n_threads > 0 ? n_threads : 1)
    for (int i = 0; i < batch; ++i) {
        orc_cr_step(states + (long)i * CR_STATE, actions + (long)i * 3, rewards + i, dones + i);
        memcpy(obs + (long)i * CR_OBS, states + (long)i * CR_STATE, sizeof(float) * CR_OBS);
    }
}
