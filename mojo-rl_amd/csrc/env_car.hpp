// CarRacingV2 (envs/car_racing/car_racing_v2.mojo) on the GPU trait's row: [obs 13 | hull 6 | wheels
// 4 x 3 | controls 3 | metadata 6 | track 300 tiles x 9 | visited 300] = 3040 floats per env
// (physics2d/car/layout.mojo:42-110).
//
// A row is 12 KB, almost all of it the track, and a step looks five points up in the tile list (the
// four wheels before the physics, the hull after it): the tile table is the step's memory traffic.
// A wavefront takes an env: it copies the table (tiles and visited flags, 12 KB, one contiguous range)
// into LDS with 16-byte loads -- every cache line is fetched once; tile by tile, the 36-byte records
// would make each line cross the vector cache nine times -- in one batch of independent loads at the
// start of the step, and lane l keeps the vertices of tiles l, l + 64, .. l + 256 in registers for both
// lookups, so a step waits for memory once.  The first tile in list order that holds a point is the
// minimum over the wavefront of each lane's first hit -- what the reference's scan-until-hit returns;
// friction and visited flag of that tile are read from the LDS copy.  The four
// wheels' forces are computed on four lanes and summed in wheel order; the rest of the (small)
// state update is done by every lane alike, and lane 0 writes the row.
//
// Arithmetic: the reference's CPU step (CarDynamics.step_with_obs in fp32, action decoding, reward and
// termination in Float64, car_racing_v2.mojo:258-287, :781-846) with the GPU trait's row protocol
// (done rows return (0, 1) untouched, tile count from the metadata); reset and track generator are the
// GPU trait's (car_racing_v2.mojo:1155-1485), the only code there that fills this row.
#pragma once
#include "mrl_device.hpp"

namespace mrl {
namespace cr {

constexpr int STATE = 3040, OBS = 13, ACT = 3;
constexpr int HULL = 13, WHEELS = 19, CTRL = 31, META = 34, TRACK = 40, VISITED = 2740;
constexpr int MAX_TILES = 300, TILE = 9;
constexpr int STEP_LANES = 64, SLOTS = 5;   // a wavefront per env; SLOTS * 64 >= MAX_TILES tiles in its registers
enum { H_X, H_Y, H_ANGLE, H_VX, H_VY, H_OMEGA };
enum { W_OMEGA, W_JOINT, W_PHASE, W_SIZE };
enum { M_STEP, M_TOTAL, M_DONE, M_TRUNC, M_VISITED, M_NUM_TILES };
constexpr double SIZE_ = 0.02, SCALE_ = 6.0, PI_ = 3.14159265358979323846;

// TileCollision.point_in_quad, physics2d/car/tile_collision.mojo:52-90
MRL_DEV bool point_in_quad(float px, float py, float v0x, float v0y, float v1x, float v1y, float v2x, float v2y,
                           float v3x, float v3y) {
    const float c0 = (v1x - v0x) * (py - v0y) - (v1y - v0y) * (px - v0x);
    const float c1 = (v2x - v1x) * (py - v1y) - (v2y - v1y) * (px - v1x);
    const float c2 = (v3x - v2x) * (py - v2y) - (v3y - v2y) * (px - v2x);
    const float c3 = (v0x - v3x) * (py - v3y) - (v0y - v3y) * (px - v3x);
    const bool all_positive = c0 >= 0.0f && c1 >= 0.0f && c2 >= 0.0f && c3 >= 0.0f;
    const bool all_negative = c0 <= 0.0f && c1 <= 0.0f && c2 <= 0.0f && c3 <= 0.0f;
    return all_positive || all_negative;
}

// The tile table of one env: a copy in LDS (`lds`, TABLE floats: tiles, then visited flags, as in the
// row) made by the wavefront, and the vertices of tiles sub + 64 * i in the registers of lane `sub`.
constexpr int TABLE = STATE - TRACK;   // 3000 floats, a multiple of 4; row + TRACK is 16-byte aligned
struct Tiles {
    float v[SLOTS][8];     // four vertices
    const float *lds;

    // FLAGS_COHERENT: the visited flags are read past the vector cache, for a kernel that steps the same
    // env again and again and so reads flags that an earlier step of its own launch has written
    template <bool FLAGS_COHERENT = false>
    MRL_DEV void load(const float *row, float *table, int sub) {
        constexpr int N4 = TABLE / 4, ROUNDS = (N4 + STEP_LANES - 1) / STEP_LANES;
        const float4 *src = reinterpret_cast<const float4 *>(row + TRACK);
        float4 *dst = reinterpret_cast<float4 *>(table);
        static_assert(N4 > STEP_LANES * (ROUNDS - 1) && N4 <= STEP_LANES * ROUNDS, "only the last round is partial");
        float4 tmp[ROUNDS];
#pragma unroll
        for (int i = 0; i < ROUNDS - 1; ++i) tmp[i] = src[sub + STEP_LANES * i];
        const int last = sub + STEP_LANES * (ROUNDS - 1);
        tmp[ROUNDS - 1] = src[last < N4 ? last : N4 - 1];
#pragma unroll
        for (int i = 0; i < ROUNDS - 1; ++i) dst[sub + STEP_LANES * i] = tmp[i];
        if (last < N4) dst[last] = tmp[ROUNDS - 1];
        if (FLAGS_COHERENT) {
            constexpr int F0 = MAX_TILES * TILE;
            float f[(MAX_TILES + STEP_LANES - 1) / STEP_LANES];
#pragma unroll
            for (int i = 0; i < (MAX_TILES + STEP_LANES - 1) / STEP_LANES; ++i) {
                const int k = sub + STEP_LANES * i;
                f[i] = __hip_atomic_load(row + VISITED + (k < MAX_TILES ? k : MAX_TILES - 1), __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int i = 0; i < (MAX_TILES + STEP_LANES - 1) / STEP_LANES; ++i) {
                const int k = sub + STEP_LANES * i;
                if (k < MAX_TILES) table[F0 + k] = f[i];
            }
        }
        // the wavefront's own LDS writes, read back by other lanes of the same wavefront
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        lds = table;
        // slots past the table (tiles 300 .. 319) read the visited flags behind it; never used
#pragma unroll
        for (int i = 0; i < SLOTS; ++i) {
            const float *T = table + (sub + STEP_LANES * i) * TILE;
#pragma unroll
            for (int k = 0; k < 8; ++k) v[i][k] = T[k];
        }
    }
    MRL_DEV float friction(int t) const { return lds[t * TILE + 8]; }
    MRL_DEV float visited(int t) const { return lds[MAX_TILES * TILE + t]; }

    // index of the first tile (list order) that holds point p, -1 if none, for NP points at once
    template <int NP>
    MRL_DEV void at(const float (&px)[NP], const float (&py)[NP], int num_tiles, int sub, int (&idx)[NP]) const {
        constexpr int NONE = 1 << 30;
#pragma unroll
        for (int p = 0; p < NP; ++p) idx[p] = NONE;
#pragma unroll
        for (int i = 0; i < SLOTS; ++i) {
            const int t = sub + STEP_LANES * i;
#pragma unroll
            for (int p = 0; p < NP; ++p)
                if (t < num_tiles && idx[p] == NONE &&
                    point_in_quad(px[p], py[p], v[i][0], v[i][1], v[i][2], v[i][3], v[i][4], v[i][5], v[i][6], v[i][7]))
                    idx[p] = t;
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int m = idx[p];
#pragma unroll
            for (int off = STEP_LANES / 2; off > 0; off >>= 1) {
                const int o = __shfl_xor(m, off, 64);
                m = o < m ? o : m;
            }
            idx[p] = m == NONE ? -1 : m;
        }
    }
};

// CarDynamics._update_steering_angle, physics2d/car/car_dynamics.mojo:118-150
MRL_DEV float update_steering_angle(float current, float target, float dt) {
    const float diff = target - current;
    const float gain = (float)50.0, max_speed = (float)3.0;
    float speed = diff * gain;
    if (speed > max_speed) speed = max_speed;
    else if (speed < -max_speed) speed = -max_speed;
    float new_angle = current + speed * dt;
    const float limit = (float)0.4;
    if (new_angle > limit) new_angle = limit;
    else if (new_angle < -limit) new_angle = -limit;
    return new_angle;
}

// WheelFriction.compute_wheel_forces, physics2d/car/wheel_friction.mojo:100-215; cos_hull / sin_hull
// are those of hull_angle
MRL_DEV void wheel_forces(float wheel_omega, float joint_angle, float hull_angle, float cos_hull, float sin_hull,
                          float hull_vx, float hull_vy, float hull_omega, float lx, float ly, float gas, float brake,
                          bool is_rear, float friction_limit, float dt, float &fx_o, float &fy_o, float &tq_o,
                          float &omega_o) {
    float omega = wheel_omega;
    const float wheel_rad = (float)(27.0 * SIZE_), moment = (float)(4000.0 * SIZE_ * SIZE_);
    const float engine_power = (float)(100000000.0 * SIZE_ * SIZE_), brake_force = (float)15.0;
    const float friction_coef = (float)(205000.0 * SIZE_ * SIZE_);
    const float zero = 0.0f, one = 1.0f;
    if (is_rear && gas > zero) {
        const float omega_abs = omega >= zero ? omega : -omega;
        const float denom = moment * (omega_abs + (float)5.0);
        omega = omega + (dt * engine_power * gas) / denom;
    }
    if (brake >= (float)0.9) {
        omega = zero;
    } else if (brake > zero) {
        const float dir = omega > zero ? -one : one;
        float val = brake_force * brake;
        const float omega_abs = omega >= zero ? omega : -omega;
        if (val > omega_abs) val = omega_abs;
        omega = omega + dir * val;
    }
    const float wheel_world_x = lx * cos_hull - ly * sin_hull;
    const float wheel_world_y = lx * sin_hull + ly * cos_hull;
    const float vx_wheel = hull_vx - hull_omega * wheel_world_y;
    const float vy_wheel = hull_vy + hull_omega * wheel_world_x;
    const float wheel_angle = hull_angle + joint_angle;
    float sin_wheel, cos_wheel;
    sincos32(wheel_angle, sin_wheel, cos_wheel);
    const float forw_x = -sin_wheel, forw_y = cos_wheel, side_x = cos_wheel, side_y = sin_wheel;
    const float vf = forw_x * vx_wheel + forw_y * vy_wheel;
    const float vs = side_x * vx_wheel + side_y * vy_wheel;
    const float vr = omega * wheel_rad;
    float f_force = (-vf + vr) * friction_coef;
    float p_force = -vs * friction_coef;
    float force_sq = f_force * f_force + p_force * p_force;
    if (force_sq < zero) force_sq = zero;
    const float force_mag = sqrtf(force_sq);
    if (force_mag > friction_limit && force_mag > (float)1e-8) {
        const float scale = friction_limit / force_mag;
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
    const float fx = p_force * side_x + f_force * forw_x;
    const float fy = p_force * side_y + f_force * forw_y;
    fx_o = fx; fy_o = fy;
    tq_o = wheel_world_x * fy - wheel_world_y * fx;
    omega_o = omega;
}

// One env step by the 64 lanes of a wavefront (sub = lane; table = TABLE floats of LDS of its own).  `head`
// = the row's first TRACK floats (observation, hull, wheels, controls, metadata) wherever the caller keeps
// them: the row itself, or a copy that a kernel holds on chip over many steps; `row` is read for the tile
// table and takes the visited flags.  Every lane returns the same reward / done and the observation the row
// now starts with; lane 0 has written `head`.
// trait_form: false = the CPU env's reward and termination arithmetic (car_racing_v2.mojo:781-846, Float64),
// true = the GPU trait's step_kernel_gpu (car_racing_v2.mojo:1622-1710: reward 0.5 * forward speed - 0.01
// (+ 100 / tiles) in fp32 from the hull state after the physics, fp32 playfield and lap tests, the episode
// total taken after the playfield penalty).  The dynamics and the decoded controls are the same in both.
template <bool FLAGS_COHERENT = false>
MRL_DEV void step_wave(float *head, float *row, float *table, const float *action, int sub, float &reward,
                       float &done, float (&ob)[OBS], bool trait_form = false) {
    float *M = head + META;
    if (M[M_DONE] > 0.5f) {   // car_racing_v2.mojo:1564-1572
#pragma unroll
        for (int k = 0; k < OBS; ++k) ob[k] = head[k];
        reward = 0.0f; done = 1.0f;
        return;
    }
    Tiles tiles;
    tiles.template load<FLAGS_COHERENT>(row, table, sub);
    int num_tiles = (int)M[M_NUM_TILES];
    if (num_tiles <= 0) num_tiles = 100;
    // ---- controls, car_racing_v2.mojo:262-268 (Float64)
    double steering_d = (double)action[0];
    steering_d = steering_d < -1.0 ? -1.0 : (steering_d > 1.0 ? 1.0 : steering_d);
    double gas_d = ((double)action[1] + 1.0) * 0.5;
    gas_d = gas_d < 0.0 ? 0.0 : (gas_d > 1.0 ? 1.0 : gas_d);
    double brake_d = ((double)action[2] + 1.0) * 0.5;
    brake_d = brake_d < 0.0 ? 0.0 : (brake_d > 1.0 ? 1.0 : brake_d);
    const float steering = (float)steering_d, gas = (float)gas_d, brake = (float)brake_d;
    const float dt = (float)0.02;
    // ---- state
    float x = head[HULL + H_X], y = head[HULL + H_Y], angle = head[HULL + H_ANGLE];
    float vx = head[HULL + H_VX], vy = head[HULL + H_VY], omega = head[HULL + H_OMEGA];
    float w_omega[4], w_phase[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) { w_omega[w] = head[WHEELS + w * W_SIZE + W_OMEGA]; w_phase[w] = head[WHEELS + w * W_SIZE + W_PHASE]; }
    // ---- steering joints (update_steering, car_dynamics.mojo:68-116)
    const float target_angle = steering * (float)0.4;
    const float joint_fl = update_steering_angle(head[WHEELS + 0 * W_SIZE + W_JOINT], target_angle, dt);
    const float joint_fr = update_steering_angle(head[WHEELS + 1 * W_SIZE + W_JOINT], target_angle, dt);
    const float joint_rl = head[WHEELS + 2 * W_SIZE + W_JOINT], joint_rr = head[WHEELS + 3 * W_SIZE + W_JOINT];
    // ---- friction limit under each wheel (get_wheel_friction_limits, tile_collision.mojo:160-230)
    float sin_a, cos_a;
    sincos32(angle, sin_a, cos_a);
    const float lxs[4] = {(float)(-55.0 * SIZE_), (float)(55.0 * SIZE_), (float)(-55.0 * SIZE_), (float)(55.0 * SIZE_)};
    const float lys[4] = {(float)(80.0 * SIZE_), (float)(80.0 * SIZE_), (float)(-82.0 * SIZE_), (float)(-82.0 * SIZE_)};
    float wpx[4], wpy[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        wpx[w] = x + lxs[w] * cos_a - lys[w] * sin_a;
        wpy[w] = y + lxs[w] * sin_a + lys[w] * cos_a;
    }
    int under[4];
    tiles.at<4>(wpx, wpy, num_tiles, sub, under);
    // ---- my wheel (sub & 3): compute_wheel_forces
    const int mw = sub & 3;
    float my_limit, my_omega, my_lx, my_ly;
    {
        float lim[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float surface = under[w] >= 0 ? tiles.friction(under[w] >= 0 ? under[w] : 0) : (float)0.6;
            lim[w] = (float)(1000000.0 * SIZE_ * SIZE_) * surface;
        }
        my_limit = mw == 0 ? lim[0] : mw == 1 ? lim[1] : mw == 2 ? lim[2] : lim[3];
        my_omega = mw == 0 ? w_omega[0] : mw == 1 ? w_omega[1] : mw == 2 ? w_omega[2] : w_omega[3];
        my_lx = (mw & 1) ? lxs[1] : lxs[0];
        my_ly = mw < 2 ? lys[0] : lys[2];
    }
    const float steer_angle = mw < 2 ? steering : 0.0f;   // the steering INPUT, as the reference passes it
    float fx, fy, tq, om;
    wheel_forces(my_omega, steer_angle, angle, cos_a, sin_a, vx, vy, omega, my_lx, my_ly, gas, brake, mw >= 2, my_limit,
                 dt, fx, fy, tq, om);
    // ---- totals in wheel order (compute_all_wheels_forces, wheel_friction.mojo:218-300)
    float total_fx = 0.0f, total_fy = 0.0f, total_torque = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        total_fx = total_fx + __shfl(fx, w, 64);
        total_fy = total_fy + __shfl(fy, w, 64);
        total_torque = total_torque + __shfl(tq, w, 64);
        const float nom = __shfl(om, w, 64);
        w_omega[w] = nom;
        w_phase[w] = w_phase[w] + nom * dt;
    }
    // ---- integrate_hull, car_dynamics.mojo:152-224
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
    // ---- tile under the hull, reward (car_racing_v2.mojo:781-809), termination (:811-846)
    const float hpx[1] = {x}, hpy[1] = {y};
    int tile_idx[1];
    tiles.at<1>(hpx, hpy, num_tiles, sub, tile_idx);
    float tiles_visited = M[M_VISITED];
    const bool fresh = tile_idx[0] >= 0 && !(tiles.visited(tile_idx[0] >= 0 ? tile_idx[0] : 0) > 0.5f);
    const float step_count = M[M_STEP] + 1.0f;
    const bool truncated = step_count >= (float)500.0;
    bool is_done = false;
    float total;
    if (trait_form) {
        float sin_h, cos_h;
        sincos32(angle, sin_h, cos_h);
        const float forward_vel = vx * cos_h + vy * sin_h;
        float step_reward = forward_vel * (float)0.5 - (float)0.01;
        if (fresh) {
            const float tile_reward = (float)100.0 / (float)num_tiles;
            step_reward = step_reward + tile_reward;
            tiles_visited = tiles_visited + 1.0f;
        }
        const float playfield = (float)(2000.0 / SCALE_);
        const float abs_x = x >= 0.0f ? x : -x, abs_y = y >= 0.0f ? y : -y;
        if (abs_x > playfield || abs_y > playfield) { is_done = true; step_reward = (float)-100.0; }
        const float progress = tiles_visited / (float)(num_tiles > 1 ? num_tiles : 1);
        if (progress >= (float)0.95) is_done = true;
        total = M[M_TOTAL] + step_reward;
        reward = step_reward;
    } else {
        double step_reward = -0.1;
        if (fresh) {
            tiles_visited = tiles_visited + 1.0f;
            step_reward += 100.0 / (double)num_tiles;
        }
        total = (float)((double)M[M_TOTAL] + step_reward);
        const double playfield = 2000.0 / SCALE_;
        const double hx = (double)x, hy = (double)y;
        const double abs_x = hx >= 0.0 ? hx : -hx, abs_y = hy >= 0.0 ? hy : -hy;
        if (abs_x > playfield || abs_y > playfield) { is_done = true; step_reward = -100.0; }
        const double progress = (double)tiles_visited / (double)(num_tiles > 1 ? num_tiles : 1);
        if (progress >= 0.95) is_done = true;
        reward = (float)step_reward;
    }
    if (truncated) is_done = true;
    done = is_done ? 1.0f : 0.0f;
    // observation (update_observation, car_dynamics.mojo:292-350; _update_observation, :848-898)
    ob[0] = x; ob[1] = y; ob[2] = angle; ob[3] = vx; ob[4] = vy; ob[5] = omega;
    ob[6] = joint_fl; ob[7] = joint_fr;
#pragma unroll
    for (int w = 0; w < 4; ++w) ob[8 + w] = w_omega[w];
    ob[12] = sqrtf(vx * vx + vy * vy);
    // ---- lane 0 writes the row (the reads above are done: every lane holds its values in registers)
    if (sub == 0) {
        head[CTRL + 0] = steering; head[CTRL + 1] = gas; head[CTRL + 2] = brake;
        head[HULL + H_X] = x; head[HULL + H_Y] = y; head[HULL + H_ANGLE] = angle;
        head[HULL + H_VX] = vx; head[HULL + H_VY] = vy; head[HULL + H_OMEGA] = omega;
        const float joints[4] = {joint_fl, joint_fr, joint_rl, joint_rr};
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            head[WHEELS + w * W_SIZE + W_OMEGA] = w_omega[w];
            head[WHEELS + w * W_SIZE + W_JOINT] = joints[w];
            head[WHEELS + w * W_SIZE + W_PHASE] = w_phase[w];
        }
#pragma unroll
        for (int k = 0; k < OBS; ++k) head[k] = ob[k];
        if (fresh) row[VISITED + tile_idx[0]] = 1.0f;
        M[M_VISITED] = tiles_visited;
        M[M_TOTAL] = total;
        M[M_STEP] = step_count;
        if (truncated) M[M_TRUNC] = 1.0f;
        M[M_DONE] = done;
    }
}

// the arctangent stand-in of the track generator (car_racing_v2.mojo:1203-1243, :1389-1430)
MRL_DEV float track_angle(float dx, float dy) {
    const float pi_f = (float)PI_;
    const float abs_dx = dx >= 0.0f ? dx : -dx, abs_dy = dy >= 0.0f ? dy : -dy;
    float out;
    if (abs_dx > abs_dy) {
        const float t = dy / dx;
        const float t2 = t * t, t3 = t2 * t, t5 = t3 * t2;
        float atan_val = t - t3 / (float)3.0 + t5 / (float)5.0;
        if (atan_val > (float)0.8) atan_val = (float)0.8;
        else if (atan_val < (float)-0.8) atan_val = (float)-0.8;
        out = atan_val;
        if (dx < 0.0f) {
            if (dy >= 0.0f) out = out + pi_f;
            else out = out - pi_f;
        }
    } else {
        const float t = dx / dy;
        const float t2 = t * t, t3 = t2 * t, t5 = t3 * t2;
        float atan_val = t - t3 / (float)3.0 + t5 / (float)5.0;
        if (atan_val > (float)0.8) atan_val = (float)0.8;
        else if (atan_val < (float)-0.8) atan_val = (float)-0.8;
        out = (float)(PI_ / 2.0) - atan_val;
        if (dy < 0.0f) out = -out;
    }
    return out;
}

MRL_DEV uint64_t combined_seed(uint64_t seed, int env) {   // car_racing_v2.mojo:1075, :1133 (seed through fp32)
    const int64_t s = (int64_t)(float)seed;
    return (uint64_t)s * 2654435761ull + (uint64_t)((int64_t)env * 12345);
}

// _generate_random_track_gpu, car_racing_v2.mojo:1302-1485, by ONE lane (a serial recurrence)
MRL_DEV int generate_track(float *row, uint64_t seed) {
    const float track_rad = (float)(900.0 / SCALE_), track_width = (float)(40.0 / SCALE_);
    const float detail_step = (float)(21.0 / SCALE_), turn_rate = (float)0.31;
    const float two_pi = (float)(2.0 * PI_), pi_f = (float)PI_;
    constexpr int num_checkpoints = 12;
    float cx[num_checkpoints], cy[num_checkpoints];
#pragma unroll 1
    for (int c = 0; c < num_checkpoints; ++c) {
        const Uniform4 rv = philox_uniform4(seed, 0, (uint64_t)c);
        const float noise = (rv.v[0] - (float)0.5) * two_pi / (float)num_checkpoints * (float)0.5;
        float alpha = two_pi * (float)c / (float)num_checkpoints + noise;
        float rad = track_rad * ((float)0.5 + rv.v[1] * (float)0.5);
        if (c == 0) { alpha = 0.0f; rad = track_rad; }
        float s, co;
        sincos32(alpha, s, co);
        cx[c] = rad * co;
        cy[c] = rad * s;
    }
    float x = cx[0], y = cy[0];
    float beta = (float)(PI_ / 2.0);
    int num_tiles = 0, dest_i = 1;
    float prev_x = x, prev_y = y;
#pragma unroll 1
    for (int it = 0; it < 500; ++it) {
        if (num_tiles >= MAX_TILES - 1) break;
        const int d = dest_i % num_checkpoints;
        float dest_x = cx[0], dest_y = cy[0];
#pragma unroll
        for (int c = 1; c < num_checkpoints; ++c) { dest_x = d == c ? cx[c] : dest_x; dest_y = d == c ? cy[c] : dest_y; }
        const float dx = dest_x - x, dy = dest_y - y;
        const float dist = sqrtf(dx * dx + dy * dy);
        float angle_to_dest = 0.0f;
        if (dist > (float)0.001) angle_to_dest = track_angle(dx, dy);
        float angle_diff = angle_to_dest - beta;
        while (angle_diff > pi_f) angle_diff = angle_diff - two_pi;
        while (angle_diff < -pi_f) angle_diff = angle_diff + two_pi;
        float steer = turn_rate;
        if (angle_diff < 0.0f) steer = -turn_rate;
        if (angle_diff > (float)-0.1 && angle_diff < (float)0.1) steer = angle_diff;
        beta = beta + steer;
        float sb, cb;
        sincos32(beta, sb, cb);
        x = x + detail_step * cb;
        y = y + detail_step * sb;
        if (dist < track_rad * (float)0.3) dest_i += 1;
        const float perp_x = -sb * track_width / (float)2.0;
        const float perp_y = cb * track_width / (float)2.0;
        float *t = row + TRACK + num_tiles * TILE;
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

// _reset_env_gpu, car_racing_v2.mojo:1155-1300, by a group of GROUP lanes of a wavefront: its lane 0
// walks the track (it writes the tiles it makes), then all lanes clear what is left of the row and
// place the car; the observation of the fresh row is (start_x, start_y, start_angle, 0, .. 0); returns the
// number of tiles of the new track
template <int GROUP>
MRL_DEV int reset_group(float *row, uint64_t cseed, int lane, float &start_x, float &start_y, float &start_angle) {
    const int sub = lane & (GROUP - 1), base = lane & ~(GROUP - 1);
    int num_tiles = 0;
    start_x = 0.0f; start_y = 0.0f; start_angle = 0.0f;
    if (sub == 0) {
        num_tiles = generate_track(row, cseed);
        const float *t0 = row + TRACK;
        const float v0x = num_tiles > 0 ? t0[0] : 0.0f, v0y = num_tiles > 0 ? t0[1] : 0.0f;
        const float v1x = num_tiles > 0 ? t0[2] : 0.0f, v1y = num_tiles > 0 ? t0[3] : 0.0f;
        const float v3x = num_tiles > 0 ? t0[6] : 0.0f, v3y = num_tiles > 0 ? t0[7] : 0.0f;
        start_x = (v0x + v3x) / (float)2.0;
        start_y = (v0y + v3y) / (float)2.0;
        const float dx = v1x - v0x, dy = v1y - v0y;
        const float dist_sq = dx * dx + dy * dy;
        if (dist_sq > (float)0.0001) start_angle = track_angle(dx, dy);
    }
    num_tiles = __shfl(num_tiles, base, 64);
    start_x = __shfl(start_x, base, 64);
    start_y = __shfl(start_y, base, 64);
    start_angle = __shfl(start_angle, base, 64);
    // everything but the tiles just made, every float written once: the car at the start of the track,
    // at rest (observation and hull), the tile count, zeros elsewhere
    for (int i = sub; i < STATE; i += GROUP) {
        if (i >= TRACK && i < TRACK + num_tiles * TILE) continue;
        float v = 0.0f;
        if (i == 0 || i == HULL + H_X) v = start_x;
        else if (i == 1 || i == HULL + H_Y) v = start_y;
        else if (i == 2 || i == HULL + H_ANGLE) v = start_angle;
        else if (i == META + M_NUM_TILES) v = (float)num_tiles;
        row[i] = v;
    }
    return num_tiles;
}

}  // namespace cr
}  // namespace mrl
