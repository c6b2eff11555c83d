/*
 * BipedalWalkerV2 and HalfCheetahPlanarV2: CPU restatement (test infrastructure, never shipped).
 *
 * BipedalWalker (row of 950 floats, physics2d/layout.mojo:280-288):
 *   constants / shapes   envs/bipedal_walker/constants_v2.mojo, bipedal_walker_v2.mojo:319-364
 *   reset                bipedal_walker_v2.mojo:366-391 (_reset_cpu), :393-466 (terrain random
 *                        walk in fp32, edges), :468-622 (bodies, joints); seed combination :1444
 *   motors               bipedal_walker_v2.mojo:931-1003
 *   physics step         bipedal_walker_v2.mojo:857-929
 *   contact flags        bipedal_walker_v2.mojo:815-855 (hull contact is sticky until reset)
 *   observation          bipedal_walker_v2.mojo:634-813 (fp64 normalisation, fp32 lidar)
 *   reward / termination bipedal_walker_v2.mojo:1025-1101 (CPU order of the terminal overrides)
 * HalfCheetah (row of 253 floats, layout.mojo:291-299):
 *   constants / shapes   envs/half_cheetah/constants.mojo, cheetah_planar_v2.mojo:288-339
 *   reset                cheetah_planar_v2.mojo:341-594; seed combination :1108
 *   observation          cheetah_planar_v2.mojo:596-656
 *   physics sub-step     cheetah_planar_v2.mojo:658-727
 *   step / reward        cheetah_planar_v2.mojo:745-846 (fp64 reward, 5 sub-steps)
 *
 * Both rows follow the batched trait's buffer protocol: obs at row[0:OBS], metadata slots as in
 * the constants files; the CPU structs' loose fields (prev_shaping, contact flags, game_over,
 * step_count, total_reward) live in those slots.
 */
#include <math.h>
#include <string.h>
#include "orc.h"

static inline float f32_sin(float x) { return (float)sin((double)x); }
static inline float f32_cos(float x) { return (float)cos((double)x); }

static void set_body(float *B, double x, double y, double vx, double vy, double inv_mass,
                     double inv_inertia, int shape) {
    memset(B, 0, sizeof(float) * ORC_BODY_SIZE);
    B[ORC_IDX_X] = (float)x; B[ORC_IDX_Y] = (float)y;
    B[ORC_IDX_VX] = (float)vx; B[ORC_IDX_VY] = (float)vy;
    B[ORC_IDX_INV_MASS] = (float)inv_mass; B[ORC_IDX_INV_INERTIA] = (float)inv_inertia;
    B[ORC_IDX_SHAPE] = (float)shape;
}

static void set_motor_joint(float *J, int a, int b, double ax, double ay, double bx, double by,
                            double lo, double hi, double max_torque) {
    memset(J, 0, sizeof(float) * ORC_JOINT_SIZE);
    J[ORC_J_BODY_A] = (float)a; J[ORC_J_BODY_B] = (float)b;
    J[ORC_J_AX] = (float)ax; J[ORC_J_AY] = (float)ay; J[ORC_J_BX] = (float)bx; J[ORC_J_BY] = (float)by;
    J[ORC_J_LO] = (float)lo; J[ORC_J_HI] = (float)hi;
    J[ORC_J_MAX_TORQUE] = (float)max_torque;
    J[ORC_J_FLAGS] = (float)(ORC_JF_LIMIT | ORC_JF_MOTOR);
}

static void rect_shape(float *S, double hw, double hh, int order) {
    /* order 0: (-w,+h)(-w,-h)(+w,-h)(+w,+h)   order 1: (-w,-h)(-w,+h)(+w,+h)(+w,-h) */
    S[0] = 0.0f; S[1] = 4.0f;
    const double sx[4] = {-1, -1, 1, 1};
    const double sy0[4] = {1, -1, -1, 1}, sy1[4] = {-1, 1, 1, -1};
    for (int i = 0; i < 4; ++i) {
        S[2 + 2 * i] = (float)(sx[i] * hw);
        S[3 + 2 * i] = (float)((order ? sy1[i] : sy0[i]) * hh);
    }
}

static void physics_substep(const orc_layout *L, float *row, const float *shapes, float *contacts,
                            int *n_out, int flat, float gx, float gy, float dt, float friction,
                            float restitution, float baumgarte, float slop, int vel_iters, int pos_iters) {
    orc_integrate_velocities(L, row, gx, gy, dt);
    int n = flat ? orc_flat_detect(L, row, shapes, 0.0f, contacts) : orc_edge_detect(L, row, shapes, contacts);
    for (int it = 0; it < vel_iters; ++it) {
        orc_contact_solve_velocity(L, row, contacts, n, friction, restitution);
        orc_joint_solve_velocity(L, row, dt);
    }
    orc_integrate_positions(L, row, dt);
    for (int it = 0; it < pos_iters; ++it) {
        orc_contact_solve_position(L, row, contacts, n, baumgarte, slop);
        orc_joint_solve_position(L, row, baumgarte, slop);
    }
    for (int k = 0; k < L->num_bodies * 3; ++k) row[L->forces_off + k] = 0.0f;
    *n_out = n;
}

/* ================================================================ BipedalWalker */
#define BW_SCALE 30.0
#define BW_FPS 50.0
#define BW_LEG_DOWN (-8.0 / BW_SCALE)
#define BW_LEG_H (34.0 / BW_SCALE)
#define BW_UPPER_W (6.4 / BW_SCALE)
#define BW_UPPER_H (34.0 / BW_SCALE)
#define BW_LOWER_W (5.12 / BW_SCALE)
#define BW_LOWER_H (34.0 / BW_SCALE)
#define BW_TERRAIN_STEP (14.0 / BW_SCALE)
#define BW_TERRAIN_HEIGHT (400.0 / BW_SCALE / 4.0)
#define BW_TERRAIN_LENGTH 200
#define BW_TERRAIN_GRASS 10
#define BW_TERRAIN_STARTPAD 20
#define BW_MOTORS_TORQUE 80.0
#define BW_LIDAR_RANGE (160.0 / BW_SCALE)
enum { BW_META_STEP = 0, BW_META_TOTAL = 1, BW_META_PREV_SHAPING = 2, BW_META_DONE = 3,
       BW_META_SCROLL = 4, BW_META_LEFT = 5, BW_META_RIGHT = 6, BW_META_GAME_OVER = 7 };

void orc_bw_layout(orc_layout *L) { orc_layout_make(L, 5, 20, 4, 128, 24, 8, 5); }

void orc_bw_shapes(float *shapes /* 5*20 */) {
    memset(shapes, 0, sizeof(float) * 100);
    const double hv[5][2] = {{-30.0 / BW_SCALE, 0.0}, {-6.0 / BW_SCALE, 30.0 / BW_SCALE},
                             {6.0 / BW_SCALE, 30.0 / BW_SCALE}, {30.0 / BW_SCALE, 0.0},
                             {0.0, -12.0 / BW_SCALE}};
    shapes[0] = 0.0f; shapes[1] = 5.0f;
    for (int i = 0; i < 5; ++i) { shapes[2 + 2 * i] = (float)hv[i][0]; shapes[3 + 2 * i] = (float)hv[i][1]; }
    rect_shape(shapes + 20, BW_UPPER_W / 2, BW_UPPER_H / 2, 0);
    rect_shape(shapes + 40, BW_LOWER_W / 2, BW_LOWER_H / 2, 0);
    rect_shape(shapes + 60, BW_UPPER_W / 2, BW_UPPER_H / 2, 0);
    rect_shape(shapes + 80, BW_LOWER_W / 2, BW_LOWER_H / 2, 0);
}

static void bw_observe(const orc_layout *L, float *row) {
    const float *B = row + L->bodies_off;
    double hull_angle = B[ORC_IDX_ANGLE], hull_omega = B[ORC_IDX_OMEGA];
    double hull_vx = B[ORC_IDX_VX], hull_vy = B[ORC_IDX_VY];
    float o[24];
    o[0] = (float)hull_angle;
    o[1] = (float)(hull_omega / 5.0);
    o[2] = (float)(hull_vx * (600.0 / BW_SCALE) / BW_FPS);
    o[3] = (float)(hull_vy * (400.0 / BW_SCALE) / BW_FPS);
    for (int leg = 0; leg < 2; ++leg) {
        const float *U = B + (2 * leg + 1) * ORC_BODY_SIZE, *W = B + (2 * leg + 2) * ORC_BODY_SIZE;
        double ua = U[ORC_IDX_ANGLE], la = W[ORC_IDX_ANGLE], uo = U[ORC_IDX_OMEGA], lo = W[ORC_IDX_OMEGA];
        float *q = o + 4 + 5 * leg;
        q[0] = (float)((ua - hull_angle) / 1.0);
        q[1] = (float)((uo - hull_omega) / 10.0);
        q[2] = (float)((la - ua) / 1.0);
        q[3] = (float)((lo - uo) / 10.0);
        q[4] = row[L->meta_off + (leg ? BW_META_RIGHT : BW_META_LEFT)] > 0.5f ? 1.0f : 0.0f;
    }
    float hull_x = B[ORC_IDX_X], hull_y = B[ORC_IDX_Y], hull_angle_rad = B[ORC_IDX_ANGLE];
    const float lidar_range = (float)BW_LIDAR_RANGE;
    for (int i = 0; i < 10; ++i) {
        float local_angle = (float)i * 1.5f / (float)9;
        float world_angle = hull_angle_rad - local_angle - (float)(3.14159265358979323846 / 2.0);
        float ray_dx = f32_cos(world_angle) * lidar_range;
        float ray_dy = f32_sin(world_angle) * lidar_range;
        o[14 + i] = orc_lidar_ray(L, row, hull_x, hull_y, ray_dx, ray_dy);
    }
    memcpy(row, o, sizeof(o));
}

void orc_bw_reset(float *row, uint64_t cseed) {
    orc_layout L; orc_bw_layout(&L);
    memset(row, 0, sizeof(float) * L.state_size);
    /* terrain: fp32 random walk over the sample points, one Philox draw per point past the start pad */
    float ty[129];
    float y = (float)BW_TERRAIN_HEIGHT, velocity = 0.0f;
    uint64_t draw = 0;
    for (int i = 0; i <= 128; ++i) {
        float terrain_height = (float)BW_TERRAIN_HEIGHT;
        velocity = 0.8f * velocity + 0.01f * (terrain_height > y ? 1.0f : -1.0f);
        if (i > BW_TERRAIN_STARTPAD) {
            float rv[4];
            orc_philox_uniform4(cseed + 1000ull, 0, draw++, rv);
            velocity = velocity + (rv[0] * 2.0f - 1.0f) / (float)BW_SCALE;
        }
        y = y + velocity;
        ty[i] = y;
    }
    row[L.edge_count_off] = 128.0f;
    for (int i = 0; i < 128; ++i) {
        float x0 = (float)i * (float)BW_TERRAIN_STEP, x1 = (float)(i + 1) * (float)BW_TERRAIN_STEP;
        float y0 = ty[i], y1 = ty[i + 1];
        float dx = x1 - x0, dy = y1 - y0;
        float length = sqrtf(dx * dx + dy * dy);
        float nx = -dy / length, ny = dx / length;
        if (ny < 0.0f) { nx = -nx; ny = -ny; }
        float *E = row + L.edges_off + i * 6;
        E[0] = x0; E[1] = y0; E[2] = x1; E[3] = y1; E[4] = nx; E[5] = ny;
    }
    float rv[4];
    orc_philox_uniform4(cseed, 0, 0, rv);
    double init_x = (double)BW_TERRAIN_STARTPAD * BW_TERRAIN_STEP;
    double init_y = BW_TERRAIN_HEIGHT + 2.0 * BW_LEG_H;
    double init_vx = ((double)rv[0] * 2.0 - 1.0) * 0.1, init_vy = ((double)rv[1] * 2.0 - 1.0) * 0.1;
    float *B = row + L.bodies_off;
    set_body(B, init_x, init_y, init_vx, init_vy, 1.0 / 5.0, 1.0 / 2.0, 0);
    for (int leg = 0; leg < 2; ++leg) {
        double upper_y = init_y + BW_LEG_DOWN - BW_UPPER_H / 2;
        set_body(B + (2 * leg + 1) * ORC_BODY_SIZE, init_x, upper_y, init_vx, init_vy, 1.0 / 0.8, 1.0 / 0.1, 2 * leg + 1);
        double lower_y = upper_y - BW_UPPER_H / 2 - BW_LOWER_H / 2;
        set_body(B + (2 * leg + 2) * ORC_BODY_SIZE, init_x, lower_y, init_vx, init_vy, 1.0 / 0.5, 1.0 / 0.05, 2 * leg + 2);
    }
    row[L.joint_count_off] = 4.0f;
    for (int leg = 0; leg < 2; ++leg) {
        float *J = row + L.joints_off + (2 * leg) * ORC_JOINT_SIZE;
        set_motor_joint(J, 0, 2 * leg + 1, 0.0, BW_LEG_DOWN, 0.0, BW_UPPER_H / 2, -0.8, 1.1, BW_MOTORS_TORQUE);
        set_motor_joint(J + ORC_JOINT_SIZE, 2 * leg + 1, 2 * leg + 2, 0.0, -BW_UPPER_H / 2, 0.0, BW_LOWER_H / 2,
                        -1.6, -0.1, BW_MOTORS_TORQUE);
    }
    bw_observe(&L, row);
    double hull_x = B[ORC_IDX_X];
    row[L.meta_off + BW_META_PREV_SHAPING] = (float)(130.0 * hull_x / BW_SCALE);
}

void orc_bw_step(float *row, const float action[4], float *reward, float *done) {
    orc_layout L; orc_bw_layout(&L);
    float shapes[100]; orc_bw_shapes(shapes);
    float contacts[20 * ORC_CONTACT_SIZE];
    const double speed[4] = {4.0, 6.0, 4.0, 6.0};
    for (int j = 0; j < 4; ++j) {
        float a = action[j];
        if (a > 1.0f) a = 1.0f;
        if (a < -1.0f) a = -1.0f;
        float sign = a >= 0.0f ? 1.0f : -1.0f;
        float *J = row + L.joints_off + j * ORC_JOINT_SIZE;
        J[ORC_J_MOTOR_SPEED] = sign * (float)speed[j];
        J[ORC_J_MAX_TORQUE] = (float)BW_MOTORS_TORQUE * fabsf(a);
    }
    int n;
    physics_substep(&L, row, shapes, contacts, &n, 0, (float)0.0, (float)-10.0, (float)(1.0 / BW_FPS),
                    (float)2.5, (float)0.0, (float)0.2, (float)0.005, 6, 2);
    int left = 0, right = 0, hull = 0;
    for (int c = 0; c < n; ++c) {
        int b = (int)contacts[c * ORC_CONTACT_SIZE + ORC_C_BODY_A];
        if (b == 2) left = 1;
        else if (b == 4) right = 1;
        if (b == 0) hull = 1;
    }
    float *M = row + L.meta_off;
    M[BW_META_LEFT] = left ? 1.0f : 0.0f;
    M[BW_META_RIGHT] = right ? 1.0f : 0.0f;
    if (hull) M[BW_META_GAME_OVER] = 1.0f;
    const float *B = row + L.bodies_off;
    M[BW_META_SCROLL] = B[ORC_IDX_X] - (float)(600.0 / BW_SCALE / 5.0);
    bw_observe(&L, row);

    int step_count = (int)M[BW_META_STEP] + 1;
    double hull_x = B[ORC_IDX_X], hull_y = B[ORC_IDX_Y], hull_angle = B[ORC_IDX_ANGLE];
    float new_shaping = (float)(130.0 * hull_x / BW_SCALE);
    float r = new_shaping - M[BW_META_PREV_SHAPING];
    r = r - (float)(5.0 * fabs(hull_angle));
    float energy = fabsf(action[0]) + fabsf(action[1]) + fabsf(action[2]) + fabsf(action[3]);
    r = r - (float)(0.00035 * BW_MOTORS_TORQUE) * energy;
    double min_height = BW_TERRAIN_HEIGHT + BW_LEG_H * 1.5, critical_height = BW_TERRAIN_HEIGHT + BW_LEG_H * 1.2;
    if (hull_y < min_height) r = r - (float)(10.0 * (min_height - hull_y));
    double vel_x = (double)row[2];
    if (vel_x > 0.0) r = r + (float)(3.0 * vel_x);
    else r = r - (float)(5.0 * fabs(vel_x));
    int terminated = 0;
    if (hull_y < critical_height) { r = -50.0f; terminated = 1; }
    if (M[BW_META_GAME_OVER] > 0.5f) { r = -100.0f; terminated = 1; }
    if (hull_x < 0.0) { r = -100.0f; terminated = 1; }
    double terrain_end = (double)(BW_TERRAIN_LENGTH - BW_TERRAIN_GRASS) * BW_TERRAIN_STEP;
    if (hull_x > terrain_end) terminated = 1;
    if (step_count >= 2000) terminated = 1;
    M[BW_META_STEP] = (float)step_count;
    M[BW_META_PREV_SHAPING] = new_shaping;
    M[BW_META_DONE] = terminated ? 1.0f : 0.0f;
    *reward = r;
    *done = terminated ? 1.0f : 0.0f;
}

/* ================================================================ HalfCheetah */
enum { HC_META_STEP = 0, HC_META_PREV_X = 1, HC_META_PREV_SHAPING = 2, HC_META_DONE = 3, HC_META_TOTAL = 4 };
static const double HC_LEN[7] = {1.0, 0.145, 0.15, 0.094, 0.133, 0.106, 0.07};
static const double HC_MASS[7] = {6.25, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0};
static const double HC_LIM[6][2] = {{-0.52, 1.05}, {-0.785, 0.785}, {-0.4, 0.785}, {-1.0, 0.7}, {-1.2, 0.87}, {-0.5, 0.5}};

void orc_hc_layout(orc_layout *L) { orc_layout_make(L, 7, 14, 6, 2, 17, 8, 7); }

void orc_hc_shapes(float *shapes /* 7*20 */) {
    memset(shapes, 0, sizeof(float) * 140);
    /* torso: half_len x radius, vertex order (-,-)(-,+)(+,+)(+,-) */
    rect_shape(shapes, 1.0 / 2, 0.046, 1);
    for (int s = 1; s < 7; ++s) rect_shape(shapes + 20 * s, 0.046, HC_LEN[s] / 2, 1);
}

static void hc_observe(const orc_layout *L, float *row) {
    const float *B = row + L->bodies_off;
#define ANG(b) ((double)B[(b) * ORC_BODY_SIZE + ORC_IDX_ANGLE])
#define OMG(b) ((double)B[(b) * ORC_BODY_SIZE + ORC_IDX_OMEGA])
    float o[17];
    o[0] = B[ORC_IDX_Y]; o[1] = B[ORC_IDX_ANGLE];
    o[2] = (float)(ANG(1) - ANG(0)); o[3] = (float)(ANG(2) - ANG(1)); o[4] = (float)(ANG(3) - ANG(2));
    o[5] = (float)(ANG(4) - ANG(0)); o[6] = (float)(ANG(5) - ANG(4)); o[7] = (float)(ANG(6) - ANG(5));
    o[8] = B[ORC_IDX_VX]; o[9] = B[ORC_IDX_VY]; o[10] = B[ORC_IDX_OMEGA];
    o[11] = (float)(OMG(1) - OMG(0)); o[12] = (float)(OMG(2) - OMG(1)); o[13] = (float)(OMG(3) - OMG(2));
    o[14] = (float)(OMG(4) - OMG(0)); o[15] = (float)(OMG(5) - OMG(4)); o[16] = (float)(OMG(6) - OMG(5));
#undef ANG
#undef OMG
    memcpy(row, o, sizeof(o));
}

void orc_hc_reset(float *row, uint64_t cseed) {
    orc_layout L; orc_hc_layout(&L);
    memset(row, 0, sizeof(float) * L.state_size);
    float rv[4];
    orc_philox_uniform4(cseed, 0, 0, rv);
    double init_x = 0.0, init_y = 0.7;
    double init_vx = ((double)rv[0] * 2.0 - 1.0) * 0.1, init_vy = ((double)rv[1] * 2.0 - 1.0) * 0.1;
    float *B = row + L.bodies_off;
    set_body(B, init_x, init_y, init_vx, init_vy, 1.0 / HC_MASS[0], 1.0 / (HC_MASS[0] * 1.0 * 1.0 / 12.0), 0);
    for (int leg = 0; leg < 2; ++leg) {
        double hip_x = leg == 0 ? init_x - 1.0 / 2 : init_x + 1.0 / 2;
        int b0 = 1 + 3 * leg;
        double tl = HC_LEN[b0], sl = HC_LEN[b0 + 1], fl = HC_LEN[b0 + 2];
        double ys[3] = {init_y - tl / 2, init_y - tl - sl / 2, init_y - tl - sl - fl / 2};
        for (int k = 0; k < 3; ++k) {
            double len = HC_LEN[b0 + k], m = HC_MASS[b0 + k];
            set_body(B + (b0 + k) * ORC_BODY_SIZE, hip_x, ys[k], init_vx, init_vy, 1.0 / m,
                     1.0 / (m * len * len / 12.0), b0 + k);
        }
    }
    row[L.joint_count_off] = 6.0f;
    float *J = row + L.joints_off;
    set_motor_joint(J + 0 * ORC_JOINT_SIZE, 0, 1, -1.0 / 2, 0.0, 0.0, HC_LEN[1] / 2, HC_LIM[0][0], HC_LIM[0][1], 1.0);
    set_motor_joint(J + 1 * ORC_JOINT_SIZE, 1, 2, 0.0, -HC_LEN[1] / 2, 0.0, HC_LEN[2] / 2, HC_LIM[1][0], HC_LIM[1][1], 1.0);
    set_motor_joint(J + 2 * ORC_JOINT_SIZE, 2, 3, 0.0, -HC_LEN[2] / 2, 0.0, HC_LEN[3] / 2, HC_LIM[2][0], HC_LIM[2][1], 1.0);
    set_motor_joint(J + 3 * ORC_JOINT_SIZE, 0, 4, 1.0 / 2, 0.0, 0.0, HC_LEN[4] / 2, HC_LIM[3][0], HC_LIM[3][1], 1.0);
    set_motor_joint(J + 4 * ORC_JOINT_SIZE, 4, 5, 0.0, -HC_LEN[4] / 2, 0.0, HC_LEN[5] / 2, HC_LIM[4][0], HC_LIM[4][1], 1.0);
    set_motor_joint(J + 5 * ORC_JOINT_SIZE, 5, 6, 0.0, -HC_LEN[5] / 2, 0.0, HC_LEN[6] / 2, HC_LIM[5][0], HC_LIM[5][1], 1.0);
    row[L.meta_off + HC_META_PREV_X] = (float)init_x;
    hc_observe(&L, row);
}

void orc_hc_step(float *row, const float action[6], float *reward, float *done) {
    orc_layout L; orc_hc_layout(&L);
    float shapes[140]; orc_hc_shapes(shapes);
    float contacts[14 * ORC_CONTACT_SIZE];
    double a[6];
    for (int j = 0; j < 6; ++j) {
        float v = action[j];
        v = v < 1.0f ? v : 1.0f;      /* max(min(a, 1), -1) */
        v = v > -1.0f ? v : -1.0f;
        a[j] = (double)v;
        float *J = row + L.joints_off + j * ORC_JOINT_SIZE;
        J[ORC_J_MOTOR_SPEED] = (a[j] >= 0.0 ? 1.0f : -1.0f) * 1000.0f;
        J[ORC_J_MAX_TORQUE] = (float)(1.0 * fabs(a[j]));
    }
    float *B = row + L.bodies_off;
    double x_before = B[ORC_IDX_X];
    int n = 0;
    for (int s = 0; s < 5; ++s)
        physics_substep(&L, row, shapes, contacts, &n, 1, (float)0.0, (float)-9.81, (float)0.01, (float)0.9,
                        (float)0.0, (float)0.2, (float)0.005, 4, 2);
    double x_after = B[ORC_IDX_X], torso_z = B[ORC_IDX_Y];
    double forward_velocity = (x_after - x_before) / (0.01 * (double)5);
    double forward_reward = 1.0 * forward_velocity;
    double ctrl_cost = 0.0;
    for (int i = 0; i < 6; ++i) {
        double c = a[i] < 1.0 ? a[i] : 1.0;
        c = c > -1.0 ? c : -1.0;
        ctrl_cost += c * c;
    }
    ctrl_cost *= 0.1;
    double height_bonus = 0.0;
    if (torso_z > 0.1) height_bonus = 1.0 * (torso_z < 0.5 ? torso_z : 0.5);
    double penalty = 0.0;
    for (int c = 0; c < n; ++c) {
        int ba = (int)contacts[c * ORC_CONTACT_SIZE + ORC_C_BODY_A], bb = (int)contacts[c * ORC_CONTACT_SIZE + ORC_C_BODY_B];
        if (bb == -1 && ba != 3 && ba != 6) penalty += 0.5;
    }
    double r = forward_reward - ctrl_cost + height_bonus - penalty;
    float *M = row + L.meta_off;
    int step_count = (int)M[HC_META_STEP] + 1;
    M[HC_META_STEP] = (float)step_count;
    M[HC_META_PREV_X] = (float)x_after;
    M[HC_META_TOTAL] = (float)((double)M[HC_META_TOTAL] + r);
    int d = step_count >= 1000;
    M[HC_META_DONE] = d ? 1.0f : 0.0f;
    hc_observe(&L, row);
    *reward = (float)r;
    *done = d ? 1.0f : 0.0f;
}

/* ================================================================ batched wrappers */
static uint64_t walker_seed(uint64_t seed, int env) {
    int64_t seed_i = (int64_t)(float)seed;
    return (uint64_t)seed_i * 2654435761ull + (uint64_t)(env + 1) * 12345ull;
}

void orc_bw_reset_batch(float *states, const float *dones, int batch, uint64_t seed) {
    for (int i = 0; i < batch; ++i)
        if (!dones || dones[i] > 0.5f) orc_bw_reset(states + (long)i * 950, walker_seed(seed, i));
}
void orc_bw_step_batch(float *states, const float *actions, float *rewards, float *dones, float *obs,
                       int batch, int n_threads) {
    (void)n_threads;
#ifdef _OPENMP
#pragma omp parallel for num_threads(n_threads > 0 ? n_threads : 1) schedule(static)
#endif
    for (int i = 0; i < batch; ++i) {
        float *row = states + (long)i * 950;
        orc_bw_step(row, actions + (long)i * 4, rewards + i, dones + i);
        memcpy(obs + (long)i * 24, row, sizeof(float) * 24);
    }
}
void orc_hc_reset_batch(float *states, const float *dones, int batch, uint64_t seed) {
    for (int i = 0; i < batch; ++i)
        if (!dones || dones[i] > 0.5f) orc_hc_reset(states + (long)i * 253, walker_seed(seed, i));
}
void orc_hc_step_batch(float *states, const float *actions, float *rewards, float *dones, float *obs,
                       int batch, int n_threads) {
    (void)n_threads;
#ifdef _OPENMP
#pragma omp parallel for num_threads(n_threads > 0 ? n_threads : 1) schedule(static)
#endif
    for (int i = 0; i < batch; ++i) {
        float *row = states + (long)i * 253;
        orc_hc_step(row, actions + (long)i * 6, rewards + i, dones + i);
        memcpy(obs + (long)i * 17, row, sizeof(float) * 17);
    }
}
