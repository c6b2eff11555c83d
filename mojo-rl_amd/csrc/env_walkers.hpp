// BipedalWalkerV2 and HalfCheetahPlanarV2 on one env row (one lane per env, row in LDS).
//
// BipedalWalker: envs/bipedal_walker/bipedal_walker_v2.mojo -- reset :366-622 (terrain random
// walk in fp32, 128 edges kept), motors :931-1003, physics :857-929, contact flags :815-855,
// observation :634-813 (fp64 normalisation, fp32 lidar over the row's edges), reward and the CPU
// order of terminal overrides :1025-1101; constants envs/bipedal_walker/constants_v2.mojo.
// HalfCheetah: envs/half_cheetah/cheetah_planar_v2.mojo -- reset :341-594, observation :596-656,
// physics sub-step :658-727 (flat ground at y = 0), step with 5 sub-steps and fp64 reward
// :745-846; constants envs/half_cheetah/constants.mojo.
// Reset seed for both: Int(f32(seed)) * 2654435761 + (env + 1) * 12345 (:1444 / :1108).
#pragma once
#include "physics2d_reg.hpp"

namespace mrl {

MRL_DEV void w_set_body(float *B, double x, double y, double vx, double vy, double inv_mass,
                        double inv_inertia, int shape) {
    for (int k = 0; k < BODY_SIZE; ++k) B[k] = 0.0f;
    B[IDX_X] = (float)x; B[IDX_Y] = (float)y; B[IDX_VX] = (float)vx; B[IDX_VY] = (float)vy;
    B[IDX_INV_MASS] = (float)inv_mass; B[IDX_INV_INERTIA] = (float)inv_inertia;
    B[IDX_SHAPE] = (float)shape;
}

MRL_DEV void w_set_motor_joint(float *J, int a, int b, double ax, double ay, double bx, double by,
                               double lo, double hi, double max_torque) {
    for (int k = 0; k < JOINT_SIZE; ++k) J[k] = 0.0f;
    J[J_BODY_A] = (float)a; J[J_BODY_B] = (float)b;
    J[J_AX] = (float)ax; J[J_AY] = (float)ay; J[J_BX] = (float)bx; J[J_BY] = (float)by;
    J[J_LO] = (float)lo; J[J_HI] = (float)hi;
    J[J_MAX_TORQUE] = (float)max_torque;
    J[J_FLAGS] = (float)(JF_LIMIT | JF_MOTOR);
}

inline void rect_shape(float *S, double hw, double hh, int order) {
    S[0] = 0.0f; S[1] = 4.0f;
    const double sx[4] = {-1, -1, 1, 1};
    const double sy0[4] = {1, -1, -1, 1}, sy1[4] = {-1, 1, 1, -1};
    for (int i = 0; i < 4; ++i) {
        S[2 + 2 * i] = (float)(sx[i] * hw);
        S[3 + 2 * i] = (float)((order ? sy1[i] : sy0[i]) * hh);
    }
}

MRL_DEV uint64_t walker_seed(uint64_t seed, int env) {
    int64_t seed_i = (int64_t)(float)seed;
    return (uint64_t)seed_i * 2654435761ull + (uint64_t)(env + 1) * 12345ull;
}


// ================================================================ BipedalWalker
namespace bw {
using L = BipedalWalkerLayout;

// hull(0) - upper leg(1) - lower leg(2), hull(0) - upper leg(3) - lower leg(4): reset_row below
struct Topology {
    static constexpr bool STATIC = true;
    static constexpr MRL_DEV int a(int j) { return (j & 1) ? j : 0; }
    static constexpr MRL_DEV int b(int j) { return j + 1; }
};
constexpr int STATE = L::STATE_SIZE, OBS = 24, ACT = 4, NSHAPE_FLOATS = 5 * SHAPE_SIZE;
constexpr double SCALE = 30.0, FPS = 50.0;
constexpr double LEG_DOWN = -8.0 / SCALE, LEG_H = 34.0 / SCALE;
constexpr double UPPER_W = 6.4 / SCALE, UPPER_H = 34.0 / SCALE, LOWER_W = 5.12 / SCALE, LOWER_H = 34.0 / SCALE;
constexpr double TERRAIN_STEP = 14.0 / SCALE, TERRAIN_HEIGHT = 400.0 / SCALE / 4.0;
constexpr int TERRAIN_LENGTH = 200, TERRAIN_GRASS = 10, TERRAIN_STARTPAD = 20, N_EDGES = 128;
constexpr double MOTORS_TORQUE = 80.0, LIDAR_RANGE = 160.0 / SCALE;
enum { META_STEP = 0, META_TOTAL = 1, META_PREV_SHAPING = 2, META_DONE = 3, META_SCROLL = 4,
       META_LEFT = 5, META_RIGHT = 6, META_GAME_OVER = 7 };

struct Shapes { float v[NSHAPE_FLOATS]; };
inline Shapes make_shapes() {
    Shapes s{};
    const double hv[5][2] = {{-30.0 / SCALE, 0.0}, {-6.0 / SCALE, 30.0 / SCALE}, {6.0 / SCALE, 30.0 / SCALE},
                             {30.0 / SCALE, 0.0}, {0.0, -12.0 / SCALE}};
    s.v[0] = 0.0f; s.v[1] = 5.0f;
    for (int i = 0; i < 5; ++i) { s.v[2 + 2 * i] = (float)hv[i][0]; s.v[3 + 2 * i] = (float)hv[i][1]; }
    rect_shape(s.v + 20, UPPER_W / 2, UPPER_H / 2, 0);
    rect_shape(s.v + 40, LOWER_W / 2, LOWER_H / 2, 0);
    rect_shape(s.v + 60, UPPER_W / 2, UPPER_H / 2, 0);
    rect_shape(s.v + 80, LOWER_W / 2, LOWER_H / 2, 0);
    for (int k = 0; k < 5; ++k) shape_set_bounds(s.v + k * SHAPE_SIZE);
    return s;
}

// observation entries 0 .. 13: hull and joint state, leg contact flags
MRL_DEV void observe_state(const float *row, float *o) {
    const float *B = row + L::BODIES_OFF;
    double hull_angle = B[IDX_ANGLE], hull_omega = B[IDX_OMEGA], hull_vx = B[IDX_VX], hull_vy = B[IDX_VY];
    o[0] = (float)hull_angle;
    o[1] = (float)(hull_omega / 5.0);
    o[2] = (float)(hull_vx * (600.0 / SCALE) / FPS);
    o[3] = (float)(hull_vy * (400.0 / SCALE) / FPS);
#pragma unroll
    for (int leg = 0; leg < 2; ++leg) {
        const float *U = B + (2 * leg + 1) * BODY_SIZE, *W = B + (2 * leg + 2) * BODY_SIZE;
        double ua = U[IDX_ANGLE], la = W[IDX_ANGLE], uo = U[IDX_OMEGA], lo = W[IDX_OMEGA];
        float *q = o + 4 + 5 * leg;
        q[0] = (float)((ua - hull_angle) / 1.0);
        q[1] = (float)((uo - hull_omega) / 10.0);
        q[2] = (float)((la - ua) / 1.0);
        q[3] = (float)((lo - uo) / 10.0);
        q[4] = row[L::META_OFF + (leg ? META_RIGHT : META_LEFT)] > 0.5f ? 1.0f : 0.0f;
    }
}

// observation entry 14 + i: lidar ray i of ten.  near != nullptr: the edges within lidar range of
// the hull in x, selected by the caller once for all its rays (every ray stays within that range)
MRL_DEV float lidar_value(const float *row, int i, const EdgeMask<L> *near) {
    const float *B = row + L::BODIES_OFF;
    const float hull_x = B[IDX_X], hull_y = B[IDX_Y], hull_angle_rad = B[IDX_ANGLE];
    const float lidar_range = (float)LIDAR_RANGE;
    float local_angle = (float)i * 1.5f / (float)9;
    float world_angle = hull_angle_rad - local_angle - (float)(3.14159265358979323846 / 2.0);
    float sn, cs;
    sincos32(world_angle, sn, cs);
    if (!(hull_x == hull_x)) return lidar_ray<L>(row, hull_x, hull_y, cs * lidar_range, sn * lidar_range);
    if (near != nullptr) return lidar_ray_near<L>(row, *near, hull_x, hull_y, cs * lidar_range, sn * lidar_range);
    EdgeMask<L> mine;
    edges_near<L>(row, hull_x - lidar_range, hull_x + lidar_range, 0.02f, mine);
    return lidar_ray_near<L>(row, mine, hull_x, hull_y, cs * lidar_range, sn * lidar_range);
}

// Ahead of contact detection by one lane per (body, vertex), once per env and by all its `SLOTS` lanes: the
// mask of the edges near any of its bodies (words = the env's WORDS mask words); lanes and stores as
// in lidar_near_share.
template <int SLOTS, int EPB>
MRL_DEV void detect_near_share(const float *row, const float *shapes, int slot, unsigned *words) {
    constexpr int PER = L::MAX_EDGES / SLOTS;
    static_assert(PER * SLOTS == L::MAX_EDGES && 4 * EPB == 64 && 4 * PER == 16, "sixteen mask bits per wavefront");
    float xlo, xhi;
    bodies_x_interval<L>(row, shapes, xlo, xhi);
    unsigned b = edges_near_bits<L, PER>(row, xlo, xhi, 0.0f, slot * PER) << (PER * (slot & 3));
    b |= __shfl_xor(b, EPB, 64);
    b |= __shfl_xor(b, 2 * EPB, 64);
    if ((slot & 3) == 0) reinterpret_cast<unsigned short *>(words)[slot >> 2] = (unsigned short)b;
}

// The lidar rays of an env spread over the lanes of a block.
//
// lidar_near_share: ahead of the rays, once per env, the mask of the edges within lidar range of the
// hull in x (every ray stays inside that range), each of the env's `SLOTS` lanes testing its share of
// the edges; the four lanes of an env in a wavefront (they sit EPB lanes apart) combine their bits and
// store sixteen of them.  words = the env's WORDS mask words.
template <int SLOTS, int EPB>
MRL_DEV void lidar_near_share(const float *row, int slot, unsigned *words) {
    constexpr int PER = L::MAX_EDGES / SLOTS;
    static_assert(PER * SLOTS == L::MAX_EDGES && 4 * EPB == 64 && 4 * PER == 16, "sixteen mask bits per wavefront");
    const float hull_x = row[L::BODIES_OFF + IDX_X], lidar_range = (float)LIDAR_RANGE;
    unsigned b = edges_near_bits<L, PER>(row, hull_x - lidar_range, hull_x + lidar_range, 0.02f, slot * PER) << (PER * (slot & 3));
    b |= __shfl_xor(b, EPB, 64);
    b |= __shfl_xor(b, 2 * EPB, 64);
    if ((slot & 3) == 0) reinterpret_cast<unsigned short *>(words)[slot >> 2] = (unsigned short)b;
}

// Lidar ray i against a share of those edges: part `part` of NPARTS takes the edges whose number is
// `part` modulo NPARTS (the edges in range are a run of neighbours, so the shares come out even); the
// ray's value is the minimum over the parts (every part starts from 1, the value of a ray that hits
// nothing, and a hit replaces it only by something smaller: the minimum over all edges, however they
// are grouped).  lidar_ray_pick looks at each edge's extent against the ray's own, as lidar_ray_near does.
template <int NPARTS>
MRL_DEV float lidar_value_part(const float *row, int i, int part, const unsigned *near) {
    static_assert(NPARTS >= 2 && NPARTS <= 4, "share masks for two to four parts");
    const float *B = row + L::BODIES_OFF;
    const float hull_x = B[IDX_X], hull_y = B[IDX_Y], hull_angle_rad = B[IDX_ANGLE];
    const float lidar_range = (float)LIDAR_RANGE;
    float local_angle = (float)i * 1.5f / (float)9;
    float world_angle = hull_angle_rad - local_angle - (float)(3.14159265358979323846 / 2.0);
    float sn, cs;
    sincos32(world_angle, sn, cs);
    const float rdx = cs * lidar_range, rdy = sn * lidar_range;
    if (!(hull_x == hull_x)) return part == 0 ? lidar_ray<L>(row, hull_x, hull_y, rdx, rdy) : 1.0f;
    const float end_x = hull_x + rdx;
    if (!(end_x == end_x)) return part == 0 ? lidar_ray<L>(row, hull_x, hull_y, rdx, rdy) : 1.0f;
    EdgeMask<L> mine;
#pragma unroll
    for (int q = 0; q < EdgeMask<L>::WORDS; ++q) {
        // bits k of word q with (32 q + k) % NPARTS == part
        unsigned share;
        if (NPARTS == 2) {
            share = part ? 0xaaaaaaaau : 0x55555555u;
        } else if (NPARTS == 4) {
            share = 0x11111111u << part;
        } else {
            const int j = (part + q) % 3;    // 32 q + k = part (mod 3)  <=>  k = part + q (mod 3)
            share = j == 0 ? 0x49249249u : (j == 1 ? 0x92492492u : 0x24924924u);
        }
        mine.w[q] = lidar_ray_pick<L>(row, near[q] & share, q, hull_x, rdx);
    }
    return lidar_ray_picked<L>(row, mine, hull_x, hull_y, rdx, rdy);
}

MRL_DEV void observe(float *row) {
    float o[OBS];
    observe_state(row, o);
    const float hull_x = row[L::BODIES_OFF + IDX_X], lidar_range = (float)LIDAR_RANGE;
    EdgeMask<L> near;
    const bool plain = !(hull_x == hull_x);
    if (!plain) edges_near<L>(row, hull_x - lidar_range, hull_x + lidar_range, 0.02f, near);
    for (int i = 0; i < 10; ++i) o[14 + i] = lidar_value(row, i, &near);
#pragma unroll
    for (int k = 0; k < OBS; ++k) row[k] = o[k];
}

MRL_DEV void reset_row(float *row, uint64_t cseed) {
    for (int k = 0; k < STATE; ++k) row[k] = 0.0f;
    float y = (float)TERRAIN_HEIGHT, velocity = 0.0f, prev_y = 0.0f;
    uint64_t draw = 0;
    for (int i = 0; i <= N_EDGES; ++i) {
        const float terrain_height = (float)TERRAIN_HEIGHT;
        velocity = 0.8f * velocity + 0.01f * (terrain_height > y ? 1.0f : -1.0f);
        if (i > TERRAIN_STARTPAD) {
            Uniform4 rv = philox_uniform4(cseed + 1000ull, 0, draw++);
            velocity = velocity + (rv.v[0] * 2.0f - 1.0f) / (float)SCALE;
        }
        y = y + velocity;
        if (i > 0) {
            float x0 = (float)(i - 1) * (float)TERRAIN_STEP, x1 = (float)i * (float)TERRAIN_STEP;
            float y0 = prev_y, y1 = y;
            float dx = x1 - x0, dy = y1 - y0;
            float length = sqrtf(dx * dx + dy * dy);
            float nx = -dy / length, ny = dx / length;
            if (ny < 0.0f) { nx = -nx; ny = -ny; }
            float *E = row + L::EDGES_OFF + (i - 1) * 6;
            E[0] = x0; E[1] = y0; E[2] = x1; E[3] = y1; E[4] = nx; E[5] = ny;
        }
        prev_y = y;
    }
    row[L::EDGE_COUNT_OFF] = (float)N_EDGES;
    Uniform4 rv = philox_uniform4(cseed, 0, 0);
    const double init_x = (double)TERRAIN_STARTPAD * TERRAIN_STEP;
    const double init_y = TERRAIN_HEIGHT + 2.0 * LEG_H;
    const double init_vx = ((double)rv.v[0] * 2.0 - 1.0) * 0.1, init_vy = ((double)rv.v[1] * 2.0 - 1.0) * 0.1;
    float *B = row + L::BODIES_OFF;
    w_set_body(B, init_x, init_y, init_vx, init_vy, 1.0 / 5.0, 1.0 / 2.0, 0);
    for (int leg = 0; leg < 2; ++leg) {
        double upper_y = init_y + LEG_DOWN - UPPER_H / 2;
        w_set_body(B + (2 * leg + 1) * BODY_SIZE, init_x, upper_y, init_vx, init_vy, 1.0 / 0.8, 1.0 / 0.1, 2 * leg + 1);
        double lower_y = upper_y - UPPER_H / 2 - LOWER_H / 2;
        w_set_body(B + (2 * leg + 2) * BODY_SIZE, init_x, lower_y, init_vx, init_vy, 1.0 / 0.5, 1.0 / 0.05, 2 * leg + 2);
    }
    row[L::JOINT_COUNT_OFF] = 4.0f;
    for (int leg = 0; leg < 2; ++leg) {
        float *J = row + L::JOINTS_OFF + (2 * leg) * JOINT_SIZE;
        w_set_motor_joint(J, 0, 2 * leg + 1, 0.0, LEG_DOWN, 0.0, UPPER_H / 2, -0.8, 1.1, MOTORS_TORQUE);
        w_set_motor_joint(J + JOINT_SIZE, 2 * leg + 1, 2 * leg + 2, 0.0, -UPPER_H / 2, 0.0, LOWER_H / 2, -1.6, -0.1,
                          MOTORS_TORQUE);
    }
    observe(row);
    double hull_x = B[IDX_X];
    row[L::META_OFF + META_PREV_SHAPING] = (float)(130.0 * hull_x / SCALE);
}

MRL_DEV void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// reset_row by the 64 lanes of a wavefront together (all lanes call it with the same row): the
// Philox draws of the terrain walk, the edges, the bodies / joints and the observation's lidar
// rays are spread over the lanes; the walk itself, a recursion through sign(height - y), stays on
// one lane.  Every value comes from the expressions of reset_row, so the row is bit-identical.
MRL_DEV void reset_row_wave(float *row, uint64_t cseed, int lane) {
    for (int k = lane; k < STATE; k += 64) row[k] = 0.0f;
    wave_sync();
    // parked in the (still unused) edge area: the noise of terrain step i at [i], the height y_i at [YS + i]
    float *tmp = row + L::EDGES_OFF;
    constexpr int YS = 200;
    static_assert(YS + N_EDGES + 1 <= N_EDGES * 6 && N_EDGES + 1 <= YS, "scratch inside the edge area");
    for (int i = TERRAIN_STARTPAD + 1 + lane; i <= N_EDGES; i += 64) {
        Uniform4 rv = philox_uniform4(cseed + 1000ull, 0, (uint64_t)(i - TERRAIN_STARTPAD - 1));
        tmp[i] = (rv.v[0] * 2.0f - 1.0f) / (float)SCALE;
    }
    wave_sync();
    if (lane == 0) {
        // the heights are one serial chain; sixteen steps at a time between registers, so that no
        // step waits for an LDS access
        float y = (float)TERRAIN_HEIGHT, velocity = 0.0f;
        constexpr int CH = 16;
        static_assert(N_EDGES % CH == 0, "whole chunks, then the last step");
        auto step = [&](int i, float noise) {
            const float terrain_height = (float)TERRAIN_HEIGHT;
            velocity = 0.8f * velocity + 0.01f * (terrain_height > y ? 1.0f : -1.0f);
            if (i > TERRAIN_STARTPAD) velocity = velocity + noise;
            y = y + velocity;
        };
        for (int i0 = 0; i0 < N_EDGES; i0 += CH) {
            float nz[CH], ys[CH];
#pragma unroll
            for (int j = 0; j < CH; ++j) nz[j] = i0 + j > TERRAIN_STARTPAD ? tmp[i0 + j] : 0.0f;
#pragma unroll
            for (int j = 0; j < CH; ++j) {
                step(i0 + j, nz[j]);
                ys[j] = y;
            }
#pragma unroll
            for (int j = 0; j < CH; ++j) tmp[YS + i0 + j] = ys[j];
        }
        step(N_EDGES, tmp[N_EDGES]);
        tmp[YS + N_EDGES] = y;
    }
    wave_sync();
    float ya[2], yb[2];   // this lane's edges lane and lane + 64: heights at both ends
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int i = lane + 64 * q + 1;
        ya[q] = tmp[YS + i - 1];
        yb[q] = tmp[YS + i];
    }
    wave_sync();   // all heights read before the first edge overwrites the scratch
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int i = lane + 64 * q + 1;
        float x0 = (float)(i - 1) * (float)TERRAIN_STEP, x1 = (float)i * (float)TERRAIN_STEP;
        float y0 = ya[q], y1 = yb[q];
        float dx = x1 - x0, dy = y1 - y0;
        float length = sqrtf(dx * dx + dy * dy);
        float nx = -dy / length, ny = dx / length;
        if (ny < 0.0f) { nx = -nx; ny = -ny; }
        float *E = row + L::EDGES_OFF + (i - 1) * 6;
        E[0] = x0; E[1] = y0; E[2] = x1; E[3] = y1; E[4] = nx; E[5] = ny;
    }
    static_assert(N_EDGES == 128, "two edges per lane");
    Uniform4 rv = philox_uniform4(cseed, 0, 0);
    const double init_x = (double)TERRAIN_STARTPAD * TERRAIN_STEP;
    const double init_y = TERRAIN_HEIGHT + 2.0 * LEG_H;
    const double init_vx = ((double)rv.v[0] * 2.0 - 1.0) * 0.1, init_vy = ((double)rv.v[1] * 2.0 - 1.0) * 0.1;
    float *B = row + L::BODIES_OFF;
    if (lane == 0) {
        row[L::EDGE_COUNT_OFF] = (float)N_EDGES;
        row[L::JOINT_COUNT_OFF] = 4.0f;
        w_set_body(B, init_x, init_y, init_vx, init_vy, 1.0 / 5.0, 1.0 / 2.0, 0);
    }
    if (lane == 1 || lane == 2) {
        const int leg = lane - 1;
        double upper_y = init_y + LEG_DOWN - UPPER_H / 2;
        w_set_body(B + (2 * leg + 1) * BODY_SIZE, init_x, upper_y, init_vx, init_vy, 1.0 / 0.8, 1.0 / 0.1, 2 * leg + 1);
        double lower_y = upper_y - UPPER_H / 2 - LOWER_H / 2;
        w_set_body(B + (2 * leg + 2) * BODY_SIZE, init_x, lower_y, init_vx, init_vy, 1.0 / 0.5, 1.0 / 0.05, 2 * leg + 2);
    }
    if (lane == 3 || lane == 4) {
        const int leg = lane - 3;
        float *J = row + L::JOINTS_OFF + (2 * leg) * JOINT_SIZE;
        w_set_motor_joint(J, 0, 2 * leg + 1, 0.0, LEG_DOWN, 0.0, UPPER_H / 2, -0.8, 1.1, MOTORS_TORQUE);
        w_set_motor_joint(J + JOINT_SIZE, 2 * leg + 1, 2 * leg + 2, 0.0, -UPPER_H / 2, 0.0, LOWER_H / 2, -1.6, -0.1,
                          MOTORS_TORQUE);
    }
    wave_sync();
    // observation: the edges within lidar range of the hull, two tested per lane; then lane 4 r + p takes
    // part p of ray r's edges and the four of a ray exchange their minima; lane 40 the rest
    unsigned near[EdgeMask<L>::WORDS];
    {
        const float hull_x = B[IDX_X], lidar_range = (float)LIDAR_RANGE;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const unsigned long long m = __ballot(edges_near_bits<L, 1>(row, hull_x - lidar_range, hull_x + lidar_range, 0.02f, lane + 64 * h) != 0u);
            near[2 * h] = (unsigned)m;
            near[2 * h + 1] = (unsigned)(m >> 32);
        }
    }
    if (lane < 40) {
        float t = lidar_value_part<4>(row, lane >> 2, lane & 3, near);
#pragma unroll
        for (int off = 1; off <= 2; off <<= 1) {
            const float other = __shfl_xor(t, off, 64);
            t = other < t ? other : t;
        }
        if ((lane & 3) == 0) row[14 + (lane >> 2)] = t;
    } else if (lane == 40) {
        float o[14];
        observe_state(row, o);
#pragma unroll
        for (int k = 0; k < 14; ++k) row[k] = o[k];
        double hull_x = B[IDX_X];
        row[L::META_OFF + META_PREV_SHAPING] = (float)(130.0 * hull_x / SCALE);
    }
    wave_sync();
}

// An env step in two halves, so that contact detection (which reads body positions, shapes and
// edges only) can run on other lanes beside the first:
//   step_motors   the action into the joint motors (writes joints only); act = the raw action
//   step_finish   physics with the `n_given` contacts in `contacts` (n_given < 0: detect here),
//                 contact flags, observation, reward, termination.
// LIDAR = false: the lidar entries of the observation (14 .. 23) are left to the caller
MRL_DEV void step_motors(float *row, const float *action, float *act) {
#pragma unroll
    for (int j = 0; j < ACT; ++j) {
        act[j] = action[j];
        float a = act[j];
        if (a > 1.0f) a = 1.0f;
        if (a < -1.0f) a = -1.0f;
        float sign = a >= 0.0f ? 1.0f : -1.0f;
        float *J = row + L::JOINTS_OFF + j * JOINT_SIZE;
        J[J_MOTOR_SPEED] = sign * (float)((j & 1) ? 6.0 : 4.0);
        J[J_MAX_TORQUE] = (float)MOTORS_TORQUE * fabsf(a);
    }
}

// what follows the physics of a step: contact flags, observation, reward, termination; `n` = the
// contacts of the step, whose body indices are still in `contacts`
// STATE_OBS = false: observation entries 0 .. 7 and 9 .. 12 are in the row already (physics_lanes leaves them)
template <bool LIDAR = true, bool STATE_OBS = true>
MRL_DEV void step_tail(float *row, const float *contacts, int n, const float *act, float &reward, float &done);

template <bool LIDAR = true>
MRL_DEV void step_finish(float *row, float *contacts, int n_given, const float *shapes, const float *act,
                         float &reward, float &done) {
    int n = reg_physics_substep<L, Topology, false, false>(row, shapes, contacts, (float)0.0, (float)-10.0, (float)(1.0 / FPS),
                                      (float)2.5, (float)0.0, (float)0.2, (float)0.005, 6, 2, n_given);
    step_tail<LIDAR>(row, contacts, n, act, reward, done);
}

template <bool LIDAR, bool STATE_OBS>
MRL_DEV void step_tail(float *row, const float *contacts, int n, const float *act, float &reward, float &done) {
    bool left = false, right = false, hull = false;
    for (int c = 0; c < n; ++c) {
        int b = (int)contacts[c * CONTACT_SIZE + C_BODY_A];
        if (b == 2) left = true;
        else if (b == 4) right = true;
        if (b == 0) hull = true;
    }
    float *M = row + L::META_OFF;
    M[META_LEFT] = left ? 1.0f : 0.0f;
    M[META_RIGHT] = right ? 1.0f : 0.0f;
    if (hull) M[META_GAME_OVER] = 1.0f;
    const float *B = row + L::BODIES_OFF;
    M[META_SCROLL] = B[IDX_X] - (float)(600.0 / SCALE / 5.0);
    static_assert(STATE_OBS || !LIDAR, "the lidar form writes the whole observation");
    if (LIDAR) {
        observe(row);
    } else if (!STATE_OBS) {
        row[8] = left ? 1.0f : 0.0f;
        row[13] = right ? 1.0f : 0.0f;
    } else {
        float o[14];
        observe_state(row, o);
#pragma unroll
        for (int k = 0; k < 14; ++k) row[k] = o[k];
    }

    int step_count = (int)M[META_STEP] + 1;
    double hull_x = B[IDX_X], hull_y = B[IDX_Y], hull_angle = B[IDX_ANGLE];
    float new_shaping = (float)(130.0 * hull_x / SCALE);
    float r = new_shaping - M[META_PREV_SHAPING];
    r = r - (float)(5.0 * ::fabs(hull_angle));
    float energy = fabsf(act[0]) + fabsf(act[1]) + fabsf(act[2]) + fabsf(act[3]);
    r = r - (float)(0.00035 * MOTORS_TORQUE) * energy;
    const double min_height = TERRAIN_HEIGHT + LEG_H * 1.5, critical_height = TERRAIN_HEIGHT + LEG_H * 1.2;
    if (hull_y < min_height) r = r - (float)(10.0 * (min_height - hull_y));
    double vel_x = (double)row[2];
    if (vel_x > 0.0) r = r + (float)(3.0 * vel_x);
    else r = r - (float)(5.0 * ::fabs(vel_x));
    bool terminated = false;
    if (hull_y < critical_height) { r = -50.0f; terminated = true; }
    if (M[META_GAME_OVER] > 0.5f) { r = -100.0f; terminated = true; }
    if (hull_x < 0.0) { r = -100.0f; terminated = true; }
    const double terrain_end = (double)(TERRAIN_LENGTH - TERRAIN_GRASS) * TERRAIN_STEP;
    if (hull_x > terrain_end) terminated = true;
    if (step_count >= 2000) terminated = true;
    M[META_STEP] = (float)step_count;
    M[META_PREV_SHAPING] = new_shaping;
    M[META_DONE] = terminated ? 1.0f : 0.0f;
    reward = r;
    done = terminated ? 1.0f : 0.0f;
}

template <bool LIDAR = true>
MRL_DEV void step_row(float *row, float *contacts, const float *shapes, int env, const float *action,
                      float &reward, float &done) {
    (void)env;
    float act[ACT];
    step_motors(row, action, act);
    step_finish<LIDAR>(row, contacts, -1, shapes, act, reward, done);
}
}  // namespace bw

// ================================================================ HalfCheetah
namespace hc {
using L = HalfCheetahLayout;

// torso(0) - thigh - shin - foot for the back (1,2,3) and front (4,5,6) legs: reset_row below
struct Topology {
    static constexpr bool STATIC = true;
    static constexpr MRL_DEV int a(int j) { return (j == 0 || j == 3) ? 0 : j; }
    static constexpr MRL_DEV int b(int j) { return j + 1; }
};
constexpr int STATE = L::STATE_SIZE, OBS = 17, ACT = 6, NSHAPE_FLOATS = 7 * SHAPE_SIZE;
enum { META_STEP = 0, META_PREV_X = 1, META_PREV_SHAPING = 2, META_DONE = 3, META_TOTAL = 4 };
__device__ constexpr double LEN[7] = {1.0, 0.145, 0.15, 0.094, 0.133, 0.106, 0.07};
__device__ constexpr double MASS[7] = {6.25, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0};
__device__ constexpr double LIM[6][2] = {{-0.52, 1.05}, {-0.785, 0.785}, {-0.4, 0.785},
                                         {-1.0, 0.7},   {-1.2, 0.87},    {-0.5, 0.5}};

struct Shapes { float v[NSHAPE_FLOATS]; };
inline Shapes make_shapes() {
    const double len[7] = {1.0, 0.145, 0.15, 0.094, 0.133, 0.106, 0.07};
    Shapes s{};
    rect_shape(s.v, 1.0 / 2, 0.046, 1);
    for (int k = 1; k < 7; ++k) rect_shape(s.v + 20 * k, 0.046, len[k] / 2, 1);
    return s;
}

MRL_DEV void observe(float *row) {
    const float *B = row + L::BODIES_OFF;
    auto ang = [&](int b) { return (double)B[b * BODY_SIZE + IDX_ANGLE]; };
    auto omg = [&](int b) { return (double)B[b * BODY_SIZE + IDX_OMEGA]; };
    float o[OBS];
    o[0] = B[IDX_Y]; o[1] = B[IDX_ANGLE];
    o[2] = (float)(ang(1) - ang(0)); o[3] = (float)(ang(2) - ang(1)); o[4] = (float)(ang(3) - ang(2));
    o[5] = (float)(ang(4) - ang(0)); o[6] = (float)(ang(5) - ang(4)); o[7] = (float)(ang(6) - ang(5));
    o[8] = B[IDX_VX]; o[9] = B[IDX_VY]; o[10] = B[IDX_OMEGA];
    o[11] = (float)(omg(1) - omg(0)); o[12] = (float)(omg(2) - omg(1)); o[13] = (float)(omg(3) - omg(2));
    o[14] = (float)(omg(4) - omg(0)); o[15] = (float)(omg(5) - omg(4)); o[16] = (float)(omg(6) - omg(5));
#pragma unroll
    for (int k = 0; k < OBS; ++k) row[k] = o[k];
}

MRL_DEV void reset_row(float *row, uint64_t cseed) {
    for (int k = 0; k < STATE; ++k) row[k] = 0.0f;
    Uniform4 rv = philox_uniform4(cseed, 0, 0);
    const double init_x = 0.0, init_y = 0.7;
    const double init_vx = ((double)rv.v[0] * 2.0 - 1.0) * 0.1, init_vy = ((double)rv.v[1] * 2.0 - 1.0) * 0.1;
    float *B = row + L::BODIES_OFF;
    w_set_body(B, init_x, init_y, init_vx, init_vy, 1.0 / MASS[0], 1.0 / (MASS[0] * 1.0 * 1.0 / 12.0), 0);
    for (int leg = 0; leg < 2; ++leg) {
        const double hip_x = leg == 0 ? init_x - 1.0 / 2 : init_x + 1.0 / 2;
        const int b0 = 1 + 3 * leg;
        const double tl = LEN[b0], sl = LEN[b0 + 1], fl = LEN[b0 + 2];
        const double ys[3] = {init_y - tl / 2, init_y - tl - sl / 2, init_y - tl - sl - fl / 2};
        for (int k = 0; k < 3; ++k) {
            const double len = LEN[b0 + k], m = MASS[b0 + k];
            w_set_body(B + (b0 + k) * BODY_SIZE, hip_x, ys[k], init_vx, init_vy, 1.0 / m,
                       1.0 / (m * len * len / 12.0), b0 + k);
        }
    }
    row[L::JOINT_COUNT_OFF] = 6.0f;
    float *J = row + L::JOINTS_OFF;
    w_set_motor_joint(J + 0 * JOINT_SIZE, 0, 1, -1.0 / 2, 0.0, 0.0, LEN[1] / 2, LIM[0][0], LIM[0][1], 1.0);
    w_set_motor_joint(J + 1 * JOINT_SIZE, 1, 2, 0.0, -LEN[1] / 2, 0.0, LEN[2] / 2, LIM[1][0], LIM[1][1], 1.0);
    w_set_motor_joint(J + 2 * JOINT_SIZE, 2, 3, 0.0, -LEN[2] / 2, 0.0, LEN[3] / 2, LIM[2][0], LIM[2][1], 1.0);
    w_set_motor_joint(J + 3 * JOINT_SIZE, 0, 4, 1.0 / 2, 0.0, 0.0, LEN[4] / 2, LIM[3][0], LIM[3][1], 1.0);
    w_set_motor_joint(J + 4 * JOINT_SIZE, 4, 5, 0.0, -LEN[4] / 2, 0.0, LEN[5] / 2, LIM[4][0], LIM[4][1], 1.0);
    w_set_motor_joint(J + 5 * JOINT_SIZE, 5, 6, 0.0, -LEN[5] / 2, 0.0, LEN[6] / 2, LIM[5][0], LIM[5][1], 1.0);
    row[L::META_OFF + META_PREV_X] = (float)init_x;
    observe(row);
}

MRL_DEV void step_row(float *row, float *contacts, const float *shapes, int env, const float *action,
                      float &reward, float &done) {
    (void)env;
    double a[ACT];
#pragma unroll
    for (int j = 0; j < ACT; ++j) {
        float v = action[j];
        v = v < 1.0f ? v : 1.0f;
        v = v > -1.0f ? v : -1.0f;
        a[j] = (double)v;
        float *J = row + L::JOINTS_OFF + j * JOINT_SIZE;
        J[J_MOTOR_SPEED] = (a[j] >= 0.0 ? 1.0f : -1.0f) * 1000.0f;
        J[J_MAX_TORQUE] = (float)(1.0 * ::fabs(a[j]));
    }
    float *B = row + L::BODIES_OFF;
    const double x_before = B[IDX_X];
    int n = 0;
    for (int s = 0; s < 5; ++s)
        n = reg_physics_substep<L, Topology, true, false>(row, shapes, contacts, (float)0.0, (float)-9.81, (float)0.01, (float)0.9,
                                     (float)0.0, (float)0.2, (float)0.005, 4, 2);
    const double x_after = B[IDX_X], torso_z = B[IDX_Y];
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
    double penalty = 0.0;
    for (int c = 0; c < n; ++c) {
        int ba = (int)contacts[c * CONTACT_SIZE + C_BODY_A], bb = (int)contacts[c * CONTACT_SIZE + C_BODY_B];
        if (bb == -1 && ba != 3 && ba != 6) penalty += 0.5;
    }
    const double r = forward_reward - ctrl_cost + height_bonus - penalty;
    float *M = row + L::META_OFF;
    const int step_count = (int)M[META_STEP] + 1;
    M[META_STEP] = (float)step_count;
    M[META_PREV_X] = (float)x_after;
    M[META_TOTAL] = (float)((double)M[META_TOTAL] + r);
    const bool d = step_count >= 1000;
    M[META_DONE] = d ? 1.0f : 0.0f;
    observe(row);
    reward = (float)r;
    done = d ? 1.0f : 0.0f;
}
}  // namespace hc

}  // namespace mrl
