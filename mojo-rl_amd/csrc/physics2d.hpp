// physics2d on one environment row, one lane per environment.
//
// `row` points at this lane's copy of the reference's flat env row
// (physics2d/layout.mojo:58-126): [obs | bodies NB*13 | forces NB*3 | joints NJ*17 |
// joint_count | edges NE*6 | edge_count | metadata].  In the step kernels the row lives in
// LDS (staged there with coalesced loads, lane stride odd so that lanes hit distinct
// banks); `contacts` is this lane's [MAX_CONTACTS][9] scratch, also in LDS.
//
// This file: the row layout, contact detection against the terrain (collision/edge_terrain.mojo:
// 174-408, collision/flat_terrain.mojo:69-204) and the lidar ray test (lidar/lidar.mojo:25-141),
// arithmetic as in the CPU statement of the reference line by line.  The integrators and the
// Gauss-Seidel sweeps (integrators/euler.mojo, solvers/impulse.mojo, joints/revolute.mojo) run on
// registers: physics2d_reg.hpp.
#pragma once
#include "mrl_device.hpp"

namespace mrl {

enum {
    BODY_SIZE = 13, IDX_X = 0, IDX_Y = 1, IDX_ANGLE = 2, IDX_VX = 3, IDX_VY = 4, IDX_OMEGA = 5,
    IDX_FX = 6, IDX_FY = 7, IDX_TAU = 8, IDX_MASS = 9, IDX_INV_MASS = 10, IDX_INV_INERTIA = 11,
    IDX_SHAPE = 12,
    SHAPE_SIZE = 20, SHAPE_POLYGON = 0, SHAPE_CIRCLE = 1, MAX_POLY_VERTS = 8,
    CONTACT_SIZE = 9, C_BODY_A = 0, C_BODY_B = 1, C_PX = 2, C_PY = 3, C_NX = 4, C_NY = 5,
    C_DEPTH = 6, C_JN = 7, C_JT = 8,
    JOINT_SIZE = 17, J_TYPE = 0, J_BODY_A = 1, J_BODY_B = 2, J_AX = 3, J_AY = 4, J_BX = 5,
    J_BY = 6, J_REF = 7, J_LO = 8, J_HI = 9, J_MAX_TORQUE = 10, J_MOTOR_SPEED = 11, J_STIFF = 12,
    J_DAMP = 13, J_FLAGS = 14, J_IMPULSE = 15, J_MOTOR_IMPULSE = 16,
    JF_LIMIT = 1, JF_MOTOR = 2, JF_SPRING = 4
};

template <int NB, int MC, int MJ, int ME, int OBS, int META, int NS>
struct Layout {
    static constexpr int NUM_BODIES = NB, MAX_CONTACTS = MC, MAX_JOINTS = MJ, MAX_EDGES = ME,
                         OBS_DIM = OBS, META_SIZE = META, NUM_SHAPES = NS;
    static constexpr int BODIES_OFF = OBS;
    static constexpr int FORCES_OFF = BODIES_OFF + NB * BODY_SIZE;
    static constexpr int JOINTS_OFF = FORCES_OFF + NB * 3;
    static constexpr int JOINT_COUNT_OFF = JOINTS_OFF + MJ * JOINT_SIZE;
    static constexpr int EDGES_OFF = JOINT_COUNT_OFF + 1;
    static constexpr int EDGE_COUNT_OFF = EDGES_OFF + ME * 6;
    static constexpr int META_OFF = EDGE_COUNT_OFF + 1;
    static constexpr int STATE_SIZE = META_OFF + META;
};

using LunarLanderLayout = Layout<3, 8, 2, 16, 8, 4, 3>;      // physics2d/layout.mojo:247-255
using BipedalWalkerLayout = Layout<5, 20, 4, 128, 24, 8, 5>; // :280-288
using HalfCheetahLayout = Layout<7, 14, 6, 2, 17, 8, 7>;     // :291-299

MRL_DEV void put_contact(float *c, int body, float px, float py, float nx, float ny, float depth) {
    c[C_BODY_A] = (float)body; c[C_BODY_B] = -1.0f;
    c[C_PX] = px; c[C_PY] = py; c[C_NX] = nx; c[C_NY] = ny;
    c[C_DEPTH] = depth; c[C_JN] = 0.0f; c[C_JT] = 0.0f;
}

// One vertex against one terrain edge whose x range it already passed.
MRL_DEV void vertex_edge_test(const float *E, int b, float world_x, float world_y, float *contacts,
                              int &count, int max_contacts) {
    float e_x0 = E[0], e_x1 = E[2];
    float e_y0 = E[1], e_y1 = E[3], e_nx = E[4], e_ny = E[5];
    float edge_dx = e_x1 - e_x0, edge_dy = e_y1 - e_y0;
    float edge_len_sq = edge_dx * edge_dx + edge_dy * edge_dy;
    if (edge_len_sq < 1e-6f) return;
    float t = ((world_x - e_x0) * edge_dx + (world_y - e_y0) * edge_dy) / edge_len_sq;
    if (t < 0.0f) t = 0.0f;
    if (t > 1.0f) t = 1.0f;
    float closest_x = e_x0 + t * edge_dx, closest_y = e_y0 + t * edge_dy;
    float dist_x = world_x - closest_x, dist_y = world_y - closest_y;
    float penetration = -(dist_x * e_nx + dist_y * e_ny);
    if (penetration > 0.0f && count < max_contacts) {
        put_contact(contacts + count * CONTACT_SIZE, b, world_x, world_y, e_nx, e_ny, penetration);
        count += 1;
    }
}

// true when the vertex passes the x-range pre-check of collision/edge_terrain.mojo:236-249
MRL_DEV bool edge_x_pass(float e_x0, float e_x1, float world_x) {
    const float margin = 0.1f;
    float x_min = e_x0 - margin, x_max = e_x1 + margin;
    if (e_x0 > e_x1) { x_min = e_x1 - margin; x_max = e_x0 + margin; }
    return !(world_x < x_min || world_x > x_max);
}

// bits [0, n) of a 32-bit word, n clamped to [0, 32]: the edges of mask word q that exist are
// word_bits(n_edges - 32 q)
MRL_DEV unsigned word_bits(int n) { return n >= 32 ? 0xffffffffu : (n <= 0 ? 0u : (1u << n) - 1u); }

// Bit e of a mask is set when terrain edge e can matter for an x interval.
template <class L>
struct EdgeMask {
    static constexpr int WORDS = (L::MAX_EDGES + 31) / 32;
    unsigned w[WORDS];
};

// Edges whose x-range pre-check (edge_x_pass) can succeed for some x in [xlo, xhi]: a superset of
// the edges any such vertex passes, decided with the same fp32 bounds the pre-check uses.
// widen = 0 gives exactly that; lidar passes its own safety margin on top.  Only the mask words
// [q0, q1) are worked out (a caller that splits the edges over several lanes); the rest is zero.
MRL_DEV bool edge_near(const float *E, float xlo, float xhi, float widen) {
    const float e_x0 = E[0], e_x1 = E[2];
    const float margin = 0.1f;
    float x_min = e_x0 - margin, x_max = e_x1 + margin;
    if (e_x0 > e_x1) { x_min = e_x1 - margin; x_max = e_x0 + margin; }
    return !(xhi < x_min - widen || xlo > x_max + widen);
}

// bits 0 .. N - 1: the mask bits of edges e0 .. e0 + N - 1 (a caller that spreads one mask over many lanes)
template <class L, int N>
MRL_DEV unsigned edges_near_bits(const float *row, float xlo, float xhi, float widen, int e0) {
    int n_edges = (int)row[L::EDGE_COUNT_OFF];
    if (n_edges > L::MAX_EDGES) n_edges = L::MAX_EDGES;
    const float *edges = row + L::EDGES_OFF;
    unsigned bits = 0;
#pragma unroll
    for (int k = 0; k < N; ++k)
        bits |= (unsigned)(e0 + k < n_edges && edge_near(edges + (e0 + k) * 6, xlo, xhi, widen)) << k;
    return bits;
}

// Slots 18 and 19 of a polygon shape (past its eight vertices) may hold max |x| and max |y| over its
// local vertices; a table whose shapes all carry them lets bodies_x_interval bound an env's vertices
// without visiting them.
constexpr int SHAPE_BOUND_X = 18, SHAPE_BOUND_Y = 19;
static_assert(2 + 2 * MAX_POLY_VERTS <= SHAPE_BOUND_X && SHAPE_BOUND_Y < SHAPE_SIZE, "free slots of a shape");
inline void shape_set_bounds(float *S) {
    float bx = 0.0f, by = 0.0f;
    for (int v = 0; v < (int)S[1] && v < MAX_POLY_VERTS; ++v) {
        const float ax = S[2 + 2 * v] < 0.0f ? -S[2 + 2 * v] : S[2 + 2 * v];
        const float ay = S[3 + 2 * v] < 0.0f ? -S[3 + 2 * v] : S[3 + 2 * v];
        bx = ax > bx ? ax : bx;
        by = ay > by ? ay : by;
    }
    S[SHAPE_BOUND_X] = bx;
    S[SHAPE_BOUND_Y] = by;
}

// An x interval that holds every polygon vertex of the row's bodies.  A vertex sits at
// fl(fl(x + fl(lx cos)) - fl(ly sin)); |fl(lx cos)| <= max |lx| and |fl(ly sin)| <= max |ly| (sine and
// cosine are at most 1 and rounding is monotone), so the same two additions with the bounds in
// place of the products enclose it, again because rounding is monotone.  A NaN centre gives the
// whole axis (a NaN coordinate passes the pre-check of every edge).
template <class L>
MRL_DEV void bodies_x_interval(const float *row, const float *shapes, float &xlo, float &xhi) {
    xlo = 3.0e38f; xhi = -3.0e38f;
    bool odd = false;
#pragma unroll
    for (int b = 0; b < L::NUM_BODIES; ++b) {
        const float *B = row + L::BODIES_OFF + b * BODY_SIZE;
        const float *S = shapes + (int)B[IDX_SHAPE] * SHAPE_SIZE;
        const float x = B[IDX_X], lo = (x - S[SHAPE_BOUND_X]) - S[SHAPE_BOUND_Y], hi = (x + S[SHAPE_BOUND_X]) + S[SHAPE_BOUND_Y];
        odd = odd || !(lo == lo) || !(hi == hi);
        xlo = lo < xlo ? lo : xlo;
        xhi = hi > xhi ? hi : xhi;
    }
    if (odd) { xlo = -3.0e38f; xhi = 3.0e38f; }
}

template <class L>
MRL_DEV void edges_near(const float *row, float xlo, float xhi, float widen, EdgeMask<L> &m, int q0 = 0,
                        int q1 = EdgeMask<L>::WORDS) {
    int n_edges = (int)row[L::EDGE_COUNT_OFF];
    if (n_edges > L::MAX_EDGES) n_edges = L::MAX_EDGES;
    const float *edges = row + L::EDGES_OFF;
#pragma unroll
    for (int q = 0; q < EdgeMask<L>::WORDS; ++q) {
        if (q < q0 || q >= q1) { m.w[q] = 0; continue; }
        // every slot of the word is tested, whether the edge exists or not (the slots are inside the
        // row), and the word is cut to the existing edges afterwards: no test depends on n_edges, so
        // the loads of a round go out together instead of one by one behind a branch each
        unsigned bits = 0;
        const int e0 = q * 32;
#pragma unroll 1
        for (int k0 = 0; k0 < 32; k0 += 8) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int k = k0 + j, e = e0 + k;
                if (e >= L::MAX_EDGES) continue;
                bits |= (unsigned)edge_near(edges + e * 6, xlo, xhi, widen) << k;
            }
        }
        m.w[q] = bits & word_bits(n_edges - e0);
    }
}

// vertex / circle against the row's terrain polyline; contacts in (body, vertex, edge) order.
//
// The x-range pre-check rejects almost every (vertex, edge) pair, but which pairs survive differs
// from lane to lane, so a plain loop over the edges makes the wavefront run the full test for the
// union of all lanes' survivors.  Instead each lane first collects its survivors of up to 32 edges
// in a bit mask (cheap, no divergence), then all lanes walk their own masks together: the
// wavefront runs the full test max-over-lanes(popcount) times.  Edges are visited in ascending
// order per lane, so the contact list is the same.
template <class L>
MRL_DEV int edge_detect(const float *row, const float *shapes, float *contacts) {
    int count = 0;
    int n_edges = (int)row[L::EDGE_COUNT_OFF];
    const float *edges = row + L::EDGES_OFF;
    constexpr bool SMALL = L::MAX_EDGES <= 16;     // edge x ranges fit in registers
    constexpr int NR = SMALL ? L::MAX_EDGES : 1;
    float ex0[NR], ex1[NR];
    if (SMALL) {
#pragma unroll
        for (int e = 0; e < NR; ++e) {
            ex0[e] = edges[e * 6];
            ex1[e] = edges[e * 6 + 2];
        }
    }
    // long polylines: one pass over the edges picks those near the env's polygon vertices at all
    // (x interval of every vertex of every body); the per-vertex loops then visit only these
    float sins[L::NUM_BODIES], coss[L::NUM_BODIES];
#pragma unroll
    for (int b = 0; b < L::NUM_BODIES; ++b) sincos32(row[L::BODIES_OFF + b * BODY_SIZE + IDX_ANGLE], sins[b], coss[b]);
    EdgeMask<L> near;
    if (!SMALL) {
        float xlo = 3.0e38f, xhi = -3.0e38f;
        bool odd = false;   // a NaN coordinate passes the pre-check of every edge
#pragma unroll
        for (int b = 0; b < L::NUM_BODIES; ++b) {
            const float *B = row + L::BODIES_OFF + b * BODY_SIZE;
            const float *S = shapes + (int)B[IDX_SHAPE] * SHAPE_SIZE;
            if ((int)S[0] != SHAPE_POLYGON) continue;
            int n_verts = (int)S[1];
            if (n_verts > MAX_POLY_VERTS) n_verts = MAX_POLY_VERTS;
            for (int v = 0; v < n_verts; ++v) {
                const float world_x = B[IDX_X] + S[2 + v * 2] * coss[b] - S[3 + v * 2] * sins[b];
                odd = odd || !(world_x == world_x);
                xlo = world_x < xlo ? world_x : xlo;
                xhi = world_x > xhi ? world_x : xhi;
            }
        }
        if (odd) { xlo = -3.0e38f; xhi = 3.0e38f; }
        edges_near<L>(row, xlo, xhi, 0.0f, near);
    }
#pragma unroll
    for (int b = 0; b < L::NUM_BODIES; ++b) {
        const float *B = row + L::BODIES_OFF + b * BODY_SIZE;
        float body_x = B[IDX_X], body_y = B[IDX_Y];
        const float *S = shapes + (int)B[IDX_SHAPE] * SHAPE_SIZE;
        int shape_type = (int)S[0];
        const float sin_a = sins[b], cos_a = coss[b];
        if (shape_type == SHAPE_POLYGON) {
            int n_verts = (int)S[1];
            if (n_verts > MAX_POLY_VERTS) n_verts = MAX_POLY_VERTS;
            for (int v = 0; v < n_verts; ++v) {
                float local_x = S[2 + v * 2], local_y = S[3 + v * 2];
                float world_x = body_x + local_x * cos_a - local_y * sin_a;
                float world_y = body_y + local_x * sin_a + local_y * cos_a;
                if (SMALL) {
                    unsigned mask = 0;
#pragma unroll
                    for (int e = 0; e < NR; ++e)
                        if (e < n_edges && edge_x_pass(ex0[e], ex1[e], world_x)) mask |= 1u << e;
                    while (mask) {
                        const int e = __ffs((int)mask) - 1;
                        mask &= mask - 1;
                        vertex_edge_test(edges + e * 6, b, world_x, world_y, contacts, count,
                                         L::MAX_CONTACTS);
                    }
                } else {
#pragma unroll
                    for (int q = 0; q < EdgeMask<L>::WORDS; ++q) {
                        unsigned mask = near.w[q];
                        while (mask) {
                            const int e = q * 32 + __ffs((int)mask) - 1;
                            mask &= mask - 1;
                            const float *E = edges + e * 6;
                            if (edge_x_pass(E[0], E[2], world_x))
                                vertex_edge_test(E, b, world_x, world_y, contacts, count, L::MAX_CONTACTS);
                        }
                    }
                }
            }
        } else if (shape_type == SHAPE_CIRCLE) {
            float radius = S[1], cox = S[2], coy = S[3];
            float cwx = body_x + cox * cos_a - coy * sin_a;
            float cwy = body_y + cox * sin_a + coy * cos_a;
            for (int e = 0; e < n_edges; ++e) {
                const float *E = edges + e * 6;
                float e_x0 = E[0], e_y0 = E[1], e_x1 = E[2], e_y1 = E[3], e_nx = E[4], e_ny = E[5];
                float edge_dx = e_x1 - e_x0, edge_dy = e_y1 - e_y0;
                float edge_len_sq = edge_dx * edge_dx + edge_dy * edge_dy;
                if (edge_len_sq < 1e-6f) continue;
                float t = ((cwx - e_x0) * edge_dx + (cwy - e_y0) * edge_dy) / edge_len_sq;
                if (t < 0.0f) t = 0.0f;
                if (t > 1.0f) t = 1.0f;
                float closest_x = e_x0 + t * edge_dx, closest_y = e_y0 + t * edge_dy;
                float dist_x = cwx - closest_x, dist_y = cwy - closest_y;
                float dist = sqrtf(dist_x * dist_x + dist_y * dist_y);
                float penetration = radius - dist;
                if (penetration > 0.0f && count < L::MAX_CONTACTS) {
                    float cnx = e_nx, cny = e_ny;
                    if (dist > 1e-6f) { cnx = dist_x / dist; cny = dist_y / dist; }
                    put_contact(contacts + count * CONTACT_SIZE, b, closest_x, closest_y, cnx, cny,
                                penetration);
                    count += 1;
                }
            }
        }
    }
    return count;
}

// edge_detect restricted to vertex v of body b, for callers that spread the vertices of an env over
// many lanes: the contacts that vertex contributes, in edge order, counted from zero; concatenating
// the lists in (body, vertex) order and cutting at MAX_CONTACTS reproduces edge_detect.  Returns
// -1 when the caller has to fall back to edge_detect: the body is not a polygon of at most
// max_verts vertices (the caller planned one lane per vertex for that many), or the vertex
// touched `cap` edges or more (the list holds cap records; the last one only signals overflow).
// near != nullptr: the mask words of the edges whose pre-check can pass for some vertex of the env
// (edges_near_bits over bodies_x_interval), worked out once for all its vertices.
template <class L>
MRL_DEV int edge_detect_vertex(const float *row, const float *shapes, int b, int v, int max_verts,
                               float *contacts, int cap, const unsigned *near = nullptr) {
    const float *B = row + L::BODIES_OFF + b * BODY_SIZE;
    const float *S = shapes + (int)B[IDX_SHAPE] * SHAPE_SIZE;
    int n_verts = (int)S[1];
    if (n_verts > MAX_POLY_VERTS) n_verts = MAX_POLY_VERTS;
    if ((int)S[0] != SHAPE_POLYGON || n_verts > max_verts) return -1;
    if (v >= n_verts) return 0;
    int n_edges = (int)row[L::EDGE_COUNT_OFF];
    const float *edges = row + L::EDGES_OFF;
    float sin_a, cos_a;
    sincos32(B[IDX_ANGLE], sin_a, cos_a);
    const float local_x = S[2 + v * 2], local_y = S[3 + v * 2];
    const float world_x = B[IDX_X] + local_x * cos_a - local_y * sin_a;
    const float world_y = B[IDX_Y] + local_x * sin_a + local_y * cos_a;
    // the x-range pre-check of 32 edges at a time into a bit mask, then the full test of the
    // survivors in ascending order (the order edge_detect visits them in)
    int count = 0;
#pragma unroll
    for (int q = 0; q < (L::MAX_EDGES + 31) / 32; ++q) {
        // (all slots tested, the word cut to the existing edges afterwards: see edges_near)
        unsigned mask = 0;
        if (near != nullptr) {
            // only the edges the caller found near the env's bodies at all; the vertex's own
            // survivors are picked first, so that lanes with unequal sets share the full tests
            unsigned cand = near[q];
            while (cand) {
                const int k = __ffs((int)cand) - 1;
                cand &= cand - 1;
                const int e = q * 32 + k;
                if (edge_x_pass(edges[e * 6], edges[e * 6 + 2], world_x)) mask |= 1u << k;
            }
        } else {
#pragma unroll
            for (int k = 0; k < 32; ++k) {
                const int e = q * 32 + k;
                if (e < L::MAX_EDGES) mask |= (unsigned)edge_x_pass(edges[e * 6], edges[e * 6 + 2], world_x) << k;
            }
        }
        mask &= word_bits(n_edges - q * 32);
        while (mask) {
            const int e = q * 32 + __ffs((int)mask) - 1;
            mask &= mask - 1;
            vertex_edge_test(edges + e * 6, b, world_x, world_y, contacts, count, cap);
        }
    }
    return count >= cap ? -1 : count;
}

template <class L>
MRL_DEV int flat_detect(const float *row, const float *shapes, float ground_y, float *contacts) {
    int count = 0;
    for (int b = 0; b < L::NUM_BODIES; ++b) {
        const float *B = row + L::BODIES_OFF + b * BODY_SIZE;
        float body_x = B[IDX_X], body_y = B[IDX_Y];
        const float *S = shapes + (int)B[IDX_SHAPE] * SHAPE_SIZE;
        int shape_type = (int)S[0];
        float sin_a, cos_a;
        sincos32(B[IDX_ANGLE], sin_a, cos_a);
        if (shape_type == SHAPE_POLYGON) {
            int n_verts = (int)S[1];
            if (n_verts > MAX_POLY_VERTS) n_verts = MAX_POLY_VERTS;
            for (int v = 0; v < n_verts; ++v) {
                float local_x = S[2 + v * 2], local_y = S[3 + v * 2];
                float world_x = body_x + local_x * cos_a - local_y * sin_a;
                float world_y = body_y + local_x * sin_a + local_y * cos_a;
                float penetration = ground_y - world_y;
                if (penetration > 0.0f && count < L::MAX_CONTACTS) {
                    put_contact(contacts + count * CONTACT_SIZE, b, world_x, world_y, 0.0f, 1.0f,
                                penetration);
                    count += 1;
                }
            }
        } else if (shape_type == SHAPE_CIRCLE) {
            float radius = S[1], cox = S[2], coy = S[3];
            float cwx = body_x + cox * cos_a - coy * sin_a;
            float cwy = body_y + cox * sin_a + coy * cos_a;
            float penetration = ground_y - (cwy - radius);
            if (penetration > 0.0f && count < L::MAX_CONTACTS) {
                put_contact(contacts + count * CONTACT_SIZE, b, cwx, cwy - radius, 0.0f, 1.0f,
                            penetration);
                count += 1;
            }
        }
    }
    return count;
}

// ray / edge test of physics2d/lidar/lidar.mojo:25-141 for one edge
MRL_DEV void lidar_edge(const float *E, float ox, float oy, float rdx, float rdy, float &min_t) {
    float ex = E[2] - E[0], ey = E[3] - E[1];
    float denom = rdx * ey - rdy * ex;
    if (denom > -1e-10f && denom < 1e-10f) return;
    float dx = ox - E[0], dy = oy - E[1];
    float t = (ex * dy - ey * dx) / denom;
    float u = (rdx * dy - rdy * dx) / denom;
    if (t >= 0.0f && t <= 1.0f && u >= 0.0f && u <= 1.0f && t < min_t) min_t = t;
}

template <class L>
MRL_DEV float lidar_ray(const float *row, float ox, float oy, float rdx, float rdy) {
    int n_edges = (int)row[L::EDGE_COUNT_OFF];
    if (n_edges > L::MAX_EDGES) n_edges = L::MAX_EDGES;
    float min_t = 1.0f;
    for (int e = 0; e < n_edges; ++e) lidar_edge(row + L::EDGES_OFF + e * 6, ox, oy, rdx, rdy, min_t);
    return min_t;
}

// Same result from a pre-selected edge set.  A hit needs a point common to the ray segment and the
// edge, so an edge whose x extent stays clear of the ray's x extent cannot hit; `near` must hold
// every edge within 0.01 of the ray's x extent (the tests t, u in [0, 1] are evaluated in fp32:
// the slack is orders of magnitude above their rounding error, and where the denominator is tiny
// a far-away edge yields |t| or |u| in the millions, never a value in [0, 1]).
template <class L>
MRL_DEV float lidar_ray_near(const float *row, const EdgeMask<L> &near, float ox, float oy, float rdx,
                             float rdy) {
    float min_t = 1.0f;
    const float ex_ = ox + rdx;
    const float rlo = (ox < ex_ ? ox : ex_) - 0.01f, rhi = (ox > ex_ ? ox : ex_) + 0.01f;
#pragma unroll
    for (int q = 0; q < EdgeMask<L>::WORDS; ++q) {
        unsigned mask = near.w[q];
        while (mask) {
            const int e = q * 32 + __ffs((int)mask) - 1;
            mask &= mask - 1;
            const float *E = row + L::EDGES_OFF + e * 6;
            const float x0 = E[0], x1 = E[2];
            const float elo = x0 < x1 ? x0 : x1, ehi = x0 < x1 ? x1 : x0;
            if (ehi < rlo || elo > rhi) continue;
            lidar_edge(E, ox, oy, rdx, rdy, min_t);
        }
    }
    return min_t;
}

// lidar_ray_near in two passes, for a caller that splits a ray's edges over several lanes: the
// candidates `cand` of mask word q that pass the x-extent test of lidar_ray_near ...
template <class L>
MRL_DEV unsigned lidar_ray_pick(const float *row, unsigned cand, int q, float ox, float rdx) {
    const float ex_ = ox + rdx;
    const float rlo = (ox < ex_ ? ox : ex_) - 0.01f, rhi = (ox > ex_ ? ox : ex_) + 0.01f;
    unsigned keep = 0;
    while (cand) {
        const int k = __ffs((int)cand) - 1;
        cand &= cand - 1;
        const float *E = row + L::EDGES_OFF + (q * 32 + k) * 6;
        const float x0 = E[0], x1 = E[2];
        const float elo = x0 < x1 ? x0 : x1, ehi = x0 < x1 ? x1 : x0;
        if (!(ehi < rlo || elo > rhi)) keep |= 1u << k;
    }
    return keep;
}
// ... and the ray against exactly those.  Lanes that walk unequal candidate sets together spend the
// intersection test only as often as the longest picked set asks, not once per candidate of any lane.
template <class L>
MRL_DEV float lidar_ray_picked(const float *row, const EdgeMask<L> &picked, float ox, float oy, float rdx,
                               float rdy) {
    float min_t = 1.0f;
#pragma unroll
    for (int q = 0; q < EdgeMask<L>::WORDS; ++q) {
        unsigned mask = picked.w[q];
        while (mask) {
            const int e = q * 32 + __ffs((int)mask) - 1;
            mask &= mask - 1;
            lidar_edge(row + L::EDGES_OFF + e * 6, ox, oy, rdx, rdy, min_t);
        }
    }
    return min_t;
}

}  // namespace mrl
