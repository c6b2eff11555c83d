/*
 * physics2d: CPU restatement on the per-env flat row (test infrastructure, never shipped).
 *
 *   layout                 physics2d/layout.mojo:58-126
 *   integrate_velocities   physics2d/integrators/euler.mojo:82-129
 *   integrate_positions    physics2d/integrators/euler.mojo:131-183 (CPU if/elif angle wrap)
 *   edge detect            physics2d/collision/edge_terrain.mojo:174-408
 *   terrain from heights   physics2d/collision/edge_terrain.mojo:93-147
 *   flat detect            physics2d/collision/flat_terrain.mojo:69-204
 *   contact velocity solve physics2d/solvers/impulse.mojo:94-331
 *   contact position solve physics2d/solvers/impulse.mojo:333-402
 *   joint velocity solve   physics2d/joints/revolute.mojo:69-320
 *   joint position solve   physics2d/joints/revolute.mojo:323-495
 *   lidar ray              physics2d/lidar/lidar.mojo:25-141
 *
 * The reference's CPU structs hold bodies / forces / joints as separate tensors that
 * alias the same [1, STATE_SIZE] row (physics2d/state.mojo:676-772); here they are
 * addressed through the row offsets directly.  Shapes and contacts are separate
 * buffers, as in the reference.
 */
#include <math.h>
#include "orc.h"

static inline float f32_sin(float x) { return (float)sin((double)x); }
static inline float f32_cos(float x) { return (float)cos((double)x); }

void orc_layout_make(orc_layout *L, int num_bodies, int max_contacts, int max_joints,
                     int max_edges, int obs_dim, int meta_size, int num_shapes) {
    L->num_bodies = num_bodies; L->max_contacts = max_contacts; L->max_joints = max_joints;
    L->max_edges = max_edges; L->obs_dim = obs_dim; L->meta_size = meta_size;
    L->num_shapes = num_shapes;
    L->bodies_off = obs_dim;
    L->forces_off = L->bodies_off + num_bodies * ORC_BODY_SIZE;
    L->joints_off = L->forces_off + num_bodies * 3;
    L->joint_count_off = L->joints_off + max_joints * ORC_JOINT_SIZE;
    L->edges_off = L->joint_count_off + 1;
    L->edge_count_off = L->edges_off + max_edges * 6;
    L->meta_off = L->edge_count_off + 1;
    L->state_size = L->meta_off + meta_size;
}

#define BODY(b) (row + L->bodies_off + (b) * ORC_BODY_SIZE)

void orc_integrate_velocities(const orc_layout *L, float *row, float gx, float gy, float dt) {
    for (int b = 0; b < L->num_bodies; ++b) {
        float *B = BODY(b);
        float inv_mass = B[ORC_IDX_INV_MASS], inv_inertia = B[ORC_IDX_INV_INERTIA];
        if (inv_mass == 0.0f) continue;
        const float *F = row + L->forces_off + b * 3;
        float vx = B[ORC_IDX_VX], vy = B[ORC_IDX_VY], omega = B[ORC_IDX_OMEGA];
        vx = vx + (F[0] * inv_mass + gx) * dt;
        vy = vy + (F[1] * inv_mass + gy) * dt;
        omega = omega + F[2] * inv_inertia * dt;
        B[ORC_IDX_VX] = vx; B[ORC_IDX_VY] = vy; B[ORC_IDX_OMEGA] = omega;
    }
}

void orc_integrate_positions(const orc_layout *L, float *row, float dt) {
    const float pi_val = (float)3.14159265358979323846;
    const float two_pi = (float)(2.0 * 3.14159265358979323846);
    for (int b = 0; b < L->num_bodies; ++b) {
        float *B = BODY(b);
        if (B[ORC_IDX_INV_MASS] == 0.0f) continue;
        float x = B[ORC_IDX_X] + B[ORC_IDX_VX] * dt;
        float y = B[ORC_IDX_Y] + B[ORC_IDX_VY] * dt;
        float angle = B[ORC_IDX_ANGLE] + B[ORC_IDX_OMEGA] * dt;
        if (angle > 100.0f || angle < -100.0f) {
            angle = 0.0f;
        } else if (angle > pi_val) {
            angle = angle - two_pi;
            if (angle > pi_val) angle = angle - two_pi;
        } else if (angle < -pi_val) {
            angle = angle + two_pi;
            if (angle < -pi_val) angle = angle + two_pi;
        }
        B[ORC_IDX_X] = x; B[ORC_IDX_Y] = y; B[ORC_IDX_ANGLE] = angle;
    }
}

static inline void put_contact(float *c, int body, float px, float py, float nx, float ny,
                               float depth) {
    c[ORC_C_BODY_A] = (float)body; c[ORC_C_BODY_B] = -1.0f;
    c[ORC_C_PX] = px; c[ORC_C_PY] = py; c[ORC_C_NX] = nx; c[ORC_C_NY] = ny;
    c[ORC_C_DEPTH] = depth; c[ORC_C_JN] = 0.0f; c[ORC_C_JT] = 0.0f;
}

int orc_edge_detect(const orc_layout *L, const float *row, const float *shapes, float *contacts) {
    int count = 0;
    int n_edges = (int)row[L->edge_count_off];
    const float *edges = row + L->edges_off;
    for (int b = 0; b < L->num_bodies; ++b) {
        const float *B = row + L->bodies_off + b * ORC_BODY_SIZE;
        float body_x = B[ORC_IDX_X], body_y = B[ORC_IDX_Y], body_angle = B[ORC_IDX_ANGLE];
        int shape_idx = (int)B[ORC_IDX_SHAPE];
        const float *S = shapes + shape_idx * ORC_SHAPE_SIZE;
        int shape_type = (int)S[0];
        float cos_a = f32_cos(body_angle), sin_a = f32_sin(body_angle);
        if (shape_type == ORC_SHAPE_POLYGON) {
            int n_verts = (int)S[1];
            for (int v = 0; v < n_verts; ++v) {
                if (v >= ORC_MAX_POLY_VERTS) break;
                float local_x = S[2 + v * 2], local_y = S[3 + v * 2];
                float world_x = body_x + local_x * cos_a - local_y * sin_a;
                float world_y = body_y + local_x * sin_a + local_y * cos_a;
                for (int e = 0; e < n_edges; ++e) {
                    const float *E = edges + e * 6;
                    float e_x0 = E[0], e_y0 = E[1], e_x1 = E[2], e_y1 = E[3], e_nx = E[4], e_ny = E[5];
                    const float margin = 0.1f;
                    float x_min = e_x0 - margin, x_max = e_x1 + margin;
                    if (e_x0 > e_x1) { x_min = e_x1 - margin; x_max = e_x0 + margin; }
                    if (world_x < x_min || world_x > x_max) continue;
                    float edge_dx = e_x1 - e_x0, edge_dy = e_y1 - e_y0;
                    float edge_len_sq = edge_dx * edge_dx + edge_dy * edge_dy;
                    if (edge_len_sq < 1e-6f) continue;
                    float t = ((world_x - e_x0) * edge_dx + (world_y - e_y0) * edge_dy) / edge_len_sq;
                    if (t < 0.0f) t = 0.0f;
                    if (t > 1.0f) t = 1.0f;
                    float closest_x = e_x0 + t * edge_dx, closest_y = e_y0 + t * edge_dy;
                    float dist_x = world_x - closest_x, dist_y = world_y - closest_y;
                    float penetration = -(dist_x * e_nx + dist_y * e_ny);
                    if (penetration > 0.0f && count < L->max_contacts) {
                        put_contact(contacts + count * ORC_CONTACT_SIZE, b, world_x, world_y, e_nx,
                                    e_ny, penetration);
                        count += 1;
                    }
                }
            }
        } else if (shape_type == ORC_SHAPE_CIRCLE) {
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
                if (penetration > 0.0f && count < L->max_contacts) {
                    float cnx = e_nx, cny = e_ny;
                    if (dist > 1e-6f) { cnx = dist_x / dist; cny = dist_y / dist; }
                    put_contact(contacts + count * ORC_CONTACT_SIZE, b, closest_x, closest_y, cnx,
                                cny, penetration);
                    count += 1;
                }
            }
        }
    }
    return count;
}

void orc_set_terrain_from_heights(const orc_layout *L, float *row, const float *heights,
                                  int n_points, double x_start, double x_spacing) {
    int n_edges = n_points - 1;
    if (n_edges > L->max_edges) n_edges = L->max_edges;
    row[L->edge_count_off] = (float)n_edges;
    for (int i = 0; i < n_edges; ++i) {
        double x0 = x_start + (double)i * x_spacing;
        double y0 = (double)heights[i];
        double x1 = x_start + (double)(i + 1) * x_spacing;
        double y1 = (double)heights[i + 1];
        double dx = x1 - x0, dy = y1 - y0;
        double length = sqrt(dx * dx + dy * dy);
        double nx = -dy / length, ny = dx / length;
        if (ny < 0) { nx = -nx; ny = -ny; }
        float *E = row + L->edges_off + i * 6;
        E[0] = (float)x0; E[1] = (float)y0; E[2] = (float)x1; E[3] = (float)y1;
        E[4] = (float)nx; E[5] = (float)ny;
    }
}

int orc_flat_detect(const orc_layout *L, const float *row, const float *shapes, float ground_y,
                    float *contacts) {
    int count = 0;
    for (int b = 0; b < L->num_bodies; ++b) {
        const float *B = row + L->bodies_off + b * ORC_BODY_SIZE;
        float body_x = B[ORC_IDX_X], body_y = B[ORC_IDX_Y], body_angle = B[ORC_IDX_ANGLE];
        int shape_idx = (int)B[ORC_IDX_SHAPE];
        const float *S = shapes + shape_idx * ORC_SHAPE_SIZE;
        int shape_type = (int)S[0];
        float cos_a = f32_cos(body_angle), sin_a = f32_sin(body_angle);
        if (shape_type == ORC_SHAPE_POLYGON) {
            int n_verts = (int)S[1];
            for (int v = 0; v < n_verts; ++v) {
                if (v >= ORC_MAX_POLY_VERTS) break;
                float local_x = S[2 + v * 2], local_y = S[3 + v * 2];
                float world_x = body_x + local_x * cos_a - local_y * sin_a;
                float world_y = body_y + local_x * sin_a + local_y * cos_a;
                float penetration = ground_y - world_y;
                if (penetration > 0.0f && count < L->max_contacts) {
                    put_contact(contacts + count * ORC_CONTACT_SIZE, b, world_x, world_y, 0.0f, 1.0f,
                                penetration);
                    count += 1;
                }
            }
        } else if (shape_type == ORC_SHAPE_CIRCLE) {
            float radius = S[1], cox = S[2], coy = S[3];
            float cwx = body_x + cox * cos_a - coy * sin_a;
            float cwy = body_y + cox * sin_a + coy * cos_a;
            float penetration = ground_y - (cwy - radius);
            if (penetration > 0.0f && count < L->max_contacts) {
                put_contact(contacts + count * ORC_CONTACT_SIZE, b, cwx, cwy - radius, 0.0f, 1.0f,
                            penetration);
                count += 1;
            }
        }
    }
    return count;
}

void orc_contact_solve_velocity(const orc_layout *L, float *row, float *contacts, int count,
                                float friction, float restitution) {
    for (int c = 0; c < count; ++c) {
        float *C = contacts + c * ORC_CONTACT_SIZE;
        int ia = (int)C[ORC_C_BODY_A], ib = (int)C[ORC_C_BODY_B];
        float point_x = C[ORC_C_PX], point_y = C[ORC_C_PY];
        float normal_x = C[ORC_C_NX], normal_y = C[ORC_C_NY];
        float *A = BODY(ia);
        float *Bb = (ib >= 0) ? BODY(ib) : 0;
        float pos_a_x = A[ORC_IDX_X], pos_a_y = A[ORC_IDX_Y];
        float vel_a_x = A[ORC_IDX_VX], vel_a_y = A[ORC_IDX_VY], omega_a = A[ORC_IDX_OMEGA];
        float inv_mass_a = A[ORC_IDX_INV_MASS], inv_inertia_a = A[ORC_IDX_INV_INERTIA];
        float inv_mass_b = 0.0f, inv_inertia_b = 0.0f, vel_b_x = 0.0f, vel_b_y = 0.0f, omega_b = 0.0f;
        float pos_b_x = point_x, pos_b_y = point_y;
        if (Bb) {
            pos_b_x = Bb[ORC_IDX_X]; pos_b_y = Bb[ORC_IDX_Y];
            vel_b_x = Bb[ORC_IDX_VX]; vel_b_y = Bb[ORC_IDX_VY]; omega_b = Bb[ORC_IDX_OMEGA];
            inv_mass_b = Bb[ORC_IDX_INV_MASS]; inv_inertia_b = Bb[ORC_IDX_INV_INERTIA];
        }
        float ra_x = point_x - pos_a_x, ra_y = point_y - pos_a_y;
        float rb_x = point_x - pos_b_x, rb_y = point_y - pos_b_y;
        float vel_at_a_x = vel_a_x - omega_a * ra_y, vel_at_a_y = vel_a_y + omega_a * ra_x;
        float vel_at_b_x = vel_b_x - omega_b * rb_y, vel_at_b_y = vel_b_y + omega_b * rb_x;
        float rel_vel_x = vel_at_a_x - vel_at_b_x, rel_vel_y = vel_at_a_y - vel_at_b_y;
        float vel_normal = rel_vel_x * normal_x + rel_vel_y * normal_y;
        if (!(vel_normal < 0.0f)) continue;

        float ra_cross_n = ra_x * normal_y - ra_y * normal_x;
        float rb_cross_n = rb_x * normal_y - rb_y * normal_x;
        float k = inv_mass_a + inv_mass_b;
        k = k + inv_inertia_a * ra_cross_n * ra_cross_n;
        k = k + inv_inertia_b * rb_cross_n * rb_cross_n;
        float j_normal = -(1.0f + restitution) * vel_normal / k;
        float old_impulse = C[ORC_C_JN];
        float new_impulse = old_impulse + j_normal;
        if (new_impulse < 0.0f) new_impulse = 0.0f;
        C[ORC_C_JN] = new_impulse;
        j_normal = new_impulse - old_impulse;
        float impulse_x = j_normal * normal_x, impulse_y = j_normal * normal_y;
        A[ORC_IDX_VX] = vel_a_x + impulse_x * inv_mass_a;
        A[ORC_IDX_VY] = vel_a_y + impulse_y * inv_mass_a;
        A[ORC_IDX_OMEGA] = omega_a + (ra_x * impulse_y - ra_y * impulse_x) * inv_inertia_a;
        if (Bb) {
            Bb[ORC_IDX_VX] = vel_b_x - impulse_x * inv_mass_b;
            Bb[ORC_IDX_VY] = vel_b_y - impulse_y * inv_mass_b;
            Bb[ORC_IDX_OMEGA] = omega_b - (rb_x * impulse_y - rb_y * impulse_x) * inv_inertia_b;
        }
        vel_a_x = A[ORC_IDX_VX]; vel_a_y = A[ORC_IDX_VY]; omega_a = A[ORC_IDX_OMEGA];
        if (Bb) { vel_b_x = Bb[ORC_IDX_VX]; vel_b_y = Bb[ORC_IDX_VY]; omega_b = Bb[ORC_IDX_OMEGA]; }
        vel_at_a_x = vel_a_x - omega_a * ra_y; vel_at_a_y = vel_a_y + omega_a * ra_x;
        vel_at_b_x = vel_b_x - omega_b * rb_y; vel_at_b_y = vel_b_y + omega_b * rb_x;
        rel_vel_x = vel_at_a_x - vel_at_b_x; rel_vel_y = vel_at_a_y - vel_at_b_y;

        float tangent_x = -normal_y, tangent_y = normal_x;
        float vel_tangent = rel_vel_x * tangent_x + rel_vel_y * tangent_y;
        float ra_cross_t = ra_x * tangent_y - ra_y * tangent_x;
        float rb_cross_t = rb_x * tangent_y - rb_y * tangent_x;
        float k_t = inv_mass_a + inv_mass_b;
        k_t = k_t + inv_inertia_a * ra_cross_t * ra_cross_t;
        k_t = k_t + inv_inertia_b * rb_cross_t * rb_cross_t;
        float j_tangent = -vel_tangent / k_t;
        float max_friction = friction * C[ORC_C_JN];
        float old_tangent = C[ORC_C_JT];
        float new_tangent = old_tangent + j_tangent;
        if (new_tangent > max_friction) new_tangent = max_friction;
        else if (new_tangent < -max_friction) new_tangent = -max_friction;
        C[ORC_C_JT] = new_tangent;
        j_tangent = new_tangent - old_tangent;
        float friction_x = j_tangent * tangent_x, friction_y = j_tangent * tangent_y;
        A[ORC_IDX_VX] = A[ORC_IDX_VX] + friction_x * inv_mass_a;
        A[ORC_IDX_VY] = A[ORC_IDX_VY] + friction_y * inv_mass_a;
        A[ORC_IDX_OMEGA] = A[ORC_IDX_OMEGA] + (ra_x * friction_y - ra_y * friction_x) * inv_inertia_a;
        if (Bb) {
            Bb[ORC_IDX_VX] = Bb[ORC_IDX_VX] - friction_x * inv_mass_b;
            Bb[ORC_IDX_VY] = Bb[ORC_IDX_VY] - friction_y * inv_mass_b;
            Bb[ORC_IDX_OMEGA] =
                Bb[ORC_IDX_OMEGA] - (rb_x * friction_y - rb_y * friction_x) * inv_inertia_b;
        }
    }
}

void orc_contact_solve_position(const orc_layout *L, float *row, const float *contacts, int count,
                                float baumgarte, float slop) {
    for (int c = 0; c < count; ++c) {
        const float *C = contacts + c * ORC_CONTACT_SIZE;
        int ia = (int)C[ORC_C_BODY_A], ib = (int)C[ORC_C_BODY_B];
        float normal_x = C[ORC_C_NX], normal_y = C[ORC_C_NY], penetration = C[ORC_C_DEPTH];
        float correction = penetration - slop;
        if (correction <= 0.0f) continue;
        correction = baumgarte * correction;
        float *A = BODY(ia);
        float *Bb = (ib >= 0) ? BODY(ib) : 0;
        float inv_mass_a = A[ORC_IDX_INV_MASS];
        float inv_mass_b = Bb ? Bb[ORC_IDX_INV_MASS] : 0.0f;
        float total = inv_mass_a + inv_mass_b;
        if (total == 0.0f) continue;
        float correction_a = correction * inv_mass_a / total;
        float correction_b = correction * inv_mass_b / total;
        A[ORC_IDX_X] = A[ORC_IDX_X] + normal_x * correction_a;
        A[ORC_IDX_Y] = A[ORC_IDX_Y] + normal_y * correction_a;
        if (Bb) {
            Bb[ORC_IDX_X] = Bb[ORC_IDX_X] - normal_x * correction_b;
            Bb[ORC_IDX_Y] = Bb[ORC_IDX_Y] - normal_y * correction_b;
        }
    }
}

void orc_joint_solve_velocity(const orc_layout *L, float *row, float dt) {
    int n_joints = (int)row[L->joint_count_off];
    for (int j = 0; j < n_joints; ++j) {
        if (j >= L->max_joints) break;
        const float *J = row + L->joints_off + j * ORC_JOINT_SIZE;
        if ((int)J[ORC_J_TYPE] != 0) continue;
        float *A = BODY((int)J[ORC_J_BODY_A]);
        float *B = BODY((int)J[ORC_J_BODY_B]);
        float angle_a = A[ORC_IDX_ANGLE], vxa = A[ORC_IDX_VX], vya = A[ORC_IDX_VY], wa = A[ORC_IDX_OMEGA];
        float inv_ma = A[ORC_IDX_INV_MASS], inv_ia = A[ORC_IDX_INV_INERTIA];
        float angle_b = B[ORC_IDX_ANGLE], vxb = B[ORC_IDX_VX], vyb = B[ORC_IDX_VY], wb = B[ORC_IDX_OMEGA];
        float inv_mb = B[ORC_IDX_INV_MASS], inv_ib = B[ORC_IDX_INV_INERTIA];
        float local_ax = J[ORC_J_AX], local_ay = J[ORC_J_AY], local_bx = J[ORC_J_BX], local_by = J[ORC_J_BY];
        float cos_a = f32_cos(angle_a), sin_a = f32_sin(angle_a);
        float cos_b = f32_cos(angle_b), sin_b = f32_sin(angle_b);
        float rax = local_ax * cos_a - local_ay * sin_a, ray = local_ax * sin_a + local_ay * cos_a;
        float rbx = local_bx * cos_b - local_by * sin_b, rby = local_bx * sin_b + local_by * cos_b;
        float va_anchor_x = vxa - wa * ray, va_anchor_y = vya + wa * rax;
        float vb_anchor_x = vxb - wb * rby, vb_anchor_y = vyb + wb * rbx;
        float cdot_x = vb_anchor_x - va_anchor_x, cdot_y = vb_anchor_y - va_anchor_y;
        float k11 = inv_ma + inv_mb + inv_ia * ray * ray + inv_ib * rby * rby;
        float k12 = -inv_ia * rax * ray - inv_ib * rbx * rby;
        float k22 = inv_ma + inv_mb + inv_ia * rax * rax + inv_ib * rbx * rbx;
        float det = k11 * k22 - k12 * k12;
        if (det < 1e-10f) det = 1e-10f;
        float inv_det = 1.0f / det;
        float inv_k11 = k22 * inv_det, inv_k12 = -k12 * inv_det, inv_k22 = k11 * inv_det;
        float impulse_x = -(inv_k11 * cdot_x + inv_k12 * cdot_y);
        float impulse_y = -(inv_k12 * cdot_x + inv_k22 * cdot_y);
        A[ORC_IDX_VX] = vxa - inv_ma * impulse_x;
        A[ORC_IDX_VY] = vya - inv_ma * impulse_y;
        A[ORC_IDX_OMEGA] = wa - inv_ia * (rax * impulse_y - ray * impulse_x);
        B[ORC_IDX_VX] = vxb + inv_mb * impulse_x;
        B[ORC_IDX_VY] = vyb + inv_mb * impulse_y;
        B[ORC_IDX_OMEGA] = wb + inv_ib * (rbx * impulse_y - rby * impulse_x);

        int flags = (int)J[ORC_J_FLAGS];
        if (flags & ORC_JF_SPRING) {
            float stiffness = J[ORC_J_STIFF], damping = J[ORC_J_DAMP], ref_angle = J[ORC_J_REF];
            float current_angle = angle_b - angle_a;
            float angle_error = current_angle - ref_angle;
            float rel_omega = wb - wa; /* pre-impulse angular velocities */
            float spring_torque = -stiffness * angle_error - damping * rel_omega;
            float angular_impulse = spring_torque * dt;
            float eff_inertia = inv_ia + inv_ib;
            if (eff_inertia > 1e-10f) {
                A[ORC_IDX_OMEGA] = A[ORC_IDX_OMEGA] - inv_ia * angular_impulse / eff_inertia;
                B[ORC_IDX_OMEGA] = B[ORC_IDX_OMEGA] + inv_ib * angular_impulse / eff_inertia;
            }
        }
        if (flags & ORC_JF_LIMIT) {
            float lower = J[ORC_J_LO], upper = J[ORC_J_HI], lim_ref = J[ORC_J_REF];
            float current_wa = A[ORC_IDX_OMEGA], current_wb = B[ORC_IDX_OMEGA];
            float relative_angle = B[ORC_IDX_ANGLE] - A[ORC_IDX_ANGLE] - lim_ref;
            float rel_omega = current_wb - current_wa;
            float lim_eff = inv_ia + inv_ib;
            if (lim_eff > 1e-10f) {
                float limit_impulse = 0.0f;
                if (relative_angle <= lower) {
                    if (rel_omega < 0.0f) limit_impulse = -rel_omega / lim_eff;
                } else if (relative_angle >= upper) {
                    if (rel_omega > 0.0f) limit_impulse = -rel_omega / lim_eff;
                }
                if (limit_impulse != 0.0f) {
                    A[ORC_IDX_OMEGA] = current_wa - inv_ia * limit_impulse;
                    B[ORC_IDX_OMEGA] = current_wb + inv_ib * limit_impulse;
                }
            }
        }
        if (flags & ORC_JF_MOTOR) {
            float motor_speed = J[ORC_J_MOTOR_SPEED], max_torque = J[ORC_J_MAX_TORQUE];
            float current_wa = A[ORC_IDX_OMEGA], current_wb = B[ORC_IDX_OMEGA];
            float rel_omega = current_wb - current_wa;
            float speed_error = motor_speed - rel_omega;
            float eff_inertia = inv_ia + inv_ib;
            if (eff_inertia > 1e-10f) {
                float motor_impulse = speed_error / eff_inertia;
                float max_impulse = max_torque * dt;
                if (motor_impulse > max_impulse) motor_impulse = max_impulse;
                if (motor_impulse < -max_impulse) motor_impulse = -max_impulse;
                A[ORC_IDX_OMEGA] = current_wa - inv_ia * motor_impulse;
                B[ORC_IDX_OMEGA] = current_wb + inv_ib * motor_impulse;
            }
        }
    }
}

void orc_joint_solve_position(const orc_layout *L, float *row, float baumgarte, float slop) {
    int n_joints = (int)row[L->joint_count_off];
    for (int j = 0; j < n_joints; ++j) {
        if (j >= L->max_joints) break;
        const float *J = row + L->joints_off + j * ORC_JOINT_SIZE;
        if ((int)J[ORC_J_TYPE] != 0) continue;
        float *A = BODY((int)J[ORC_J_BODY_A]);
        float *B = BODY((int)J[ORC_J_BODY_B]);
        float xa = A[ORC_IDX_X], ya = A[ORC_IDX_Y], angle_a = A[ORC_IDX_ANGLE];
        float inv_ma = A[ORC_IDX_INV_MASS], inv_ia = A[ORC_IDX_INV_INERTIA];
        float xb = B[ORC_IDX_X], yb = B[ORC_IDX_Y], angle_b = B[ORC_IDX_ANGLE];
        float inv_mb = B[ORC_IDX_INV_MASS], inv_ib = B[ORC_IDX_INV_INERTIA];
        float local_ax = J[ORC_J_AX], local_ay = J[ORC_J_AY], local_bx = J[ORC_J_BX], local_by = J[ORC_J_BY];
        float cos_a = f32_cos(angle_a), sin_a = f32_sin(angle_a);
        float cos_b = f32_cos(angle_b), sin_b = f32_sin(angle_b);
        float rax = local_ax * cos_a - local_ay * sin_a, ray = local_ax * sin_a + local_ay * cos_a;
        float rbx = local_bx * cos_b - local_by * sin_b, rby = local_bx * sin_b + local_by * cos_b;
        float anchor_ax = xa + rax, anchor_ay = ya + ray;
        float anchor_bx = xb + rbx, anchor_by = yb + rby;
        float cx = anchor_bx - anchor_ax, cy = anchor_by - anchor_ay;
        float error = sqrtf(cx * cx + cy * cy);
        if (error < slop) continue;
        float k11 = inv_ma + inv_mb + inv_ia * ray * ray + inv_ib * rby * rby;
        float k12 = -inv_ia * rax * ray - inv_ib * rbx * rby;
        float k22 = inv_ma + inv_mb + inv_ia * rax * rax + inv_ib * rbx * rbx;
        float det = k11 * k22 - k12 * k12;
        if (det < 1e-10f) det = 1e-10f;
        float inv_det = 1.0f / det;
        float inv_k11 = k22 * inv_det, inv_k12 = -k12 * inv_det, inv_k22 = k11 * inv_det;
        float correction_x = -baumgarte * (inv_k11 * cx + inv_k12 * cy);
        float correction_y = -baumgarte * (inv_k12 * cx + inv_k22 * cy);
        A[ORC_IDX_X] = xa - inv_ma * correction_x;
        A[ORC_IDX_Y] = ya - inv_ma * correction_y;
        A[ORC_IDX_ANGLE] = angle_a - inv_ia * (rax * correction_y - ray * correction_x);
        B[ORC_IDX_X] = xb + inv_mb * correction_x;
        B[ORC_IDX_Y] = yb + inv_mb * correction_y;
        B[ORC_IDX_ANGLE] = angle_b + inv_ib * (rbx * correction_y - rby * correction_x);

        int flags = (int)J[ORC_J_FLAGS];
        if (flags & ORC_JF_LIMIT) {
            float lower = J[ORC_J_LO], upper = J[ORC_J_HI], pos_ref = J[ORC_J_REF];
            float cur_a = A[ORC_IDX_ANGLE], cur_b = B[ORC_IDX_ANGLE];
            float relative_angle = cur_b - cur_a - pos_ref;
            float eff = inv_ia + inv_ib;
            if (eff > 1e-10f) {
                float angle_correction = 0.0f;
                if (relative_angle < lower) angle_correction = baumgarte * (lower - relative_angle);
                else if (relative_angle > upper) angle_correction = baumgarte * (upper - relative_angle);
                if (angle_correction != 0.0f) {
                    A[ORC_IDX_ANGLE] = cur_a - inv_ia * angle_correction / eff;
                    B[ORC_IDX_ANGLE] = cur_b + inv_ib * angle_correction / eff;
                }
            }
        }
    }
}

float orc_lidar_ray(const orc_layout *L, const float *row, float ox, float oy, float rdx, float rdy) {
    int n_edges = (int)row[L->edge_count_off];
    float min_t = 1.0f;
    for (int e = 0; e < n_edges; ++e) {
        if (e >= L->max_edges) break;
        const float *E = row + L->edges_off + e * 6;
        float ex = E[2] - E[0], ey = E[3] - E[1];
        float denom = rdx * ey - rdy * ex;
        float t = -1.0f;
        if (!(denom > -1e-10f && denom < 1e-10f)) {
            float dx = ox - E[0], dy = oy - E[1];
            float tt = (ex * dy - ey * dx) / denom;
            float u = (rdx * dy - rdy * dx) / denom;
            if (tt >= 0.0f && tt <= 1.0f && u >= 0.0f && u <= 1.0f) t = tt;
        }
        if (t >= 0.0f && t < min_t) min_t = t;
    }
    return min_t;
}
