/*
 * CPU parity oracle for the mojo-rl rollout / PPO-update hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library may include, link
 * or call this code; it exists so that the tests, the smoke check and the
 * bench's cpu_baseline leg have an independent CPU statement of what the HIP
 * kernels must compute.  Each function cites the reference file:line whose
 * arithmetic (order of operations included) it restates.
 *
 * Conventions shared with the HIP side:
 *   - all state is fp32 unless the reference's CPU code computes in Float64,
 *     in which case the same Float64 steps are taken here;
 *   - no FMA contraction (build with -ffp-contract=off);
 *   - sinf/cosf of an fp32 angle are the correctly rounded fp32 values,
 *     obtained as (float)sin((double)x);
 *   - random streams: xorshift32 and Philox4x32-10 as documented in orc_rng.c.
 *
 * Parity status (which functions are pinned by an independent check lives in
 * tests/test_oracle_*.py).  Unpinned by construction, because the Mojo
 * standard library is not available to diff against:
 *   - the seed/offset -> key/counter packing and the u32 -> f32 map of
 *     random.philox.Random.step_uniform (orc_philox_uniform4): parity unpinned;
 *   - the global random_float64() stream (weight init, host shuffle): not
 *     restated; callers pass explicit arrays instead: parity unpinned;
 *   - last-ulp behaviour of Mojo's fp32 sin/cos/exp/log/tanh: parity unpinned
 *     (this oracle uses correctly rounded values).
 */
#ifndef ORC_H
#define ORC_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------------------------------------------------------- rng --- */
uint32_t orc_xorshift32(uint32_t s);
/* returns uniform in [0,1] and advances *state (deep_rl/gpu/random.mojo:20-29) */
float orc_random_uniform(uint32_t *state);
float orc_random_range(uint32_t *state, float lo, float hi);
/* raw Philox4x32-10 block */
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);
/* the call_index-th step_uniform() of Random(seed, offset) */
void orc_philox_uniform4(uint64_t seed, uint64_t offset, uint64_t call_index, float out[4]);

/* ------------------------------------------------------------ CartPole --- */
#define ORC_CARTPOLE_STATE 4
void orc_cartpole_step(float s[4], int32_t *steps, int action, float *reward, float *done);
void orc_cartpole_reset(float s[4], int32_t *steps, int env, uint32_t seed);
void orc_cartpole_step_batch(float *states, int32_t *steps, const float *actions, float *rewards,
                             float *dones, float *obs, int batch);
void orc_cartpole_reset_batch(float *states, int32_t *steps, int batch, uint32_t seed);
void orc_cartpole_selective_reset_batch(float *states, int32_t *steps, float *dones, int batch,
                                        uint32_t seed);

/* ------------------------------------------------------------ Pendulum --- */
#define ORC_PENDULUM_STATE 8
void orc_pendulum_step(float s[8], float action, float *reward, float *done);
void orc_pendulum_reset(float s[8], int env, uint64_t seed);
void orc_pendulum_step_batch(float *states, const float *actions, float *rewards, float *dones,
                             float *obs, int batch);
void orc_pendulum_reset_batch(float *states, int batch, uint64_t seed);
void orc_pendulum_selective_reset_batch(float *states, float *dones, int batch, uint64_t seed);

/* ----------------------------------------------------------- physics2d --- */
enum {
    ORC_BODY_SIZE = 13, ORC_IDX_X = 0, ORC_IDX_Y = 1, ORC_IDX_ANGLE = 2, ORC_IDX_VX = 3,
    ORC_IDX_VY = 4, ORC_IDX_OMEGA = 5, ORC_IDX_FX = 6, ORC_IDX_FY = 7, ORC_IDX_TAU = 8,
    ORC_IDX_MASS = 9, ORC_IDX_INV_MASS = 10, ORC_IDX_INV_INERTIA = 11, ORC_IDX_SHAPE = 12,
    ORC_SHAPE_SIZE = 20, ORC_SHAPE_POLYGON = 0, ORC_SHAPE_CIRCLE = 1, ORC_MAX_POLY_VERTS = 8,
    ORC_CONTACT_SIZE = 9, ORC_C_BODY_A = 0, ORC_C_BODY_B = 1, ORC_C_PX = 2, ORC_C_PY = 3,
    ORC_C_NX = 4, ORC_C_NY = 5, ORC_C_DEPTH = 6, ORC_C_JN = 7, ORC_C_JT = 8,
    ORC_JOINT_SIZE = 17, ORC_J_TYPE = 0, ORC_J_BODY_A = 1, ORC_J_BODY_B = 2, ORC_J_AX = 3,
    ORC_J_AY = 4, ORC_J_BX = 5, ORC_J_BY = 6, ORC_J_REF = 7, ORC_J_LO = 8, ORC_J_HI = 9,
    ORC_J_MAX_TORQUE = 10, ORC_J_MOTOR_SPEED = 11, ORC_J_STIFF = 12, ORC_J_DAMP = 13,
    ORC_J_FLAGS = 14, ORC_J_IMPULSE = 15, ORC_J_MOTOR_IMPULSE = 16,
    ORC_JF_LIMIT = 1, ORC_JF_MOTOR = 2, ORC_JF_SPRING = 4
};

/* offsets of the per-env flat row, physics2d/layout.mojo:58-126 */
typedef struct {
    int num_bodies, max_contacts, max_joints, max_edges, obs_dim, meta_size, num_shapes;
    int bodies_off, forces_off, joints_off, joint_count_off, edges_off, edge_count_off, meta_off;
    int state_size;
} orc_layout;

void orc_layout_make(orc_layout *L, int num_bodies, int max_contacts, int max_joints,
                     int max_edges, int obs_dim, int meta_size, int num_shapes);

void orc_integrate_velocities(const orc_layout *L, float *row, float gx, float gy, float dt);
void orc_integrate_positions(const orc_layout *L, float *row, float dt);
int  orc_edge_detect(const orc_layout *L, const float *row, const float *shapes, float *contacts);
int  orc_flat_detect(const orc_layout *L, const float *row, const float *shapes, float ground_y,
                     float *contacts);
void orc_contact_solve_velocity(const orc_layout *L, float *row, float *contacts, int count,
                                float friction, float restitution);
void orc_contact_solve_position(const orc_layout *L, float *row, const float *contacts, int count,
                                float baumgarte, float slop);
void orc_joint_solve_velocity(const orc_layout *L, float *row, float dt);
void orc_joint_solve_position(const orc_layout *L, float *row, float baumgarte, float slop);
/* returns hit fraction in [0,1] (1 = no hit), physics2d/lidar/lidar.mojo:25-141 */
float orc_lidar_ray(const orc_layout *L, const float *row, float ox, float oy, float dx, float dy);
void orc_set_terrain_from_heights(const orc_layout *L, float *row, const float *heights, int n_points,
                                  double x_start, double x_spacing);

/* --------------------------------------------------------- LunarLander --- */
#define ORC_LL_STATE 192
#define ORC_LL_OBS 8
void orc_ll_layout(orc_layout *L);
void orc_ll_shapes(float shapes[3 * 20]);
uint64_t orc_ll_combined_seed(uint64_t seed, int env);
void orc_ll_reset(float *row, uint64_t combined_seed);
/* contacts_out (8*9 floats) and n_contacts_out may be NULL */
/* wind / turbulence setting of all LunarLander rows stepped from now on (off by default) */
void orc_ll_set_wind(int enable, double wind_power, double turbulence_power);
void orc_ll_step(float *row, int env, int action, float *reward, float *done,
                 float *contacts_out, int *n_contacts_out);
/* the continuous-action overload: a0 = main throttle in [-1, 1], a1 = side control in [-1, 1] */
void orc_ll_step_continuous(float *row, int env, float a0, float a1, float *reward, float *done,
                            float *contacts_out, int *n_contacts_out);
void orc_ll_step_continuous_batch(float *states, const float *actions, float *rewards, float *dones,
                                  float *obs, int batch);
void orc_ll_reset_batch(float *states, int batch, uint64_t seed);
void orc_ll_selective_reset_batch(float *states, const float *dones, int batch, uint64_t seed);
void orc_ll_step_batch(float *states, const float *actions, float *rewards, float *dones,
                       float *obs, int batch, int n_threads);

/* ---------------------------------------- BipedalWalker / HalfCheetah --- */
#define ORC_BW_STATE 950
#define ORC_HC_STATE 253
void orc_bw_layout(orc_layout *L);
void orc_bw_shapes(float *shapes /* 5*20 */);
void orc_bw_reset(float *row, uint64_t combined_seed);
void orc_bw_step(float *row, const float action[4], float *reward, float *done);
/* dones == NULL: reset every env; otherwise only rows with dones > 0.5 (flags are left as they are) */
void orc_bw_reset_batch(float *states, const float *dones, int batch, uint64_t seed);
void orc_bw_step_batch(float *states, const float *actions, float *rewards, float *dones, float *obs,
                       int batch, int n_threads);
void orc_hc_layout(orc_layout *L);
void orc_hc_shapes(float *shapes /* 7*20 */);
void orc_hc_reset(float *row, uint64_t combined_seed);
void orc_hc_step(float *row, const float action[6], float *reward, float *done);
void orc_hc_reset_batch(float *states, const float *dones, int batch, uint64_t seed);
void orc_hc_step_batch(float *states, const float *actions, float *rewards, float *dones, float *obs,
                       int batch, int n_threads);

/* ------------------------------------------------------------- MLP/NN --- */
enum { ORC_LINEAR = 0, ORC_LINEAR_RELU = 1, ORC_LINEAR_TANH = 2, ORC_STOCHASTIC_ACTOR = 3 };
typedef struct { int kind, in_dim, out_dim; } orc_layer; /* out_dim = action_dim for actor head */

int orc_layer_param_size(const orc_layer *l);
int orc_layer_cache_size(const orc_layer *l);
int orc_layer_out_dim(const orc_layer *l);
int orc_mlp_param_size(const orc_layer *ls, int n);
int orc_mlp_cache_size(const orc_layer *ls, int n);
/* cache may be NULL (no-cache forward) */
void orc_mlp_forward(const orc_layer *ls, int n, int batch, const float *in, const float *params,
                     float *out, float *cache);
/* accumulates into grads (caller zeroes), writes grad_in (may be NULL) */
void orc_mlp_backward(const orc_layer *ls, int n, int batch, const float *grad_out,
                      const float *params, const float *cache, float *grads, float *grad_in);

/* ------------------------------------------------------ PPO utilities --- */
void orc_sample_categorical(const float *logits, int n, int num_actions, uint32_t seed,
                            float *actions, float *log_probs);
void orc_sample_gaussian(const float *actor_out, int n, int action_dim, uint64_t seed,
                         float *actions, float *log_probs);
/* ---------------------------------------------------------- CarRacingV2 --- */
#define ORC_CR_STATE 3040
int orc_cr_tile_at(const float *row, float x, float y, int num_tiles);
uint64_t orc_cr_combined_seed(uint64_t seed, int env);
void orc_cr_reset(float *row, uint64_t combined_seed);
void orc_cr_step(float *row, const float *action, float *reward, float *done);
/* 0 (default): the CPU env's step, car_racing_v2.mojo:258-287; 1: the GPU trait's step_kernel_gpu, :1556-1716 */
void orc_cr_set_step_form(int form);
/* dones == NULL: every row; otherwise rows with dones > 0.5 (their flag is cleared) */
void orc_cr_reset_batch(float *states, float *dones, int batch, uint64_t seed);
void orc_cr_step_batch(float *states, const float *actions, float *rewards, float *dones, float *obs, int batch,
                       int n_threads);

/* ------------------------------------------------- HopperPlanar / Walker2dPlanar ---
 * envs/mujoco_planar/hopper_planar.mojo, walker_planar.mojo (Float64 CPU structs); which = 0 hopper
 * (row of 62 floats, obs 11, action 3), 1 walker (98, 17, 6); row layout in orc_planar.c */
int orc_planar_state_size(int which);
void orc_planar_reset(int which, float *row, uint64_t combined_seed);
void orc_planar_step(int which, float *row, const float *action, float *reward, float *done);
void orc_planar_reset_batch(int which, float *states, const float *dones, int batch, uint64_t seed);
void orc_planar_step_batch(int which, float *states, const float *actions, float *rewards, float *dones,
                           float *obs, int batch, int n_threads);

void orc_add_obs_noise(float *obs, int n, int obs_dim, float noise_std, uint32_t seed);
void orc_gae(int T, int N, const float *rewards, const float *values, const float *dones,
             const float *bootstrap, double gamma, double lam, float *adv, float *ret);
void orc_normalize_advantages(float *adv, int n);               /* ppo.mojo:2356-2371 */
void orc_normalize_minibatch_host(float *adv, int n);           /* ppo.mojo:2478-2511 + 637-653 */
void orc_normalize_minibatch_fused(float *adv, int n);          /* kernels.mojo:507-599 */
void orc_ppo_actor_grad_discrete(const float *logits, const float *old_logp, const float *adv,
                                 const float *actions, int mb, int num_actions, float clip_eps,
                                 float ent_coef, float *grad_logits, float *kl);
void orc_ppo_actor_grad_gaussian(const float *actor_out, const float *old_logp, const float *adv,
                                 const float *actions, int mb, int action_dim, float clip_eps,
                                 float ent_coef, float *grad_out, float *kl);
/* convention 0 = discrete agent (ppo.mojo:538-633), 1 = continuous (kernels.mojo:416-486) */
void orc_ppo_critic_grad(const float *values, const float *old_values, const float *returns, int mb,
                         int convention, int clipped, float value_coef, float clip_eps, float *grad);
float orc_clip_grad_norm(float *g, int n, float max_norm);     /* returns the scale applied */
void orc_adam_step(float *p, const float *g, float *state, int n, int t, double lr, double b1,
                   double b2, double eps);
void orc_clamp_log_std(float *params, int offset, int action_dim);
typedef struct { double count, mean, var_sum; } orc_rms;
void orc_rms_update(orc_rms *r, const float *x, int n);
void orc_rms_normalize(const orc_rms *r, float *x, int n);
/* shuffle_indices, core/utils/shuffle.mojo:21-48, on the draws u[0 .. n-2] in consumption order */
void orc_shuffle_indices(int n, const double *u, int32_t *indices);

#ifdef __cplusplus
}
#endif
#endif
