/*
 * libmrl_hip.so -- C ABI of the MI355X (gfx950) rollout / PPO-update path for mojo-rl.
 *
 * Every entry point replaces one interface of the reference (cited per function as
 * file:line under the reference tree).  Conventions:
 *   - all data pointers are DEVICE pointers to fp32 buffers in the reference's own
 *     layouts (row-major, obs at offset 0 of each env row, rollout buffers time-major);
 *   - the caller owns every buffer; the library owns only its mrl_ctx;
 *   - every call only enqueues work on the context's stream (no synchronisation),
 *     like DeviceContext.enqueue_function in the reference.  One exception: the context holds two
 *     workspaces (layer-by-layer MLP intermediates; policy temporaries of a rollout step) that grow
 *     on the first call that needs more than they hold, and growing drains the stream, frees and
 *     allocates.  mrl_ctx_reserve sizes them ahead so that no later call does;
 *   - return value 0 = success; non-zero = failure, text in mrl_last_error()
 *     (thread-local).  A Mojo shim turns non-zero into `raise Error(...)`.
 */
#ifndef MRL_H
#define MRL_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mrl_ctx mrl_ctx;

enum {
    MRL_OK = 0,
    MRL_E_ARG = -1,      /* bad argument (null pointer, size, unknown id) */
    MRL_E_HIP = -2,      /* a HIP runtime call failed */
    MRL_E_UNSUPPORTED = -3,
    MRL_E_SYNC = -4      /* a kernel gave up waiting at one of its internal barriers */
};

enum mrl_env_id {
    MRL_ENV_CARTPOLE = 0,    /* envs/cartpole.mojo:120 CartPoleEnv */
    MRL_ENV_PENDULUM = 1,    /* envs/pendulum/pendulum_v2.mojo:57 PendulumV2 */
    MRL_ENV_LUNARLANDER = 2, /* envs/lunar_lander/lunar_lander_v2.mojo:123 LunarLanderV2 */
    MRL_ENV_BIPEDAL = 3,     /* envs/bipedal_walker/bipedal_walker_v2.mojo:103 BipedalWalkerV2 */
    MRL_ENV_HALFCHEETAH = 4, /* envs/half_cheetah/cheetah_planar_v2.mojo:91 HalfCheetahPlanarV2 */
    /* LunarLanderV2 as a GPUContinuousEnv: the step_kernel_gpu overload with ACTION_DIM = 2
     * (lunar_lander_v2.mojo:1520-1588); rows, reset and selective reset are those of
     * MRL_ENV_LUNARLANDER */
    MRL_ENV_LUNARLANDER_CONTINUOUS = 5,
    /* envs/car_racing/car_racing_v2.mojo:90 CarRacingV2 behind GPUContinuousEnv (:947-1150): the trait's
     * row, reset and done-row protocol.  NOTE the reward: by default the step pays what the reference's
     * CPU env pays (-0.1 per step + 100 / tiles per new tile, Float64, :258-287 and :781-846), which is
     * NOT what the reference's step_kernel_gpu pays (0.5 * forward speed - 0.01 + 100 / tiles in fp32,
     * :1636-1666): returns of a run trained with the default are not comparable with the reference's
     * train_gpu.  mrl_car_racing_set_step_form(ctx, MRL_CAR_STEP_GPU_TRAIT) selects the trait's. */
    MRL_ENV_CARRACING = 6,
    /* envs/mujoco_planar/hopper_planar.mojo:162 HopperPlanar and walker_planar.mojo:168 Walker2dPlanar: Float64
     * CPU structs in the reference (reset() / step(action) on lists of Float64), which has no
     * GPUContinuousEnv form of them and hence no row layout; here they stand behind the same calls as the
     * other envs, on rows of this library's own: [obs fp32 (11 / 17) | one float of padding | the struct's
     * Float64 state, two floats per double: torso x, y, angle, vx, vy, omega; (x, y, angle) of the other
     * bodies; joint_angles; joint_velocities; step_count, done, total_reward, prev_x] = 62 / 98 floats.
     * states must be 8-byte aligned.  A row whose done flag is set returns (0, 1) untouched, as elsewhere. */
    MRL_ENV_HOPPER_PLANAR = 7,
    MRL_ENV_WALKER2D_PLANAR = 8
};

/* layer kinds of an MLP description; deep_rl/model/{linear,linear_relu,linear_tanh,stochastic_actor}.mojo */
enum mrl_layer_kind {
    MRL_LINEAR = 0,
    MRL_LINEAR_RELU = 1,
    MRL_LINEAR_TANH = 2,
    MRL_STOCHASTIC_ACTOR = 3 /* out_dim = action_dim; output is [mean | clamped log_std] */
};

typedef struct {
    int32_t kind;    /* mrl_layer_kind */
    int32_t in_dim;
    int32_t out_dim;
} mrl_layer;

#define MRL_MAX_LAYERS 8

/* Seq2[...] nest flattened to its leaf layers; deep_rl/model/sequential.mojo:867-953 (seq()) */
typedef struct {
    int32_t n_layers;
    mrl_layer layers[MRL_MAX_LAYERS];
} mrl_mlp_desc;

/* ------------------------------------------------------------------ library / context */

int mrl_version(void);
const char *mrl_last_error(void);

/* hip_stream: a hipStream_t, or NULL for the default stream.  Replaces the DeviceContext
 * argument every reference GPU method takes (one in-order stream). */
int mrl_ctx_create(void *hip_stream, mrl_ctx **out);
int mrl_ctx_destroy(mrl_ctx *ctx);
/* blocks until the context's stream has drained; DeviceContext.synchronize() */
int mrl_ctx_synchronize(mrl_ctx *ctx);

/* Workspaces of the context, in floats: what they hold now (either pointer may be NULL), and a
 * request to hold at least that much (0 = leave as is; never shrinks).  mrl_ctx_reserve drains the
 * stream when it has to grow one; after a run of the caller's largest shapes mrl_ctx_workspace
 * tells what to reserve in the next process.  No counterpart in the reference, whose DeviceContext
 * allocates inside its layers' forward calls. */
int mrl_ctx_workspace(mrl_ctx *ctx, uint64_t *mlp_floats, uint64_t *rollout_floats);
int mrl_ctx_reserve(mrl_ctx *ctx, uint64_t mlp_floats, uint64_t rollout_floats);

/* The fused collection kernels let groups of wavefronts of a workgroup meet at barriers of their own
 * (counters in LDS).  Every such wait is bounded: after `polls` polls (MRL_DEFAULT_SPIN_LIMIT unless
 * set here; 0 restores the default) the waiting wavefront gives up, the workgroup stops stepping, the
 * kernel ends normally and the next mrl_ctx_synchronize returns MRL_E_SYNC (once).  What the calls since
 * the last synchronize wrote is void then: a workgroup that gave up stores neither its env rows nor its
 * observations nor its episode sums (they keep the values from before the launch), the other workgroups'
 * envs have advanced, and rollout rows and the finished-episode list hold a mixture -- reset the envs
 * and clear done_count before collecting again.  No counterpart
 * in the reference; a tiny limit is how a test exercises the error path without hanging anything. */
#define MRL_DEFAULT_SPIN_LIMIT (1u << 22)
int mrl_ctx_set_spin_limit(mrl_ctx *ctx, unsigned polls);

/* Device-time accounting per phase, the counterpart of the perf_counter_ns phase timers that
 * train_gpu prints (deep_agents/ppo/ppo.mojo:2062-2067, :2777-2838) measured with HIP events on
 * the context's stream instead of host enqueue times.  mrl_profile_begin arms it (at most
 * max_marks phase boundaries are recorded); mrl_profile_end synchronises, adds up the time of
 * each phase id (MRL_PHASE_*) into total_ms[n_phases] / counts[n_phases] and disarms it. */
enum {
    MRL_PHASE_POLICY_FWD = 0, /* actor + critic forward of a rollout step */
    MRL_PHASE_SAMPLE = 1,     /* sampling + pre-step stores */
    MRL_PHASE_ENV = 2,        /* env step (+ auto-reset) */
    MRL_PHASE_POST = 3,       /* post-step stores and episode accounting */
    MRL_PHASE_COLLECT = 4,    /* a fused launch of mrl_rollout_steps (all of the above, many steps) */
    MRL_PHASE_COUNT = 5
};
int mrl_profile_begin(mrl_ctx *ctx, int max_marks);
/* Time only every `every`-th call of mrl_rollout_step (1, the default: all of them).  An event
 * between two kernels costs device time of its own; sampling keeps a long timed run close to an
 * untimed one while the per-phase averages still come from launches inside it. */
int mrl_profile_sample_every(mrl_ctx *ctx, int every);
int mrl_profile_end(mrl_ctx *ctx, int n_phases, double *total_ms, int *counts);

/* ------------------------------------------------------------------ environments
 * GPUDiscreteEnv / GPUContinuousEnv, core/env_traits.mojo:230-397:
 *   comptime STATE_SIZE / OBS_DIM / NUM_ACTIONS / ACTION_DIM   -> mrl_env_dims
 *   reset_kernel_gpu[B,S](ctx, states, rng_seed)               -> mrl_env_reset
 *   selective_reset_kernel_gpu[B,S](ctx, states, dones, seed)  -> mrl_env_selective_reset
 *   step_kernel_gpu[B,S,O](ctx, states, actions, rewards,
 *                          dones, obs, rng_seed)               -> mrl_env_step
 * states [batch, STATE_SIZE]; actions [batch] (discrete, stored as fp32) or
 * [batch, ACTION_DIM]; rewards, dones [batch]; obs [batch, OBS_DIM].
 * num_actions is 0 for continuous-only envs, action_dim 0 for discrete-only ones. */
int mrl_env_dims(int env_id, int *state_size, int *obs_dim, int *num_actions, int *action_dim);
int mrl_env_reset(mrl_ctx *ctx, int env_id, int batch, float *states, uint64_t seed);
int mrl_env_selective_reset(mrl_ctx *ctx, int env_id, int batch, float *states, float *dones,
                            uint64_t seed);
int mrl_env_step(mrl_ctx *ctx, int env_id, int batch, float *states, const float *actions,
                 float *rewards, float *dones, float *obs, uint64_t seed);
/* CartPole's state row has no slot for the step counter behind the 500-step truncation of the
 * reference's CPU step (envs/cartpole.mojo:454-457), so the counters live beside the rows: by
 * default in an int32[batch] array that the context creates, zeroed, on the first call that sees a
 * `states` pointer, and keeps until the context is destroyed.  This call puts them in the caller's
 * hands instead: `steps` (device, int32[batch], initialised by the caller) becomes the counter array
 * of `states` -- a caller that copies or moves its rows copies the counters along and binds them to
 * the new pointer.  steps = NULL forgets the pointer (and frees a library-made array). */
int mrl_cartpole_bind_steps(mrl_ctx *ctx, const float *states, int batch, int32_t *steps);
/* LunarLanderV2's struct parameters ENABLE_WIND / WIND_POWER / TURBULENCE_POWER
 * (envs/lunar_lander/lunar_lander_v2.mojo:123-127; defaults off, 15.0, 1.5) as a setting of the
 * context, for both action forms: while no leg touches the ground every step first adds
 * tanh(sin(0.02 t) + sin(pi 0.01 t)) * power as an impulse to the lander's vx (wind) and omega
 * (turbulence), computed in Float64 as _apply_wind does (:983-1023), with t = the row's step
 * count as in the GPU trait (:2041-2105).  Takes effect for steps enqueued after the call. */
int mrl_lunar_set_wind(mrl_ctx *ctx, int enable, double wind_power, double turbulence_power);
/* Which of the reference's two CarRacingV2 steps the context's env steps follow (plain and fused).  The
 * dynamics, the controls, the visited flags and the observation are the same in both; they differ in the
 * reward and in the precision of the termination tests:
 *   MRL_CAR_STEP_CPU_ENV (default)  CarRacingV2.step, car_racing_v2.mojo:258-287: reward -0.1 (+ 100 /
 *       tiles for a new tile) in Float64, -100 off the playfield, tests in Float64, episode total taken
 *       before the playfield penalty (:781-846);
 *   MRL_CAR_STEP_GPU_TRAIT          step_kernel_gpu, car_racing_v2.mojo:1556-1716, which the reference's
 *       train_gpu runs: reward 0.5 * (vx cos(angle) + vy sin(angle)) - 0.01 (+ 100 / tiles) in fp32 from
 *       the hull state after the physics, fp32 tests, episode total taken after the penalty.
 * Takes effect for steps enqueued after the call. */
enum { MRL_CAR_STEP_CPU_ENV = 0, MRL_CAR_STEP_GPU_TRAIT = 1 };
int mrl_car_racing_set_step_form(mrl_ctx *ctx, int form);
/* step, then re-initialise rows that finished with the selective-reset protocol, then write
 * obs from the (possibly fresh) row: the sequence step_kernel_gpu -> selective_reset_kernel_gpu
 * -> _extract_obs_from_state_kernel of deep_agents/ppo/ppo.mojo:2148-2285 in one launch.
 * rewards/dones report the step that just happened. */
int mrl_env_step_autoreset(mrl_ctx *ctx, int env_id, int batch, float *states, const float *actions,
                           float *rewards, float *dones, float *obs, uint64_t step_seed,
                           uint64_t reset_seed);

/* ------------------------------------------------------------------ MLP
 * Model.forward_gpu_no_cache_ws / forward_gpu_ws / backward_gpu_ws,
 * deep_rl/model/model.mojo:200-273; Seq2 chaining deep_rl/model/sequential.mojo:537-848.
 * params [L0|L1|...], each [W (in x out, row-major) | b] (+ log_std for the actor head);
 * cache (nullable) blocked per layer [batch x CACHE_i]; backward OVERWRITES grads.
 * No workspace argument: intermediates stay on chip. */
int mrl_mlp_param_size(const mrl_mlp_desc *desc);
int mrl_mlp_cache_size(const mrl_mlp_desc *desc); /* floats per sample */
int mrl_mlp_out_dim(const mrl_mlp_desc *desc);
int mrl_mlp_forward(mrl_ctx *ctx, const mrl_mlp_desc *desc, int batch, const float *in,
                    const float *params, float *out, float *cache);
int mrl_mlp_backward(mrl_ctx *ctx, const mrl_mlp_desc *desc, int batch, const float *grad_out,
                     const float *params, const float *cache, float *grads, float *grad_in);

/* ------------------------------------------------------------------ PPO pieces */

/* _sample_actions_kernel, deep_agents/ppo/ppo.mojo:4064-4123 */
int mrl_sample_categorical(mrl_ctx *ctx, const float *logits, int n, int num_actions, uint32_t seed,
                           float *actions, float *log_probs);
/* _sample_continuous_actions_kernel, deep_agents/ppo/kernels.mojo:12-98 */
int mrl_sample_gaussian(mrl_ctx *ctx, const float *actor_out, int n, int action_dim, uint32_t seed,
                        float *actions, float *log_probs);
/* add_obs_noise_kernel, deep_agents/ppo/kernels.mojo:882-925 (called at ppo_continuous.mojo:2557 and
 * :2705): obs[i, d] += noise_std * z with z standard normal from Philox(seed + i * obs_dim + d) by
 * Box-Muller, in place; nothing happens for noise_std <= 0. */
int mrl_add_obs_noise(mrl_ctx *ctx, float *obs, int n, int obs_dim, float noise_std, uint32_t seed);
/* The action of the evaluation policies without sampling.  continuous != 0: the mean of the
 * Gaussian head, actions[i, j] = actor_out[i, j] with actor_out rows [mean (A) | log_std (A)]
 * (extract_deterministic_actions in evaluate_gpu, deep_agents/ppo/ppo_continuous.mojo:807-822).
 * continuous == 0: the first index of the largest logit as a float, which is the argmax of the
 * softmax probabilities that select_action(training=False) takes (ppo.mojo:988-1027). */
int mrl_greedy_actions(mrl_ctx *ctx, const float *actor_out, int n, int num_actions, int continuous,
                       float *actions);
/* host GAE loop of train_gpu, deep_agents/ppo/ppo.mojo:2317-2353 (time-major, idx = t*N + env) */
int mrl_gae(mrl_ctx *ctx, int T, int N, const float *rewards, const float *values,
            const float *dones, const float *bootstrap, double gamma, double lam, float *adv,
            float *ret);
/* (x - mean) / (sqrt(var + 1e-8) + 1e-8) in place: ppo.mojo:2356-2371, :2478-2511 + :637-653,
 * kernels.mojo:507-599 */
int mrl_normalize_advantages(mrl_ctx *ctx, float *x, int n);
/* RunningMeanStd.update / normalize of the reward stream, core/utils/normalization.mojo:188-292
 * (used at deep_agents/ppo/ppo_continuous.mojo:2867-2871 on host copies).  state is a DEVICE
 * array of 3 doubles (count, mean, var_sum), zero-initialised by the caller; all sums in Float64. */
int mrl_rms_update(mrl_ctx *ctx, double *state, const float *x, int n);
int mrl_rms_normalize(mrl_ctx *ctx, const double *state, float *x, int n);
/* indices[0..n) = a pseudo-random permutation of 0..n-1 determined by seed; stands where the
 * reference runs a host Fisher-Yates shuffle (deep_agents/ppo/ppo.mojo:2425-2434,
 * core/utils/shuffle.mojo:21-82) and copies the indices to the device. */
int mrl_permutation(mrl_ctx *ctx, int32_t *indices, int n, uint64_t seed);
/* shuffle_indices, core/utils/shuffle.mojo:21-48 (the same loop inline at deep_agents/ppo/ppo.mojo:
 * 2425-2434), on draws that the caller supplies: indices[0..n) = the result of
 *     for i = n-1 .. 1:  j = min(Int(u * Float64(i + 1)), i);  swap(indices[i], indices[j])
 * started from 0..n-1, where iteration i takes u = uniforms[n - 1 - i] (device, Float64, n - 1 values in
 * [0, 1], i.e. the draws of random_float64() in the order the loop consumes them).  Index for index the
 * permutation of the serial loop, computed in parallel; workspace is device scratch of 2n + 1 int32.
 * A caller that feeds the reference's own random stream gets the reference's minibatches; without one,
 * mrl_permutation is the cheaper call. */
int mrl_permutation_from_uniforms(mrl_ctx *ctx, int32_t *indices, int n, const double *uniforms,
                                  int32_t *workspace);
/* mean of kl[0..mb) against target_kl on the device: flag[0] is set to 1 when the mean exceeds
 * target_kl (never cleared by the library), flag[1] receives the bits of the mean (flag holds 4
 * int32; [2] and [3] belong to mrl_ppo_update_minibatch).  Replaces
 * the per-minibatch D2H copy + host mean of ppo.mojo:2557-2573 / ppo_continuous.mojo:3062-3086. */
int mrl_kl_check(mrl_ctx *ctx, const float *kl, int mb, float target_kl, int32_t *flag);
/* params[i] = lo + u_i (hi - lo): the uniform fills behind Xavier / Kaiming
 * (deep_rl/initializer/initializers.mojo:69-104) and StochasticActor.init_params_small
 * (deep_rl/model/stochastic_actor.mojo:95-128); u from Philox(seed). */
int mrl_init_uniform(mrl_ctx *ctx, float *params, int n, float lo, float hi, uint64_t seed);
/* ppo_gather_minibatch_kernel ppo.mojo:135-191 / kernels.mojo:161-226: rows of the rollout
 * buffers picked by int32 indices */
int mrl_gather_minibatch(mrl_ctx *ctx, const int32_t *indices, int mb, int obs_dim, int act_dim,
                         const float *r_obs, const float *r_actions, const float *r_adv,
                         const float *r_ret, const float *r_logp, const float *r_values,
                         float *mb_obs, float *mb_actions, float *mb_adv, float *mb_ret,
                         float *mb_logp, float *mb_values);
/* ppo_actor_grad_with_kl_kernel, ppo.mojo:285-378 */
int mrl_ppo_actor_grad_discrete(mrl_ctx *ctx, const float *logits, const float *old_log_probs,
                                const float *advantages, const float *actions, int mb,
                                int num_actions, float clip_eps, float entropy_coef,
                                float *grad_logits, float *kl);
/* ppo_continuous_actor_grad_kernel, kernels.mojo:230-412 */
int mrl_ppo_actor_grad_gaussian(mrl_ctx *ctx, const float *actor_out, const float *old_log_probs,
                                const float *advantages, const float *actions, int mb,
                                int action_dim, float clip_eps, float entropy_coef, float *grad_out,
                                float *kl);
/* convention 0: ppo.mojo:538-633 (2*c_v*(V-R)/MB); convention 1: kernels.mojo:416-486 ((V-R)/MB) */
int mrl_ppo_critic_grad(mrl_ctx *ctx, const float *values, const float *old_values,
                        const float *returns, int mb, int convention, int clipped, float value_coef,
                        float clip_eps, float *grad_values);
/* gradient_norm_kernel + reduce + apply, ppo.mojo:382-534 / kernels.mojo:603-805; in place */
int mrl_clip_grad_norm(mrl_ctx *ctx, float *grads, int n, float max_norm);
/* mrl_clip_grad_norm for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * per-block partial sums live in a file-scope device array of 1 KiB that every device holds from
 * library load to process end, instead of in memory obtained from hipMalloc; its address is looked
 * up by mrl_ctx_create.  The call allocates and frees nothing, and gives the results of
 * mrl_clip_grad_norm bit for bit.  n is limited to MRL_CLIP_STATIC_MAX_N elements; a larger n is
 * rejected with MRL_E_ARG.  All calls on one device share that device's array: calls that overlap
 * on one device (two streams, two threads) race. */
#define MRL_CLIP_STATIC_MAX_N (1 << 24)
int mrl_clip_grad_norm_static(mrl_ctx *ctx, float *grads, int n, float max_norm);
/* Adam.step_gpu, deep_rl/optimizer/adam.mojo:52-105, :162-247.  t is the optimiser's step count
 * AFTER the increment (1 on the first call); state is [n, 2] interleaved (m, v). */
int mrl_adam_step(mrl_ctx *ctx, float *params, const float *grads, float *state, int n, int t,
                  double lr, double beta1, double beta2, double eps);
/* clamp_log_std_params_kernel, kernels.mojo:842-873 */
int mrl_clamp_log_std(mrl_ctx *ctx, float *params, int offset, int action_dim);

/* ------------------------------------------------------------------ fused rollout step
 * One time step of train_gpu's collection loop (deep_agents/ppo/ppo.mojo:2069-2285 for a
 * discrete-action env, deep_agents/ppo/ppo_continuous.mojo:2619-2850 for a continuous one):
 * actor + critic forward on obs, categorical or Gaussian sampling, store of (obs, action,
 * log_prob, value) into rollout row t, env step with auto-reset, store of (reward, done), episode accounting.  The rollout buffers are the
 * reference's time-major ones ([T*N, ...], row = t*N + env); ep_return / ep_length are
 * the per-env accumulators of deep_rl/gpu/rl_kernels.mojo:103-227; finished episodes are
 * appended to done_returns / done_lengths (capacity done_cap) through the counter
 * done_count instead of being copied to the host every step. */
/* Policy half of a collection step for a discrete-action agent, one launch when both nets are
 * IN -> H -> H -> out with H in {64, 256} and ReLU or tanh hidden layers (layer by layer
 * otherwise): actor + critic forward (Model.forward_gpu_no_cache_ws, ppo.mojo:2073-2090),
 * _sample_actions_kernel (ppo.mojo:4064-4123) and _store_pre_step_kernel (ppo.mojo:662-690).
 * actions [n] feeds the env step; r_* are the rollout rows of this time step. */
int mrl_policy_step_discrete(mrl_ctx *ctx, const mrl_mlp_desc *actor, const mrl_mlp_desc *critic, int n,
                             const float *obs, const float *actor_params, const float *critic_params,
                             uint32_t seed, float *actions, float *r_obs, float *r_actions,
                             float *r_log_probs, float *r_values);

/* Same for a continuous-action agent (deep_agents/ppo/ppo_continuous.mojo:2619-2686): the actor
 * ends in a StochasticActor head, actions [n, A] are drawn as in kernels.mojo:12-98. */
int mrl_policy_step_gaussian(mrl_ctx *ctx, const mrl_mlp_desc *actor, const mrl_mlp_desc *critic, int n,
                             const float *obs, const float *actor_params, const float *critic_params,
                             uint32_t seed, float *actions, float *r_obs, float *r_actions,
                             float *r_log_probs, float *r_values);

/* num_actions > 0: discrete agent (r_actions [T*N]); num_actions == 0: continuous agent whose
 * actor ends in a StochasticActor head of the env's ACTION_DIM (r_actions [T*N, ACTION_DIM]). */
typedef struct {
    int32_t env_id, n_envs, obs_dim, num_actions;
    float *states, *obs;                     /* [N, STATE_SIZE], [N, OBS] current observation */
    const float *actor_params, *critic_params;
    mrl_mlp_desc actor, critic;
    float *r_obs, *r_actions, *r_log_probs, *r_values, *r_rewards, *r_dones; /* rollout buffers */
    float *ep_return, *ep_length;            /* [N] */
    float *done_returns, *done_lengths;      /* [done_cap] */
    int32_t *done_count;                     /* [1] */
    int32_t done_cap;
} mrl_rollout;

int mrl_rollout_step(mrl_ctx *ctx, const mrl_rollout *r, int t, uint32_t sample_seed,
                     uint64_t step_seed, uint64_t reset_seed);

/* The collection loop itself, `for t in range(rollout_len)` of train_gpu (deep_agents/ppo/ppo.mojo:
 * 2058-2293, ppo_continuous.mojo:2600-2850): steps t0 .. t0 + n_steps - 1 of the rollout, step
 * t0 + k with the seeds  sample_seed + k * sample_stride (mod 2^32),  step_seed + k * step_stride
 * and reset_seed + k * reset_stride (mod 2^64) -- the reference derives its per-step seeds from
 * the step counter in the same affine way.  Buffers end up as after n_steps calls of
 * mrl_rollout_step with those seeds, except that the order of the finished-episode list
 * (done_returns / done_lengths) inside the call is unspecified.  Where the env and the networks
 * allow it (LunarLander with hidden width 256; CartPole and Pendulum with hidden width 64) the
 * whole range is ONE launch: each workgroup keeps its 32 envs on the chip (rows in LDS, or state
 * in registers for the two small envs) and alternates policy forward and env step on them, so
 * states and observations cross HBM once per call instead of twice per step; otherwise the
 * steps are issued one by one.  Enqueue only. */
int mrl_rollout_steps(mrl_ctx *ctx, const mrl_rollout *r, int t0, int n_steps, uint32_t sample_seed,
                      uint32_t sample_stride, uint64_t step_seed, uint64_t step_stride,
                      uint64_t reset_seed, uint64_t reset_stride);
/* 1 when mrl_rollout_steps runs this descriptor as one launch per call, 0 when it issues the
 * steps one by one (no counterpart in the reference: a caller that times launches asks this). */
int mrl_rollout_fused(const mrl_rollout *r);

/* ------------------------------------------------------------------ minibatch update
 * The body of train_gpu's minibatch loop (deep_agents/ppo/ppo.mojo:2438-2727 for DeepPPOAgent,
 * deep_agents/ppo/ppo_continuous.mojo:3000-3260 for DeepPPOContinuousAgent) as one enqueue-only
 * call: gather the rows `indices` of the rollout, normalise the minibatch's advantages, actor
 * forward / loss gradient (+ per-sample KL) / backward / global-norm clip / Adam (/ log_std
 * clamp), and the same for the critic.  On return (in stream order) the parameter and optimiser
 * buffers are updated in place and actor_grads / critic_grads hold the clipped gradients.
 * continuous = 0: logits head, critic gradient 2 c_v (V - R) / MB; continuous = 1: StochasticActor
 * head, critic gradient (V - R) / MB.  actor_t / critic_t are the optimisers' step counts after
 * this step (Adam.t += 1 stays on the host, deep_rl/optimizer/adam.mojo:170).
 * KL early stop (target_kl > 0): the mean KL is tested on the device; kl_flag is 4 int32 --
 * [0] raised (and left raised) when a minibatch's mean KL exceeds target_kl, [1] bits of the
 * last mean, [2] number of updates applied since the caller cleared it; once [0] is up the call
 * still computes gradients but leaves parameters and optimiser state untouched, which is where
 * the reference's `break` (ppo.mojo:2566-2573) leaves them. */
typedef struct {
    int32_t minibatch, obs_dim, act_width, continuous;
    mrl_mlp_desc actor, critic;
    float *actor_params, *critic_params;
    float *actor_grads, *critic_grads;
    float *actor_state, *critic_state;       /* Adam (m, v) interleaved, [P, 2] */
    const float *r_obs, *r_actions, *r_log_probs, *r_values, *advantages, *returns; /* [T*N, ...] */
    float *mb_obs, *mb_actions, *mb_adv, *mb_ret, *mb_logp, *mb_val;                /* [MB, ...] scratch: the gathered
                                                 minibatch when the nets run layer by layer, untouched when the fused
                                                 forward reads the rollout rows itself */
    float *actor_out, *values, *g_actor_out, *g_values, *kl;
    float *actor_cache, *critic_cache;       /* [MB * CACHE_SIZE] */
    int32_t *kl_flag;                        /* [4], may be NULL when target_kl <= 0 */
    float clip_epsilon, entropy_coef, value_loss_coef, max_grad_norm, target_kl;
    int32_t clip_value, norm_adv_per_minibatch;
    double actor_lr, critic_lr, beta1, beta2, eps;
} mrl_update;

int mrl_ppo_update_minibatch(mrl_ctx *ctx, const mrl_update *u, const int32_t *indices, int actor_t,
                             int critic_t);
/* n_minibatches consecutive minibatches of `indices` (a permutation of the rollout); minibatch k
 * runs with step counts actor_t0 + k + 1 / critic_t0 + k + 1 */
int mrl_ppo_update_epoch(mrl_ctx *ctx, const mrl_update *u, const int32_t *indices, int n_minibatches,
                         int actor_t0, int critic_t0);

/* The statistics that the fused update normalises a minibatch's advantages with
 * (deep_agents/ppo/ppo.mojo:2478-2511 with the kernel at :637-653 -- mean and variance over the
 * minibatch's gathered advantages): stats[2k] = mean, stats[2k + 1] = sqrt(variance + 1e-8) of the
 * rows indices[k * minibatch .. (k + 1) * minibatch) of `advantages`, for k < n_minibatches.  This is
 * the launch mrl_ppo_update_epoch makes ahead of its minibatches, written to the caller's buffer
 * (device, 2 * n_minibatches floats); a normalised advantage is (A - mean) / (stats[2k + 1] + 1e-8). */
int mrl_minibatch_adv_stats(mrl_ctx *ctx, const int32_t *indices, const float *advantages, int minibatch,
                            int n_minibatches, float *stats);

#ifdef __cplusplus
}
#endif
#endif
