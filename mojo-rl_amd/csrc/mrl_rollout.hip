// One time step of the PPO collection loop (deep_agents/ppo/ppo.mojo:2069-2285) without any
// host round trip, in two launches: [policy + value forward, sampling, pre-step stores] and
// [env step with auto-reset, post-step stores, episode accounting].  Finished episodes are appended to a device-side list through
// a counter instead of being copied to the host after every step.
#include "mrl_host.hpp"
#include "mrl_device.hpp"
#include "policy_sample.hpp"

namespace mrl {

int launch_policy(mrl_ctx *ctx, const mrl_mlp_desc &a, const mrl_mlp_desc &c, bool gauss, const float *obs,
                  int n, const float *ap, const float *cp, uint32_t seed, float *actions, float *r_obs,
                  float *r_actions, float *r_logp, float *r_values);

// sampling (ppo.mojo:4064-4123) fused with _store_pre_step_kernel (ppo.mojo:662-690):
// rollout row t gets obs, action, log-prob and value; `actions` feeds the env step.
__global__ __launch_bounds__(256) void sample_store_kernel(
    const float *__restrict__ logits, const float *__restrict__ values, const float *__restrict__ obs,
    int n, int A, int obs_dim, uint32_t seed, float *__restrict__ actions, float *__restrict__ r_obs,
    float *__restrict__ r_actions, float *__restrict__ r_logp, float *__restrict__ r_values) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int sel;
    float logp;
    sample_categorical(logits + (long)i * A, A, seed, i, sel, logp);
    actions[i] = (float)sel;
    r_actions[i] = (float)sel;
    r_logp[i] = logp;
    r_values[i] = values[i];
    for (int k = 0; k < obs_dim; ++k) r_obs[(long)i * obs_dim + k] = obs[(long)i * obs_dim + k];
}

// continuous counterpart: _sample_continuous_actions_kernel (kernels.mojo:12-98) fused with
// the pre-step store (ppo_continuous.mojo:2672-2686)
__global__ __launch_bounds__(256) void sample_store_gaussian_kernel(
    const float *__restrict__ actor_out, const float *__restrict__ values, const float *__restrict__ obs,
    int n, int A, int obs_dim, uint32_t seed, float *__restrict__ actions, float *__restrict__ r_obs,
    float *__restrict__ r_actions, float *__restrict__ r_logp, float *__restrict__ r_values) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float act[16];
    const float *head = actor_out + (long)i * 2 * A;   // [mean (A) | log_std (A)]
    float total = 0.0f;
    for (int j0 = 0; j0 < A; j0 += 16) {   // any action width, 16 components at a time
        const int m = min(16, A - j0);
        total = total + sample_gaussian_part(head + j0, head + A + j0, m, A, j0, seed, i, act);
        for (int j = 0; j < m; ++j) {
            actions[(long)i * A + j0 + j] = act[j];
            r_actions[(long)i * A + j0 + j] = act[j];
        }
    }
    r_logp[i] = total;
    r_values[i] = values[i];
    for (int k = 0; k < obs_dim; ++k) r_obs[(long)i * obs_dim + k] = obs[(long)i * obs_dim + k];
}

}  // namespace mrl

using namespace mrl;

extern "C" {

// floats per env after the policy temporaries: actions (<= 8), reward, done
#define MRL_ROLLOUT_TAIL 10

// layer-by-layer fallback needs logits/values temporaries
static int ensure_rollout_ws(mrl_ctx *ctx, size_t need) {
    return mrl::grow_workspace(ctx, &ctx->rollout_ws, &ctx->rollout_ws_floats, need);
}

static int policy_step(mrl_ctx *ctx, const char *who, bool gauss, const mrl_mlp_desc *actor,
                       const mrl_mlp_desc *critic, int n, const float *obs, const float *actor_params,
                       const float *critic_params, uint32_t seed, float *actions, float *r_obs,
                       float *r_actions, float *r_log_probs, float *r_values) {
    MRL_CHECK_ARG(ctx && actor && critic, "%s: NULL argument", who);
    MRL_CHECK_ARG(n >= 0, "%s: negative n", who);
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(obs && actor_params && critic_params && actions && r_obs && r_actions && r_log_probs &&
                      r_values, "%s: NULL buffer", who);
    MRL_CHECK_ARG(actor->n_layers >= 1 && actor->n_layers <= MRL_MAX_LAYERS && critic->n_layers >= 1 &&
                      critic->n_layers <= MRL_MAX_LAYERS, "%s: bad layer count", who);
    const bool head_is_actor = actor->layers[actor->n_layers - 1].kind == MRL_STOCHASTIC_ACTOR;
    MRL_CHECK_ARG(head_is_actor == gauss,
                  gauss ? "%s: actor must end in a StochasticActor head" : "%s: actor must end in logits", who);
    const int na = mrl_mlp_out_dim(actor), nv = mrl_mlp_out_dim(critic);   // na = 2A for a Gaussian actor
    MRL_CHECK_ARG(na > 0 && nv == 1, "%s: critic must end in 1 value", who);
    MRL_CHECK_ARG(actor->layers[0].in_dim == critic->layers[0].in_dim,
                  "%s: actor and critic read different observation widths", who);
    const int od = actor->layers[0].in_dim;
    profile_mark(ctx, -1);
    int rc = launch_policy(ctx, *actor, *critic, gauss, obs, n, actor_params, critic_params, seed, actions,
                           r_obs, r_actions, r_log_probs, r_values);
    if (rc == MRL_OK) {
        profile_mark(ctx, MRL_PHASE_POLICY_FWD);
        return MRL_OK;
    }
    if (rc != MRL_E_UNSUPPORTED) return rc;
    rc = ensure_rollout_ws(ctx, (size_t)n * (na + 1) + (size_t)n * (MRL_ROLLOUT_TAIL));
    if (rc) return rc;
    float *head = ctx->rollout_ws, *values = head + (size_t)n * na;
    rc = mrl_mlp_forward(ctx, actor, n, obs, actor_params, head, nullptr);
    if (rc) return rc;
    rc = mrl_mlp_forward(ctx, critic, n, obs, critic_params, values, nullptr);
    if (rc) return rc;
    profile_mark(ctx, MRL_PHASE_POLICY_FWD);
    if (gauss)
        hipLaunchKernelGGL(sample_store_gaussian_kernel, dim3(grid_for(n, 256)), dim3(256), 0, ctx->stream,
                           head, values, obs, n, na / 2, od, seed, actions, r_obs, r_actions, r_log_probs,
                           r_values);
    else
        hipLaunchKernelGGL(sample_store_kernel, dim3(grid_for(n, 256)), dim3(256), 0, ctx->stream, head,
                           values, obs, n, na, od, seed, actions, r_obs, r_actions, r_log_probs, r_values);
    MRL_CHECK_LAUNCH();
    profile_mark(ctx, MRL_PHASE_SAMPLE);
    return MRL_OK;
}

int mrl_policy_step_discrete(mrl_ctx *ctx, const mrl_mlp_desc *actor, const mrl_mlp_desc *critic, int n,
                             const float *obs, const float *actor_params, const float *critic_params,
                             uint32_t seed, float *actions, float *r_obs, float *r_actions,
                             float *r_log_probs, float *r_values) {
    return policy_step(ctx, "mrl_policy_step_discrete", false, actor, critic, n, obs, actor_params,
                       critic_params, seed, actions, r_obs, r_actions, r_log_probs, r_values);
}

int mrl_policy_step_gaussian(mrl_ctx *ctx, const mrl_mlp_desc *actor, const mrl_mlp_desc *critic, int n,
                             const float *obs, const float *actor_params, const float *critic_params,
                             uint32_t seed, float *actions, float *r_obs, float *r_actions,
                             float *r_log_probs, float *r_values) {
    return policy_step(ctx, "mrl_policy_step_gaussian", true, actor, critic, n, obs, actor_params,
                       critic_params, seed, actions, r_obs, r_actions, r_log_probs, r_values);
}

int mrl_rollout_step(mrl_ctx *ctx, const mrl_rollout *r, int t, uint32_t sample_seed,
                     uint64_t step_seed, uint64_t reset_seed) {
    MRL_CHECK_ARG(ctx && r, "mrl_rollout_step: NULL argument");
    MRL_CHECK_ARG(r->n_envs > 0 && t >= 0, "mrl_rollout_step: bad sizes");
    MRL_CHECK_ARG(r->states && r->obs && r->actor_params && r->critic_params && r->r_obs &&
                      r->r_actions && r->r_log_probs && r->r_values && r->r_rewards && r->r_dones &&
                      r->ep_return && r->ep_length && r->done_returns && r->done_lengths && r->done_count,
                  "mrl_rollout_step: NULL buffer in descriptor");
    int ss, od, na, ad;
    int rc = mrl_env_dims(r->env_id, &ss, &od, &na, &ad);
    if (rc) return rc;
    const bool gauss = r->num_actions == 0;
    MRL_CHECK_ARG(od == r->obs_dim && (gauss ? ad > 0 : (na > 0 && na == r->num_actions)),
                  "mrl_rollout_step: descriptor does not match the env's observation / action space");
    const int head = gauss ? 2 * ad : na;    // width of the actor's output
    const int aw = gauss ? ad : 1;           // floats per stored action
    MRL_CHECK_ARG(mrl_mlp_out_dim(&r->actor) == head && r->actor.layers[0].in_dim == od,
                  "mrl_rollout_step: actor must map obs_dim to the env's action head");
    const int N = r->n_envs;
    rc = ensure_rollout_ws(ctx, (size_t)N * (head + 1) + (size_t)N * MRL_ROLLOUT_TAIL);
    if (rc) return rc;
    // [head N*head | values N] are used by the layer-by-layer policy path; the tail holds the
    // step's actions (up to 8 per env), rewards and dones
    float *actions = ctx->rollout_ws + (size_t)N * (head + 1);
    float *rewards = actions + (size_t)N * 8, *dones = rewards + N;
    const size_t row = (size_t)t * N;
    profile_step_begin(ctx);
    rc = policy_step(ctx, "mrl_rollout_step", gauss, &r->actor, &r->critic, N, r->obs, r->actor_params,
                     r->critic_params, sample_seed, actions, r->r_obs + row * od, r->r_actions + row * aw,
                     r->r_log_probs + row, r->r_values + row);
    if (rc) {
        profile_step_end(ctx);
        return rc;
    }
    profile_mark(ctx, -1);
    // the env-step kernel also stores (reward, done) into rollout row t and does the episode
    // accounting for its envs
    const Accounting acc{r->r_rewards + row, r->r_dones + row, r->ep_return, r->ep_length,
                         r->done_returns, r->done_lengths, r->done_count, r->done_cap};
    rc = env_step_accounting(ctx, r->env_id, N, r->states, actions, rewards, dones, r->obs, step_seed,
                             reset_seed, acc);
    if (rc == MRL_OK) profile_mark(ctx, MRL_PHASE_ENV);
    profile_step_end(ctx);
    return rc;
}

}  // extern "C"
