// Fused collection-step policy kernel:
//   actor  IN -> H -> H -> A   and   critic  IN -> H -> H -> 1   (ReLU or tanh hidden layers),
//   action sampling, and the pre-step rollout stores, in ONE launch.
// Discrete agents: logits head + categorical sampling.  It replaces, per time step of
// deep_agents/ppo/ppo.mojo:2069-2146, six tiled-matmul launches, _sample_actions_kernel
// (ppo.mojo:4064-4123) and _store_pre_step_kernel (ppo.mojo:662-690).
// Continuous agents: StochasticActor head [mean | clamp(log_std)] + Gaussian sampling
// (deep_agents/ppo/ppo_continuous.mojo:2619-2686, deep_agents/ppo/kernels.mojo:12-98).
//
// One workgroup = 32 environments (rows) and 2H threads: threads [0, H) run the actor, threads
// [H, 2H) the critic, side by side (two wavefronts per SIMD hide each other's LDS and L2
// latencies).  The 32 x H hidden activations never leave the CU:
//   layers 0 and 1:         fp32 MFMA 32x32x2, each wavefront owns 64 output columns (two
//                           accumulator tiles), A operand from LDS, B operand (the weights)
//                           streamed from L2 a block of k-steps ahead of the MFMAs that use it
//                           -- all workgroups read the same 256 KB;
//   layer 2 (N = A or 1):   H/32 lanes per row, shuffle reduction.
// With 8192 envs this is 256 workgroups of 8 wavefronts: one per CU of the MI355X.
#include "mrl_host.hpp"
#include "mrl_device.hpp"
#include "mlp_tile.hpp"
#include "policy_sample.hpp"

namespace mrl {

static_assert(SAMPLE_A_MAX == PA_MAX, "the sampler's action limit is the policy tile's");

template <int H, int ACT, bool GAUSS, int TPW>
__global__ __launch_bounds__(TPW == 1 ? 2 * H : 4 * H / TPW) void policy_kernel(
    const float *__restrict__ obs, int n, int IN, int A, const float *__restrict__ actor_p,
    const float *__restrict__ critic_p, uint32_t seed, float *__restrict__ actions,
    float *__restrict__ r_obs, float *__restrict__ r_actions, float *__restrict__ r_logp,
    float *__restrict__ r_values) {
    __shared__ float xs[PR * XS_LD];
    __shared__ float hT[2][H * HT_LD];
    __shared__ float h2[2][PR * (H + 1)];
    __shared__ float logits[PR * (PA_MAX + 1)];
    __shared__ float vals[PR];
    __shared__ __align__(16) float w2s[2][HEAD_LDS(H)];
    constexpr int TN = 2 * H / TPW;          // threads per net
    // a block works on both nets (2 TN threads) or, launched with TN threads and grid.y = 2, on the
    // net blockIdx.y alone: a batch of few row tiles then spreads over twice as many CUs
    const int t = threadIdx.x, nthr = blockDim.x;
    const int net = t / TN + blockIdx.y;     // 0 = actor, 1 = critic
    const bool has_actor = blockIdx.y == 0, has_critic = nthr > TN || blockIdx.y == 1;
    const int row0 = blockIdx.x * PR;
    const int nrow = min(PR, n - row0);

    // every load that does not depend on an earlier phase goes out first: the net's operands, its
    // head parameters, the observation tile (rows beyond the batch read as zero; the tile also goes
    // straight out to rollout[t])
    const float *p = net ? critic_p : actor_p;
    HiddenOperands<H, TPW, 8> ops;
    ops.load(p, IN);
    float xv[(PR * PIN_MAX + TN - 1) / TN];
#pragma unroll
    for (int q = 0; q < (int)(sizeof(xv) / sizeof(float)); ++q) {
        const int i = t + q * nthr;
        xv[q] = (i < PR * IN && i / IN < nrow) ? obs[(long)row0 * IN + i] : 0.0f;
    }
    stage_head(p + IN * H + H + H * H + H, H, net ? 1 : A, GAUSS && net == 0, w2s[net], t % TN, TN);
#pragma unroll
    for (int q = 0; q < (int)(sizeof(xv) / sizeof(float)); ++q) {
        const int i = t + q * nthr;
        if (i < PR * IN) {
            const int r = i / IN, k = i - r * IN;
            xs[r * XS_LD + k] = xv[q];
            if (r < nrow && has_actor) r_obs[(long)row0 * IN + i] = xv[q];
        }
    }
    __syncthreads();

    hidden_stack<H, ACT, TPW, 8>(p, IN, xs, hT[net], h2[net], TileCache{}, ops);
    if (net == 0) head<H>(w2s[0], A, h2[0], logits, PA_MAX + 1, t % TN, TN);
    else head<H>(w2s[1], 1, h2[1], vals, 1, t % TN, TN);
    __syncthreads();

    if (t < nrow && has_critic) r_values[row0 + t] = vals[t];
    if (t < nrow && !GAUSS && has_actor) {   // categorical sampling, one lane per env
        const int i = row0 + t;
        int sel;
        float logp;
        sample_categorical_few(logits + t * (PA_MAX + 1), A, seed, i, sel, logp);
        actions[i] = (float)sel;
        r_actions[i] = (float)sel;
        r_logp[i] = logp;
    }
    if (GAUSS && has_actor) {
        // Gaussian sampling, one lane per (env, action component): the components have Philox streams of
        // their own; the log-probability is their sum in component order, taken by the env's lane
        __shared__ float part[PR * PA_MAX];
        for (int e = t; e < nrow * A; e += nthr) {
            const int r = e / A, j = e - r * A;
            float act;
            part[r * PA_MAX + j] = sample_gaussian_part(logits + r * (PA_MAX + 1) + j, w2s[0] + HEAD_LOG_STD(H) + j, 1, A,
                                                        j, seed, row0 + r, &act);
            actions[(long)row0 * A + e] = act;
            r_actions[(long)row0 * A + e] = act;
        }
        __syncthreads();
        if (t < nrow) {
            float logp = 0.0f;
            for (int j = 0; j < A; ++j) logp = logp + part[t * PA_MAX + j];
            r_logp[row0 + t] = logp;
        }
    }
}

// true when the pair (actor, critic) has the shape this kernel is specialised for
constexpr int PTPW = 2;   // accumulator tiles per wavefront in the policy kernel (1 measured no faster)
constexpr int POLICY_SPLIT_BELOW = 256;   // CUs of the MI355X: up to this many workgroups run side by side

bool policy_fusable(const mrl_mlp_desc &a, const mrl_mlp_desc &c, bool gauss, int *H, int *act) {
    if (a.n_layers != 3 || c.n_layers != 3) return false;
    const int k0 = a.layers[0].kind;
    if (k0 != MRL_LINEAR_RELU && k0 != MRL_LINEAR_TANH) return false;
    for (const mrl_mlp_desc *d : {&a, &c}) {
        if (d->layers[0].kind != k0 || d->layers[1].kind != k0) return false;
        if (d->layers[0].in_dim != a.layers[0].in_dim || d->layers[0].in_dim > PIN_MAX) return false;
        if (d->layers[0].out_dim != a.layers[0].out_dim || d->layers[1].out_dim != a.layers[0].out_dim)
            return false;
    }
    if (a.layers[2].kind != (gauss ? MRL_STOCHASTIC_ACTOR : MRL_LINEAR) || c.layers[2].kind != MRL_LINEAR)
        return false;
    const int h = a.layers[0].out_dim;
    if (h != 64 && h != 256) return false;
    if (a.layers[2].out_dim > PA_MAX || c.layers[2].out_dim != 1) return false;
    *H = h;
    *act = (k0 == MRL_LINEAR_RELU) ? 1 : 2;
    return true;
}

int launch_policy(mrl_ctx *ctx, const mrl_mlp_desc &a, const mrl_mlp_desc &c, bool gauss, const float *obs,
                  int n, const float *ap, const float *cp, uint32_t seed, float *actions, float *r_obs,
                  float *r_actions, float *r_logp, float *r_values) {
    int H = 0, act = 0;
    if (!policy_fusable(a, c, gauss, &H, &act)) return MRL_E_UNSUPPORTED;
    const int IN = a.layers[0].in_dim, A = a.layers[2].out_dim;
    // few row tiles: actor and critic of a tile go to workgroups of their own (twice the CUs at work),
    // at hidden width 256 with one column tile per wavefront (eight wavefronts per net: two per SIMD,
    // where a workgroup of four would leave each SIMD a single wavefront with nothing to overlap)
    const int tiles = (n + PR - 1) / PR;
    const bool split = 2 * tiles <= POLICY_SPLIT_BELOW;
    dim3 grid(tiles, split ? 2 : 1);
#define MRL_LAUNCH(HH, AA, GG)                                                                         \
    if (split && HH == 256)                                                                             \
        hipLaunchKernelGGL((policy_kernel<HH, AA, GG, 1>), grid, dim3(2 * HH), 0, ctx->stream, obs,     \
                           n, IN, A, ap, cp, seed, actions, r_obs, r_actions, r_logp, r_values);        \
    else                                                                                                \
        hipLaunchKernelGGL((policy_kernel<HH, AA, GG, PTPW>), grid, dim3((split ? 2 : 4) * HH / PTPW), 0, ctx->stream, obs, \
                           n, IN, A, ap, cp, seed, actions, r_obs, r_actions, r_logp, r_values)
    if (gauss) {
        if (H == 256 && act == 1) MRL_LAUNCH(256, 1, true);
        else if (H == 256 && act == 2) MRL_LAUNCH(256, 2, true);
        else if (H == 64 && act == 1) MRL_LAUNCH(64, 1, true);
        else MRL_LAUNCH(64, 2, true);
    } else {
        if (H == 256 && act == 1) MRL_LAUNCH(256, 1, false);
        else if (H == 256 && act == 2) MRL_LAUNCH(256, 2, false);
        else if (H == 64 && act == 1) MRL_LAUNCH(64, 1, false);
        else MRL_LAUNCH(64, 2, false);
    }
#undef MRL_LAUNCH
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

}  // namespace mrl
