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

namespace mrl {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int PR = 32;        // rows (envs) per workgroup
constexpr int PIN_MAX = 32;   // max observation width
constexpr int PA_MAX = 8;     // max number of discrete actions
constexpr int XS_LD = PIN_MAX + 1;
constexpr int HT_LD = PR + 1;

template <int ACT>
MRL_DEV float activate(float x) {
    if (ACT == 1) return x > 0.0f ? x : 0.0f;
    if (ACT == 2) return tanhf(x);
    return x;
}

// hidden stack of one net for the block's 32 rows; leaves act(layer1) in h2[32][H+1]
template <int H, int ACT>
MRL_DEV void hidden_stack(const float *__restrict__ p, int IN, const float *xs, float *hT, float *h2) {
    const int t = threadIdx.x % H, lane = t & 63, w = t >> 6, half = lane >> 5, l31 = lane & 31;
    const float *W0 = p, *b0 = p + IN * H;
    const float *W1 = b0 + H, *b1 = W1 + H * H;
    const int col0 = 64 * w + l31, col1 = col0 + 32;
    {   // layer 0 (K = IN <= 32, padded to even with zeros): wavefront w owns columns [64w, 64w + 64)
        floatx16 c0 = {0}, c1 = {0};
        for (int kk = 0; kk < (IN + 1) / 2; ++kk) {
            const int k = 2 * kk + half;
            const bool in = k < IN;
            const float a = in ? xs[l31 * XS_LD + k] : 0.0f;
            const float bv0 = in ? W0[k * H + col0] : 0.0f;
            const float bv1 = in ? W0[k * H + col1] : 0.0f;
            c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bv0, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bv1, c1, 0, 0, 0);
        }
        const float bb0 = b0[col0], bb1 = b0[col1];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = 8 * (v >> 2) + 4 * half + (v & 3);
            hT[col0 * HT_LD + row] = activate<ACT>(c0[v] + bb0);
            hT[col1 * HT_LD + row] = activate<ACT>(c1[v] + bb1);
        }
    }
    __syncthreads();
    {   // layer 1 (H x H): weights streamed from L2 one block of KB k-steps ahead of the MFMAs
        constexpr int KB = 8;
        floatx16 c0 = {0}, c1 = {0};
        const float *Wc = W1 + col0;
        float a[KB], bv0[KB], bv1[KB], na[KB], nb0[KB], nb1[KB];
#pragma unroll
        for (int j = 0; j < KB; ++j) {
            const int k = 2 * j + half;
            a[j] = hT[k * HT_LD + l31];
            bv0[j] = Wc[k * H];
            bv1[j] = Wc[k * H + 32];
        }
        for (int blk = 0; blk < H / (2 * KB); ++blk) {
            const bool more = blk + 1 < H / (2 * KB);
            if (more) {
#pragma unroll
                for (int j = 0; j < KB; ++j) {
                    const int k = 2 * ((blk + 1) * KB + j) + half;
                    na[j] = hT[k * HT_LD + l31];
                    nb0[j] = Wc[k * H];
                    nb1[j] = Wc[k * H + 32];
                }
            }
#pragma unroll
            for (int j = 0; j < KB; ++j) {
                c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], bv0[j], c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], bv1[j], c1, 0, 0, 0);
            }
            if (more) {
#pragma unroll
                for (int j = 0; j < KB; ++j) { a[j] = na[j]; bv0[j] = nb0[j]; bv1[j] = nb1[j]; }
            }
        }
        const float bb0 = b1[col0], bb1 = b1[col1];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = 8 * (v >> 2) + 4 * half + (v & 3);
            h2[row * (H + 1) + col0] = activate<ACT>(c0[v] + bb0);
            h2[row * (H + 1) + col1] = activate<ACT>(c1[v] + bb1);
        }
    }
    __syncthreads();
}

// out[r][a] = h2[r] . W2[:, a] + b2[a] for the block's rows; TPR = H/32 lanes cooperate per row
template <int H>
MRL_DEV void head(const float *__restrict__ W2, int A, const float *h2, float *out, int out_ld) {
    constexpr int TPR = H / PR;
    const int t = threadIdx.x % H, r = t / TPR, part = t % TPR;
    const float *b2 = W2 + H * A;
    float acc[PA_MAX];
#pragma unroll
    for (int a = 0; a < PA_MAX; ++a) acc[a] = 0.0f;
    for (int i = 0; i < PR; ++i) {
        const int n = i * TPR + part;
        const float hv = h2[r * (H + 1) + n];
#pragma unroll
        for (int a = 0; a < PA_MAX; ++a)
            if (a < A) acc[a] = fmaf(hv, W2[n * A + a], acc[a]);
    }
#pragma unroll
    for (int a = 0; a < PA_MAX; ++a) {
        float v = acc[a];
#pragma unroll
        for (int off = TPR / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
        if (part == 0 && a < A) out[r * out_ld + a] = v + b2[a];
    }
}

template <int H, int ACT, bool GAUSS>
__global__ __launch_bounds__(2 * H) void policy_kernel(
    const float *__restrict__ obs, int n, int IN, int A, const float *__restrict__ actor_p,
    const float *__restrict__ critic_p, uint32_t seed, float *__restrict__ actions,
    float *__restrict__ r_obs, float *__restrict__ r_actions, float *__restrict__ r_logp,
    float *__restrict__ r_values) {
    __shared__ float xs[PR * XS_LD];
    __shared__ float hT[2][H * HT_LD];
    __shared__ float h2[2][PR * (H + 1)];
    __shared__ float logits[PR * (PA_MAX + 1)];
    __shared__ float vals[PR];
    const int t = threadIdx.x;
    const int net = t / H;                   // 0 = actor, 1 = critic
    const int row0 = blockIdx.x * PR;
    const int nrow = min(PR, n - row0);

    // observation tile in (rows beyond the batch read as zero), and straight out to rollout[t]
    for (int i = t; i < PR * IN; i += 2 * H) {
        const int r = i / IN, k = i - r * IN;
        float v = 0.0f;
        if (r < nrow) {
            v = obs[(long)row0 * IN + i];
            r_obs[(long)row0 * IN + i] = v;
        }
        xs[r * XS_LD + k] = v;
    }
    __syncthreads();

    const float *p = net ? critic_p : actor_p;
    hidden_stack<H, ACT>(p, IN, xs, hT[net], h2[net]);
    if (net == 0) head<H>(p + IN * H + H + H * H + H, A, h2[0], logits, PA_MAX + 1);
    else head<H>(p + IN * H + H + H * H + H, 1, h2[1], vals, 1);
    __syncthreads();

    if (t < nrow && !GAUSS) {   // categorical sampling, one lane per env
        const int i = row0 + t;
        const float *l = logits + t * (PA_MAX + 1);
        uint32_t rng = seed ^ ((uint32_t)i * 2654435761u);
        rng = xorshift32(rng);
        float max_logit = l[0];
        for (int a = 1; a < A; ++a) if (l[a] > max_logit) max_logit = l[a];
        float sum_exp = 0.0f;
        for (int a = 0; a < A; ++a) sum_exp = sum_exp + expf(l[a] - max_logit);
        const float u = random_uniform(rng);
        float cumsum = 0.0f;
        int sel = 0;
        for (int a = 0; a < A; ++a) {
            float prob = expf(l[a] - max_logit) / sum_exp;
            cumsum = cumsum + prob;
            if (u < cumsum) { sel = a; break; }
        }
        const float pr = expf(l[sel] - max_logit) / sum_exp;
        actions[i] = (float)sel;
        r_actions[i] = (float)sel;
        r_logp[i] = logf(pr + 1e-8f);
        r_values[i] = vals[t];
    }
    if (t < nrow && GAUSS) {    // Gaussian sampling, one lane per env, one Philox stream per (env, j)
        const int i = row0 + t;
        const float *mean_row = logits + t * (PA_MAX + 1);
        const float *log_std_p = actor_p + IN * H + H + H * H + H + H * A + A;
        const float EPS = 1e-6f, LOG_2PI = (float)1.8378770664093453;
        float total = 0.0f;
        for (int j = 0; j < A; ++j) {
            const float mean = mean_row[j];
            float log_std = log_std_p[j];
            if (log_std < -5.0f) log_std = -5.0f;
            else if (log_std > 2.0f) log_std = 2.0f;
            Uniform4 rv = philox_uniform4((uint64_t)((int64_t)seed + (int64_t)i * A + j), 0, 0);
            const float u1 = rv.v[0] + 1e-8f;
            const float mag = sqrtf(-2.0f * logf(u1));
            const float noise = mag * cosf(rv.v[1] * (float)6.283185307179586);
            const float std = expf(log_std);
            const float action = mean + std * noise;
            actions[(long)i * A + j] = action;
            r_actions[(long)i * A + j] = action;
            const float an = (action - mean) / (std + EPS);
            total = total + -0.5f * (LOG_2PI + 2.0f * log_std + an * an);
        }
        r_logp[i] = total;
        r_values[i] = vals[t];
    }
}

// true when the pair (actor, critic) has the shape this kernel is specialised for
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
    dim3 grid((n + PR - 1) / PR);
#define MRL_LAUNCH(HH, AA, GG)                                                                         \
    hipLaunchKernelGGL((policy_kernel<HH, AA, GG>), grid, dim3(2 * HH), 0, ctx->stream, obs, n, IN, A, ap, \
                       cp, seed, actions, r_obs, r_actions, r_logp, r_values)
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
