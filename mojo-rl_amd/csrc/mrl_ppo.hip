// PPO elementwise and reduction kernels: samplers, GAE, advantage normalisation, minibatch
// gather, loss gradients, global-norm clipping, Adam.  All are HBM-bound: one pass over the
// data, coalesced, reductions by wavefront shuffles and one small second stage.
#include "mrl_host.hpp"
#include "mrl_device.hpp"
#include "ppo_grads.hpp"
#include "policy_sample.hpp"

namespace mrl {

constexpr int TPB = 256;

MRL_DEV float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// block sum, result valid in every lane of wavefront 0 (and in thread 0)
MRL_DEV float block_sum(float v, float *smem) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (lane == 0) smem[w] = v;
    __syncthreads();
    float r = 0.0f;
    if (w == 0) {
        r = (lane < (int)(blockDim.x >> 6)) ? smem[lane] : 0.0f;
        r = wave_sum(r);
    }
    __syncthreads();
    return r;
}

// ---------------------------------------------------------------- samplers

// deep_agents/ppo/ppo.mojo:4064-4123
__global__ __launch_bounds__(TPB) void sample_categorical_kernel(const float *__restrict__ logits,
                                                                 int n, int A, uint32_t seed,
                                                                 float *__restrict__ actions,
                                                                 float *__restrict__ log_probs) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int sel;
    float logp;
    if (A <= SAMPLE_A_MAX) sample_categorical_few(logits + (long)i * A, A, seed, i, sel, logp);
    else sample_categorical(logits + (long)i * A, A, seed, i, sel, logp);
    actions[i] = (float)sel;
    log_probs[i] = logp;
}

// deep_agents/ppo/kernels.mojo:12-98
__global__ __launch_bounds__(TPB) void sample_gaussian_kernel(const float *__restrict__ actor_out,
                                                              int n, int A, uint32_t seed,
                                                              float *__restrict__ actions,
                                                              float *__restrict__ log_probs) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float *o = actor_out + (long)i * 2 * A;
    log_probs[i] = sample_gaussian(o, o + A, A, seed, i, actions + (long)i * A);
}

// add_obs_noise_kernel, deep_agents/ppo/kernels.mojo:882-925: Gaussian noise on every observation
// entry, one Philox stream per (env, entry), Box-Muller as in the Gaussian sampler
__global__ __launch_bounds__(TPB) void obs_noise_kernel(float *__restrict__ obs, int n, int obs_dim,
                                                        float noise_std, uint32_t seed) {
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;   // one thread per (env, entry)
    if (e >= (long)n * obs_dim) return;
    Uniform4 rv = philox_uniform4((uint64_t)((int64_t)seed + e), 0, 0);
    const float u1 = rv.v[0] + 1e-8f;
    const float mag = sqrtf(-2.0f * log32(u1));
    const float noise = mag * cos32(rv.v[1] * (float)6.283185307179586);
    obs[e] = obs[e] + noise * noise_std;
}

// ---------------------------------------------------------------- GAE
// One lane per env scans t = T-1 .. 0; index t*N + env makes every step of the scan a
// coalesced row access.  The scan itself is serial, its loads are not: the rows of the next
// GAE_U steps are requested while the current ones are scanned, so a wavefront waits for memory
// once per GAE_U steps instead of once per step.  deep_agents/ppo/ppo.mojo:2317-2353
constexpr int GAE_U = 16;

struct GaeScan {
    float gae, next_val, gamma, decay;
    MRL_DEV void step(float r, float v, float d, float *adv, float *ret) {
        float nv = next_val;
        if (d > 0.5f) { nv = 0.0f; gae = 0.0f; }
        const float delta = r + gamma * nv - v;
        gae = delta + decay * gae;
        *adv = gae;
        *ret = gae + v;
        next_val = v;
    }
};

__global__ __launch_bounds__(64) void gae_kernel(int T, int N, const float *__restrict__ rewards,
                                                 const float *__restrict__ values,
                                                 const float *__restrict__ dones,
                                                 const float *__restrict__ bootstrap, float gamma,
                                                 float decay, float *__restrict__ adv,
                                                 float *__restrict__ ret) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= N) return;
    GaeScan s{0.0f, bootstrap[e], gamma, decay};
    int t = T - 1;
    for (; (t + 1) % GAE_U != 0; --t) {   // the steps above the last whole group
        const long idx = (long)t * N + e;
        s.step(rewards[idx], values[idx], dones[idx], adv + idx, ret + idx);
    }
    // t + 1 is a multiple of GAE_U: groups t, t - 1, .. t - GAE_U + 1
    float r[GAE_U], v[GAE_U], d[GAE_U], nr[GAE_U], nv[GAE_U], nd[GAE_U];
    if (t >= 0) {
#pragma unroll
        for (int j = 0; j < GAE_U; ++j) {
            const long idx = (long)(t - j) * N + e;
            r[j] = rewards[idx]; v[j] = values[idx]; d[j] = dones[idx];
        }
    }
    for (; t >= 0; t -= GAE_U) {
        const bool more = t - GAE_U >= 0;
        if (more) {
#pragma unroll
            for (int j = 0; j < GAE_U; ++j) {
                const long idx = (long)(t - GAE_U - j) * N + e;
                nr[j] = rewards[idx]; nv[j] = values[idx]; nd[j] = dones[idx];
            }
        }
#pragma unroll
        for (int j = 0; j < GAE_U; ++j) {
            const long idx = (long)(t - j) * N + e;
            s.step(r[j], v[j], d[j], adv + idx, ret + idx);
        }
        if (more) {
#pragma unroll
            for (int j = 0; j < GAE_U; ++j) { r[j] = nr[j]; v[j] = nv[j]; d[j] = nd[j]; }
        }
    }
}

// ---------------------------------------------------------------- advantage normalisation
// pass 1: per-block sums -> scratch[0..nb); pass 2: mean; pass 3: per-block sum of squared
// deviations; pass 4: (x - mean) / (sqrt(var + 1e-8) + 1e-8).  Two-pass variance like the
// reference (ppo.mojo:2356-2371), with fp32 sums taken blockwise.
__global__ __launch_bounds__(TPB) void partial_sum_kernel(const float *__restrict__ x, int n,
                                                          const float *__restrict__ mean_ptr,
                                                          float *__restrict__ out) {
    __shared__ float smem[4];
    const float mean = mean_ptr ? *mean_ptr : 0.0f;
    float s = 0.0f;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        float d = x[i] - mean;
        s += mean_ptr ? d * d : x[i];
    }
    s = block_sum(s, smem);
    if (threadIdx.x == 0) out[blockIdx.x] = s;
}

// out[0] = sum(in[0..nb)) / n
__global__ __launch_bounds__(TPB) void finish_mean_kernel(const float *__restrict__ in, int nb, int n,
                                                          float *__restrict__ out) {
    __shared__ float smem[4];
    float s = 0.0f;
    for (int i = threadIdx.x; i < nb; i += blockDim.x) s += in[i];
    s = block_sum(s, smem);
    if (threadIdx.x == 0) out[0] = s / (float)n;
}

__global__ __launch_bounds__(TPB) void normalize_apply_kernel(float *__restrict__ x, int n,
                                                              const float *__restrict__ stats) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float mean = stats[0], variance = stats[1];
    const float std = sqrtf(variance + 1e-8f);
    x[i] = (x[i] - mean) / (std + 1e-8f);
}

// ---------------------------------------------------------------- reward RunningMeanStd
// core/utils/normalization.mojo:188-292 in Float64: batch mean and variance (two passes), merged
// into (count, mean, var_sum) with Chan's formula; normalise with var = 1 while count < 2.
MRL_DEV double wave_sum_d(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

MRL_DEV double block_sum_d(double v, double *smem) {
    v = wave_sum_d(v);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) smem[w] = v;
    __syncthreads();
    double t = 0.0;
    for (int k = 0; k < (int)(blockDim.x >> 6); ++k) t += smem[k];
    __syncthreads();
    return t;
}

// mean_ptr == nullptr: out[b] = sum x; else out[b] = sum (x - *mean_ptr)^2
__global__ __launch_bounds__(TPB) void rms_partial_kernel(const float *__restrict__ x, int n,
                                                          const double *__restrict__ mean_ptr,
                                                          double *__restrict__ out) {
    __shared__ double smem[4];
    const double mean = mean_ptr ? *mean_ptr : 0.0;
    double s = 0.0;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        double d = (double)x[i] - mean;
        s += mean_ptr ? d * d : (double)x[i];
    }
    s = block_sum_d(s, smem);
    if (threadIdx.x == 0) out[blockIdx.x] = s;
}

__global__ __launch_bounds__(TPB) void rms_batch_mean_kernel(const double *__restrict__ in, int nb, int n,
                                                             double *__restrict__ out) {
    __shared__ double smem[4];
    double s = 0.0;
    for (int i = threadIdx.x; i < nb; i += blockDim.x) s += in[i];
    s = block_sum_d(s, smem);
    if (threadIdx.x == 0) out[0] = s / (double)n;
}

// state = (count, mean, var_sum)
__global__ __launch_bounds__(TPB) void rms_merge_kernel(const double *__restrict__ in, int nb, int n,
                                                        const double *__restrict__ batch_mean,
                                                        double *__restrict__ state) {
    __shared__ double smem[4];
    double s = 0.0;
    for (int i = threadIdx.x; i < nb; i += blockDim.x) s += in[i];
    s = block_sum_d(s, smem);
    if (threadIdx.x != 0) return;
    const double bm = *batch_mean, bv = s / (double)n;
    const double count = state[0], mean = state[1], var_sum = state[2];
    const double new_count = count + (double)n;
    if (count == 0.0) {
        state[1] = bm;
        state[2] = bv * (double)n;
    } else {
        const double delta = bm - mean;
        state[1] = mean + delta * (double)n / new_count;
        state[2] = var_sum + bv * (double)n + delta * delta * count * (double)n / new_count;
    }
    state[0] = new_count;
}

__global__ __launch_bounds__(TPB) void rms_normalize_kernel(const double *__restrict__ state,
                                                            float *__restrict__ x, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const double count = state[0], mean = state[1];
    const double var = (count < 2.0) ? 1.0 : state[2] / count;
    const double std = sqrt(var + 1e-8);
    x[i] = (float)(((double)x[i] - mean) / (std + 1e-8));
}

// ---------------------------------------------------------------- permutation
// A keyed bijection of [0, 2^k) (balanced Feistel network on k = 2h bits, round keys from
// Philox) with cycle walking down to [0, n): idx[i] = P(i).  One pass, no sort, no scratch.
// It stands where the reference shuffles on the host (Fisher-Yates driven by the global
// random_float64 stream, deep_agents/ppo/ppo.mojo:2425-2434, core/utils/shuffle.mojo:21-82).
constexpr int PERM_ROUNDS = 8;
struct PermKeys { uint32_t k[PERM_ROUNDS]; };

MRL_DEV uint32_t perm_mix(uint32_t x) {
    x ^= x >> 16; x *= 0x85ebca6bu; x ^= x >> 13; x *= 0xc2b2ae35u; x ^= x >> 16;
    return x;
}

__global__ __launch_bounds__(TPB) void permutation_kernel(int32_t *__restrict__ idx, int n, int half_bits,
                                                          PermKeys keys) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const uint32_t mask = (1u << half_bits) - 1u;
    uint32_t x = (uint32_t)i;
    do {
        uint32_t l = x >> half_bits, r = x & mask;
#pragma unroll
        for (int k = 0; k < PERM_ROUNDS; ++k) {
            const uint32_t f = perm_mix(r ^ keys.k[k]) & mask;
            const uint32_t nl = r;
            r = l ^ f;
            l = nl;
        }
        x = (l << half_bits) | r;
    } while (x >= (uint32_t)n);
    idx[i] = (int32_t)x;
}

// host Philox4x32-10 block (round keys of the permutation)
static void philox4x32_10_host(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// ---------------------------------------------------------------- parameter initialisation
// p[i] = lo + u_i * (hi - lo), u_i = lane (i % 4) of Philox(seed, offset = i / 4): the uniform
// fills of deep_rl/initializer/initializers.mojo:69-104 (Xavier / Kaiming bounds are formed by
// the caller) and StochasticActor.init_params_small (stochastic_actor.mojo:95-128).
__global__ __launch_bounds__(TPB) void init_uniform_kernel(float *__restrict__ p, int n, float lo, float hi,
                                                           uint64_t seed) {
    int q = blockIdx.x * blockDim.x + threadIdx.x;
    if (q * 4 >= n) return;
    Uniform4 u = philox_uniform4(seed, (uint64_t)q, 0);
#pragma unroll
    for (int k = 0; k < 4; ++k)
        if (q * 4 + k < n) p[q * 4 + k] = lo + u.v[k] * (hi - lo);
}

// ---------------------------------------------------------------- KL early stop
// mean of the minibatch's per-sample KL estimates compared with target_kl on the device
// (ppo.mojo:2557-2573, ppo_continuous.mojo:3062-3086 do this on the host after a copy):
// flag[0] = 1 once mean KL > target (sticky), flag[1] = bit pattern of the last mean.
__global__ __launch_bounds__(TPB) void kl_check_kernel(const float *__restrict__ kl, int mb, float target,
                                                       int32_t *__restrict__ flag) {
    __shared__ float smem[4];
    float s = 0.0f;
    for (int i = threadIdx.x; i < mb; i += blockDim.x) s = s + kl[i];
    s = block_sum(s, smem);
    if (threadIdx.x == 0) {
        const float mean = s / (float)mb;
        flag[1] = __float_as_int(mean);
        if (mean > target) flag[0] = 1;
    }
}

// ---------------------------------------------------------------- gather
__global__ __launch_bounds__(TPB) void gather_kernel(const int32_t *__restrict__ idx, int mb, int obs_dim,
                                                     int act_dim, const float *r_obs, const float *r_act,
                                                     const float *r_adv, const float *r_ret,
                                                     const float *r_logp, const float *r_val,
                                                     float *mb_obs, float *mb_act, float *mb_adv,
                                                     float *mb_ret, float *mb_logp, float *mb_val) {
    // one lane per output float of the widest array (obs): consecutive lanes copy consecutive words
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const int w = obs_dim;
    if (i >= (long)mb * w) return;
    int b = (int)(i / w), c = (int)(i - (long)b * w);
    long src = idx[b];
    mb_obs[i] = r_obs[src * obs_dim + c];
    if (c < act_dim) mb_act[(long)b * act_dim + c] = r_act[src * act_dim + c];
    if (c == 0) {
        mb_adv[b] = r_adv[src];
        mb_ret[b] = r_ret[src];
        mb_logp[b] = r_logp[src];
        mb_val[b] = r_val[src];
    }
}

// ---------------------------------------------------------------- loss gradients
// (per-sample formulas in ppo_grads.hpp)
__global__ __launch_bounds__(TPB) void actor_grad_discrete_kernel(
    const float *__restrict__ logits, const float *__restrict__ old_logp,
    const float *__restrict__ adv, const float *__restrict__ actions, int mb, int A, float clip_eps,
    float ent_coef, float *__restrict__ grad_logits, float *__restrict__ kl) {
    int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= mb) return;
    kl[b] = actor_grad_discrete_one(b, logits, old_logp, adv, actions, mb, A, clip_eps, ent_coef, grad_logits);
}

__global__ __launch_bounds__(TPB) void actor_grad_gaussian_kernel(
    const float *__restrict__ actor_out, const float *__restrict__ old_logp,
    const float *__restrict__ adv, const float *__restrict__ actions, int mb, int A, float clip_eps,
    float ent_coef, float *__restrict__ grad_out, float *__restrict__ kl_out) {
    int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= mb) return;
    kl_out[b] = actor_grad_gaussian_one(b, actor_out, old_logp, adv, actions, mb, A, clip_eps, ent_coef, grad_out);
}

__global__ __launch_bounds__(TPB) void critic_grad_kernel(const float *__restrict__ values,
                                                          const float *__restrict__ old_values,
                                                          const float *__restrict__ returns, int mb,
                                                          int convention, int clipped,
                                                          float value_coef, float clip_eps,
                                                          float *__restrict__ grad) {
    int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= mb) return;
    grad[b] = critic_grad_one(b, values, old_values, returns, mb, convention, clipped, value_coef, clip_eps);
}

// ---------------------------------------------------------------- clip by global norm
__global__ __launch_bounds__(TPB) void sq_partial_kernel(const float *__restrict__ g, int n,
                                                         float *__restrict__ out) {
    __shared__ float smem[4];
    float s = 0.0f;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        s += g[i] * g[i];
    s = block_sum(s, smem);
    if (threadIdx.x == 0) out[blockIdx.x] = s;
}

// every block re-reduces the (few) partial sums, then scales its slice: no single-block stage
__global__ __launch_bounds__(TPB) void clip_apply_kernel(float *__restrict__ g, int n,
                                                         const float *__restrict__ partial, int nb,
                                                         float max_norm) {
    __shared__ float smem[4];
    __shared__ float scale_s;
    float s = 0.0f;
    for (int i = threadIdx.x; i < nb; i += blockDim.x) s += partial[i];
    s = block_sum(s, smem);
    if (threadIdx.x == 0) {
        float norm = sqrtf(s);
        float scale = 1.0f;
        if (norm > max_norm) scale = max_norm / (norm + 1e-8f);
        scale_s = scale;
    }
    __syncthreads();
    const float scale = scale_s;
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) g[i] = g[i] * scale;
}

// ---------------------------------------------------------------- Adam
// deep_rl/optimizer/adam.mojo:52-105; state interleaved (m, v) per parameter -> one 8-byte access
__global__ __launch_bounds__(TPB) void adam_kernel(float *__restrict__ p, const float *__restrict__ g,
                                                   float2 *__restrict__ state, int n, float lr,
                                                   float beta1, float beta2, float omb1, float omb2,
                                                   float eps, float bc1, float bc2) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float gi = g[i];
    float2 mv = state[i];
    float m_new = beta1 * mv.x + omb1 * gi;
    float v_new = beta2 * mv.y + omb2 * gi * gi;
    state[i] = make_float2(m_new, v_new);
    float m_hat = m_new / bc1, v_hat = v_new / bc2;
    p[i] = p[i] - lr * m_hat / (sqrtf(v_hat) + eps);
}

__global__ void clamp_log_std_kernel(float *params, int offset, int A) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= A) return;
    float v = params[offset + i];
    if (v < -5.0f) params[offset + i] = -5.0f;
    else if (v > 2.0f) params[offset + i] = 2.0f;
}

}  // namespace mrl

using namespace mrl;

// ---------------------------------------------------------------- allocation-free clip
// Scratch of mrl_clip_grad_norm_static: the per-block partial sums of squares live in this
// file-scope array instead of memory obtained from hipMalloc (each device the library runs on holds
// its own 1 KiB copy until the process ends).  In host code the array's name is only a handle for the
// symbol: the device address is looked up once per device and kept in g_clip_scratch_ptr.
constexpr int CLIP_STATIC_PARTIALS = 256;
constexpr int CLIP_STATIC_MAX_DEVICES = 64;
static __device__ __align__(256) float g_clip_scratch[CLIP_STATIC_PARTIALS];
static float *g_clip_scratch_ptr[CLIP_STATIC_MAX_DEVICES] = {};

namespace mrl {
// Looks the address of this device's copy of the scratch array up; `device` must be the current
// device.  Called by mrl_ctx_create, and again (a no-op then) by the entry point itself.
int clip_static_setup(int device) {
    if (device < 0 || device >= CLIP_STATIC_MAX_DEVICES)
        return set_error(MRL_E_ARG, "clip_static_setup: device %d outside 0..%d", device, CLIP_STATIC_MAX_DEVICES - 1);
    if (g_clip_scratch_ptr[device] != nullptr) return MRL_OK;
    float *p = nullptr;
    hipError_t e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(g_clip_scratch));
    if (e != hipSuccess || p == nullptr)
        return set_error(MRL_E_HIP, "hipGetSymbolAddress(g_clip_scratch) failed: %s", hipGetErrorString(e));
    g_clip_scratch_ptr[device] = p;
    return MRL_OK;
}
}  // namespace mrl

extern "C" {

int mrl_sample_categorical(mrl_ctx *ctx, const float *logits, int n, int num_actions, uint32_t seed,
                           float *actions, float *log_probs) {
    MRL_CHECK_ARG(ctx, "mrl_sample_categorical: ctx is NULL");
    MRL_CHECK_ARG(n >= 0 && num_actions > 0, "mrl_sample_categorical: bad sizes");
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(logits && actions && log_probs, "mrl_sample_categorical: NULL buffer");
    hipLaunchKernelGGL(sample_categorical_kernel, dim3(grid_for(n, TPB)), dim3(TPB), 0, ctx->stream,
                       logits, n, num_actions, seed, actions, log_probs);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_sample_gaussian(mrl_ctx *ctx, const float *actor_out, int n, int action_dim, uint32_t seed,
                        float *actions, float *log_probs) {
    MRL_CHECK_ARG(ctx, "mrl_sample_gaussian: ctx is NULL");
    MRL_CHECK_ARG(n >= 0 && action_dim > 0, "mrl_sample_gaussian: bad sizes");
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(actor_out && actions && log_probs, "mrl_sample_gaussian: NULL buffer");
    hipLaunchKernelGGL(sample_gaussian_kernel, dim3(grid_for(n, TPB)), dim3(TPB), 0, ctx->stream,
                       actor_out, n, action_dim, seed, actions, log_probs);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

__global__ __launch_bounds__(256) void greedy_actions_kernel(const float *__restrict__ actor_out, int n, int A,
                                                             int continuous, float *__restrict__ actions) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (continuous) {
        if (i >= n * A) return;
        const int row = i / A, j = i - row * A;
        actions[i] = actor_out[(size_t)row * 2 * A + j];
    } else {
        if (i >= n) return;
        const float *l = actor_out + (size_t)i * A;
        int best = 0;
        float top = l[0];
        for (int a = 1; a < A; ++a)
            if (l[a] > top) { top = l[a]; best = a; }
        actions[i] = (float)best;
    }
}

int mrl_greedy_actions(mrl_ctx *ctx, const float *actor_out, int n, int num_actions, int continuous,
                       float *actions) {
    MRL_CHECK_ARG(ctx, "mrl_greedy_actions: ctx is NULL");
    MRL_CHECK_ARG(n >= 0 && num_actions > 0, "mrl_greedy_actions: bad sizes");
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(actor_out && actions, "mrl_greedy_actions: NULL buffer");
    const long work = continuous ? (long)n * num_actions : (long)n;
    hipLaunchKernelGGL(greedy_actions_kernel, dim3(grid_for(work, 256)), dim3(256), 0, ctx->stream, actor_out, n,
                       num_actions, continuous, actions);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_gae(mrl_ctx *ctx, int T, int N, const float *rewards, const float *values,
            const float *dones, const float *bootstrap, double gamma, double lam, float *adv,
            float *ret) {
    MRL_CHECK_ARG(ctx, "mrl_gae: ctx is NULL");
    MRL_CHECK_ARG(T >= 0 && N >= 0, "mrl_gae: negative size");
    if (T == 0 || N == 0) return MRL_OK;
    MRL_CHECK_ARG(rewards && values && dones && bootstrap && adv && ret, "mrl_gae: NULL buffer");
    hipLaunchKernelGGL(gae_kernel, dim3(grid_for(N, 64)), dim3(64), 0, ctx->stream, T, N, rewards,
                       values, dones, bootstrap, (float)gamma, (float)(gamma * lam), adv, ret);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_normalize_advantages(mrl_ctx *ctx, float *x, int n) {
    MRL_CHECK_ARG(ctx, "mrl_normalize_advantages: ctx is NULL");
    MRL_CHECK_ARG(n >= 0, "mrl_normalize_advantages: negative size");
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(x, "mrl_normalize_advantages: NULL buffer");
    int nb = std::min(1024, grid_for(n, TPB));
    float *part = ctx->reduce_scratch;         // [0, nb)
    float *stats = ctx->reduce_scratch + 2048;  // mean, variance
    hipLaunchKernelGGL(partial_sum_kernel, dim3(nb), dim3(TPB), 0, ctx->stream, x, n, (const float *)nullptr, part);
    hipLaunchKernelGGL(finish_mean_kernel, dim3(1), dim3(TPB), 0, ctx->stream, part, nb, n, stats);
    hipLaunchKernelGGL(partial_sum_kernel, dim3(nb), dim3(TPB), 0, ctx->stream, x, n, (const float *)stats, part);
    hipLaunchKernelGGL(finish_mean_kernel, dim3(1), dim3(TPB), 0, ctx->stream, part, nb, n, stats + 1);
    hipLaunchKernelGGL(normalize_apply_kernel, dim3(grid_for(n, TPB)), dim3(TPB), 0, ctx->stream, x, n, stats);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_rms_update(mrl_ctx *ctx, double *state, const float *x, int n) {
    MRL_CHECK_ARG(ctx, "mrl_rms_update: ctx is NULL");
    MRL_CHECK_ARG(n >= 0, "mrl_rms_update: negative size");
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(state && x, "mrl_rms_update: NULL buffer");
    const int nb = std::min(1024, grid_for(n, TPB));
    double *part = reinterpret_cast<double *>(ctx->reduce_scratch);   // [0, nb) doubles
    double *bm = part + 1024;
    hipLaunchKernelGGL(rms_partial_kernel, dim3(nb), dim3(TPB), 0, ctx->stream, x, n, (const double *)nullptr, part);
    hipLaunchKernelGGL(rms_batch_mean_kernel, dim3(1), dim3(TPB), 0, ctx->stream, part, nb, n, bm);
    hipLaunchKernelGGL(rms_partial_kernel, dim3(nb), dim3(TPB), 0, ctx->stream, x, n, (const double *)bm, part);
    hipLaunchKernelGGL(rms_merge_kernel, dim3(1), dim3(TPB), 0, ctx->stream, part, nb, n, bm, state);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_rms_normalize(mrl_ctx *ctx, const double *state, float *x, int n) {
    MRL_CHECK_ARG(ctx, "mrl_rms_normalize: ctx is NULL");
    MRL_CHECK_ARG(n >= 0, "mrl_rms_normalize: negative size");
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(state && x, "mrl_rms_normalize: NULL buffer");
    hipLaunchKernelGGL(rms_normalize_kernel, dim3(grid_for(n, TPB)), dim3(TPB), 0, ctx->stream, state, x, n);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_permutation(mrl_ctx *ctx, int32_t *indices, int n, uint64_t seed) {
    MRL_CHECK_ARG(ctx, "mrl_permutation: ctx is NULL");
    MRL_CHECK_ARG(n >= 0 && n <= (1 << 30), "mrl_permutation: n = %d out of range", n);
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(indices, "mrl_permutation: NULL buffer");
    int half_bits = 1;
    while ((1ll << (2 * half_bits)) < (long long)n) ++half_bits;
    PermKeys keys;
    for (int k = 0; k < PERM_ROUNDS; k += 4) {
        uint32_t ctr[4] = {(uint32_t)(k / 4), 0x7065726du, 0u, 0u};
        uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
        uint32_t out[4];
        philox4x32_10_host(ctr, key, out);
        for (int j = 0; j < 4 && k + j < PERM_ROUNDS; ++j) keys.k[k + j] = out[j];
    }
    hipLaunchKernelGGL(permutation_kernel, dim3(grid_for(n, TPB)), dim3(TPB), 0, ctx->stream, indices, n,
                       half_bits, keys);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_kl_check(mrl_ctx *ctx, const float *kl, int mb, float target_kl, int32_t *flag) {
    MRL_CHECK_ARG(ctx, "mrl_kl_check: ctx is NULL");
    MRL_CHECK_ARG(mb > 0, "mrl_kl_check: minibatch must be positive");
    MRL_CHECK_ARG(kl && flag, "mrl_kl_check: NULL buffer");
    hipLaunchKernelGGL(kl_check_kernel, dim3(1), dim3(TPB), 0, ctx->stream, kl, mb, target_kl, flag);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_init_uniform(mrl_ctx *ctx, float *params, int n, float lo, float hi, uint64_t seed) {
    MRL_CHECK_ARG(ctx, "mrl_init_uniform: ctx is NULL");
    MRL_CHECK_ARG(n >= 0, "mrl_init_uniform: negative size");
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(params, "mrl_init_uniform: NULL buffer");
    hipLaunchKernelGGL(init_uniform_kernel, dim3(grid_for((n + 3) / 4, TPB)), dim3(TPB), 0, ctx->stream,
                       params, n, lo, hi, seed);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_gather_minibatch(mrl_ctx *ctx, const int32_t *indices, int mb, int obs_dim, int act_dim,
                         const float *r_obs, const float *r_actions, const float *r_adv,
                         const float *r_ret, const float *r_logp, const float *r_values,
                         float *mb_obs, float *mb_actions, float *mb_adv, float *mb_ret,
                         float *mb_logp, float *mb_values) {
    MRL_CHECK_ARG(ctx, "mrl_gather_minibatch: ctx is NULL");
    MRL_CHECK_ARG(mb >= 0 && obs_dim > 0 && act_dim > 0 && act_dim <= obs_dim,
                  "mrl_gather_minibatch: bad sizes (need 0 < act_dim <= obs_dim)");
    if (mb == 0) return MRL_OK;
    MRL_CHECK_ARG(indices && r_obs && r_actions && r_adv && r_ret && r_logp && r_values && mb_obs &&
                      mb_actions && mb_adv && mb_ret && mb_logp && mb_values,
                  "mrl_gather_minibatch: NULL buffer");
    hipLaunchKernelGGL(gather_kernel, dim3(grid_for((long)mb * obs_dim, TPB)), dim3(TPB), 0, ctx->stream,
                       indices, mb, obs_dim, act_dim, r_obs, r_actions, r_adv, r_ret, r_logp, r_values,
                       mb_obs, mb_actions, mb_adv, mb_ret, mb_logp, mb_values);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_ppo_actor_grad_discrete(mrl_ctx *ctx, const float *logits, const float *old_log_probs,
                                const float *advantages, const float *actions, int mb,
                                int num_actions, float clip_eps, float entropy_coef,
                                float *grad_logits, float *kl) {
    MRL_CHECK_ARG(ctx, "mrl_ppo_actor_grad_discrete: ctx is NULL");
    MRL_CHECK_ARG(mb >= 0 && num_actions > 0, "mrl_ppo_actor_grad_discrete: bad sizes");
    if (mb == 0) return MRL_OK;
    MRL_CHECK_ARG(logits && old_log_probs && advantages && actions && grad_logits && kl,
                  "mrl_ppo_actor_grad_discrete: NULL buffer");
    hipLaunchKernelGGL(actor_grad_discrete_kernel, dim3(grid_for(mb, TPB)), dim3(TPB), 0, ctx->stream,
                       logits, old_log_probs, advantages, actions, mb, num_actions, clip_eps,
                       entropy_coef, grad_logits, kl);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_ppo_actor_grad_gaussian(mrl_ctx *ctx, const float *actor_out, const float *old_log_probs,
                                const float *advantages, const float *actions, int mb,
                                int action_dim, float clip_eps, float entropy_coef, float *grad_out,
                                float *kl) {
    MRL_CHECK_ARG(ctx, "mrl_ppo_actor_grad_gaussian: ctx is NULL");
    MRL_CHECK_ARG(mb >= 0 && action_dim > 0, "mrl_ppo_actor_grad_gaussian: bad sizes");
    if (mb == 0) return MRL_OK;
    MRL_CHECK_ARG(actor_out && old_log_probs && advantages && actions && grad_out && kl,
                  "mrl_ppo_actor_grad_gaussian: NULL buffer");
    hipLaunchKernelGGL(actor_grad_gaussian_kernel, dim3(grid_for(mb, TPB)), dim3(TPB), 0, ctx->stream,
                       actor_out, old_log_probs, advantages, actions, mb, action_dim, clip_eps,
                       entropy_coef, grad_out, kl);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_ppo_critic_grad(mrl_ctx *ctx, const float *values, const float *old_values,
                        const float *returns, int mb, int convention, int clipped, float value_coef,
                        float clip_eps, float *grad_values) {
    MRL_CHECK_ARG(ctx, "mrl_ppo_critic_grad: ctx is NULL");
    MRL_CHECK_ARG(mb >= 0 && (convention == 0 || convention == 1), "mrl_ppo_critic_grad: bad arguments");
    if (mb == 0) return MRL_OK;
    MRL_CHECK_ARG(values && returns && grad_values && (!clipped || old_values),
                  "mrl_ppo_critic_grad: NULL buffer");
    hipLaunchKernelGGL(critic_grad_kernel, dim3(grid_for(mb, TPB)), dim3(TPB), 0, ctx->stream, values,
                       old_values, returns, mb, convention, clipped, value_coef, clip_eps, grad_values);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_add_obs_noise(mrl_ctx *ctx, float *obs, int n, int obs_dim, float noise_std, uint32_t seed) {
    MRL_CHECK_ARG(ctx, "mrl_add_obs_noise: ctx is NULL");
    MRL_CHECK_ARG(n >= 0 && obs_dim > 0, "mrl_add_obs_noise: bad sizes");
    if (n == 0 || !(noise_std > 0.0f)) return MRL_OK;   // the reference's kernel returns at once for std <= 0
    MRL_CHECK_ARG(obs, "mrl_add_obs_noise: NULL buffer");
    hipLaunchKernelGGL(obs_noise_kernel, dim3(grid_for((long)n * obs_dim, TPB)), dim3(TPB), 0, ctx->stream, obs, n,
                       obs_dim, noise_std, seed);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_clip_grad_norm(mrl_ctx *ctx, float *grads, int n, float max_norm) {
    MRL_CHECK_ARG(ctx, "mrl_clip_grad_norm: ctx is NULL");
    MRL_CHECK_ARG(n >= 0, "mrl_clip_grad_norm: negative size");
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(grads, "mrl_clip_grad_norm: NULL buffer");
    int nb = std::min(256, grid_for(n, TPB));
    float *part = ctx->reduce_scratch + 1024;
    hipLaunchKernelGGL(sq_partial_kernel, dim3(nb), dim3(TPB), 0, ctx->stream, grads, n, part);
    hipLaunchKernelGGL(clip_apply_kernel, dim3(grid_for(n, TPB)), dim3(TPB), 0, ctx->stream, grads, n,
                       part, nb, max_norm);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_clip_grad_norm_static(mrl_ctx *ctx, float *grads, int n, float max_norm) {
    MRL_CHECK_ARG(ctx, "mrl_clip_grad_norm_static: ctx is NULL");
    MRL_CHECK_ARG(n >= 0, "mrl_clip_grad_norm_static: negative size");
    MRL_CHECK_ARG(n <= MRL_CLIP_STATIC_MAX_N,
                  "mrl_clip_grad_norm_static: n = %d exceeds the limit of %d elements of the allocation-free "
                  "variant (use mrl_clip_grad_norm)", n, MRL_CLIP_STATIC_MAX_N);
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(grads, "mrl_clip_grad_norm_static: NULL buffer");
    // the array of the CONTEXT's device (its stream runs there), whatever device is current on this thread;
    // mrl_ctx_create looked the address up with that device current
    const int dev = ctx->device;
    MRL_CHECK_ARG(dev >= 0 && dev < CLIP_STATIC_MAX_DEVICES && g_clip_scratch_ptr[dev] != nullptr,
                  "mrl_clip_grad_norm_static: the scratch array of device %d was not resolved at context creation", dev);
    float *part = g_clip_scratch_ptr[dev];
    // same kernels and block count as mrl_clip_grad_norm: the results are the same bit for bit.
    // Every partial that the second kernel reads has been written by the first: nothing to clear.
    int nb = std::min(CLIP_STATIC_PARTIALS, grid_for(n, TPB));
    hipLaunchKernelGGL(sq_partial_kernel, dim3(nb), dim3(TPB), 0, ctx->stream, grads, n, part);
    hipLaunchKernelGGL(clip_apply_kernel, dim3(grid_for(n, TPB)), dim3(TPB), 0, ctx->stream, grads, n,
                       part, nb, max_norm);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_adam_step(mrl_ctx *ctx, float *params, const float *grads, float *state, int n, int t,
                  double lr, double beta1, double beta2, double eps) {
    MRL_CHECK_ARG(ctx, "mrl_adam_step: ctx is NULL");
    MRL_CHECK_ARG(n >= 0 && t >= 1, "mrl_adam_step: need n >= 0 and step count t >= 1");
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(params && grads && state, "mrl_adam_step: NULL buffer");
    // bias corrections in fp64 then rounded, as the host code of the reference does
    float bc1 = (float)(1.0 - pow(beta1, (double)t));
    float bc2 = (float)(1.0 - pow(beta2, (double)t));
    hipLaunchKernelGGL(adam_kernel, dim3(grid_for(n, TPB)), dim3(TPB), 0, ctx->stream, params, grads,
                       reinterpret_cast<float2 *>(state), n, (float)lr, (float)beta1, (float)beta2,
                       (float)(1.0 - beta1), (float)(1.0 - beta2), (float)eps, bc1, bc2);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_clamp_log_std(mrl_ctx *ctx, float *params, int offset, int action_dim) {
    MRL_CHECK_ARG(ctx && params, "mrl_clamp_log_std: NULL argument");
    MRL_CHECK_ARG(offset >= 0 && action_dim > 0, "mrl_clamp_log_std: bad sizes");
    hipLaunchKernelGGL(clamp_log_std_kernel, dim3(grid_for(action_dim, 64)), dim3(64), 0, ctx->stream,
                       params, offset, action_dim);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

}  // extern "C"
