// Environment kernels and their C entry points.
//
// Physics envs (LunarLander): one wavefront-sized workgroup handles 64 consecutive env rows.
// The rows are contiguous in the reference's [B, STATE_SIZE] buffer, so the block copies them
// HBM -> LDS with coalesced 16-byte loads, each lane then steps its own env entirely out of
// LDS (row stride odd => the 64 lanes touch 64 distinct banks for any field), and the fields
// that a step can change are copied back with coalesced stores.  HBM sees each row once in
// and the changed part once out; nothing is re-read.
#include "mrl_host.hpp"
#include "env_classic.hpp"
#include "env_lunar.hpp"

namespace mrl {

constexpr int EPB = 64;  // envs per block == wavefront size

// ---------------------------------------------------------------- CartPole / Pendulum

__global__ __launch_bounds__(256) void cartpole_step_kernel(float *states, int32_t *steps,
                                                            const float *actions, float *rewards,
                                                            float *dones, float *obs, int batch) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= batch) return;
    float4 v = reinterpret_cast<const float4 *>(states)[i];
    float s[4] = {v.x, v.y, v.z, v.w};
    int32_t st = steps[i];
    float r, d;
    cartpole::step(s, st, (int)actions[i], r, d);
    float4 o = make_float4(s[0], s[1], s[2], s[3]);
    reinterpret_cast<float4 *>(states)[i] = o;
    reinterpret_cast<float4 *>(obs)[i] = o;
    steps[i] = st;
    rewards[i] = r;
    dones[i] = d;
}

// mode 0: reset every env; mode 1: reset envs with dones > 0.5 and clear the flag
__global__ __launch_bounds__(256) void cartpole_reset_kernel(float *states, int32_t *steps,
                                                             float *dones, int batch, uint32_t seed,
                                                             int selective) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= batch) return;
    if (selective) {
        if (dones[i] < 0.5f) return;
    }
    float s[4];
    int32_t st;
    cartpole::reset(s, st, i, seed);
    reinterpret_cast<float4 *>(states)[i] = make_float4(s[0], s[1], s[2], s[3]);
    steps[i] = st;
    if (selective) dones[i] = 0.0f;
}

__global__ __launch_bounds__(256) void pendulum_step_kernel(float *states, const float *actions,
                                                            float *rewards, float *dones,
                                                            float *obs, int batch) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= batch) return;
    float4 *row = reinterpret_cast<float4 *>(states) + 2 * (size_t)i;
    float4 a = row[0], b = row[1];
    float s[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float r, d;
    pendulum::step(s, actions[i], r, d);
    row[0] = make_float4(s[0], s[1], s[2], s[3]);
    row[1] = make_float4(s[4], s[5], s[6], s[7]);
    obs[3 * (size_t)i + 0] = s[0];
    obs[3 * (size_t)i + 1] = s[1];
    obs[3 * (size_t)i + 2] = s[2];
    rewards[i] = r;
    dones[i] = d;
}

__global__ __launch_bounds__(256) void pendulum_reset_kernel(float *states, float *dones, int batch,
                                                             uint64_t seed, int selective) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= batch) return;
    if (selective) {
        if (!(dones[i] > 0.5f)) return;
    }
    float s[8];
    pendulum::reset(s, i, seed);
    float4 *row = reinterpret_cast<float4 *>(states) + 2 * (size_t)i;
    row[0] = make_float4(s[0], s[1], s[2], s[3]);
    row[1] = make_float4(s[4], s[5], s[6], s[7]);
    if (selective) dones[i] = 0.0f;
}

// ---------------------------------------------------------------- LunarLander

constexpr int LL_STRIDE = ll::STATE + 1;              // 193: odd => conflict-free lane access
constexpr int LL_CSTRIDE = 8 * CONTACT_SIZE + 1;      // 73
constexpr int LL_DYN = ll::L::JOINTS_OFF;             // [0, 56): obs + bodies + forces

MRL_DEV void stage_in(float *lds, const float *g, int nenv, int lane) {
    // rows are 192 floats = 48 float4, never straddled by a 16-byte load
    const float4 *src = reinterpret_cast<const float4 *>(g);
    const int total4 = nenv * (ll::STATE / 4);
    for (int i = lane; i < total4; i += EPB) {
        float4 v = src[i];
        int f = i * 4;
        int r = f / ll::STATE, c = f - r * ll::STATE;
        float *d = lds + r * LL_STRIDE + c;
        d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
    }
}

MRL_DEV void stage_out_range(const float *lds, float *g, int nenv, int lane, int c0, int c1,
                             const int *row_flag, int want_flag) {
    const int w = c1 - c0;
    const int total = nenv * w;
    for (int i = lane; i < total; i += EPB) {
        int r = i / w, c = c0 + (i - r * w);
        if (row_flag == nullptr || row_flag[r] == want_flag) g[(size_t)r * ll::STATE + c] = lds[r * LL_STRIDE + c];
    }
}

// AUTORESET = false: GPUDiscreteEnv.step_kernel_gpu.  AUTORESET = true: step, then rows that
// finished are re-initialised in place (selective reset) before the observation is copied out.
template <bool AUTORESET>
__global__ __launch_bounds__(EPB) void ll_step_kernel(float *states, const float *actions,
                                                      float *rewards, float *dones, float *obs,
                                                      const float *shapes_g, int batch,
                                                      uint64_t reset_seed) {
    __shared__ float rows[EPB * LL_STRIDE];
    __shared__ float cts[EPB * LL_CSTRIDE];
    __shared__ float shapes[3 * SHAPE_SIZE];
    __shared__ int was_reset[EPB];
    const int lane = threadIdx.x;
    const int env0 = blockIdx.x * EPB;
    const int nenv = min(EPB, batch - env0);
    float *gbase = states + (size_t)env0 * ll::STATE;

    stage_in(rows, gbase, nenv, lane);
    if (lane < 3 * SHAPE_SIZE) shapes[lane] = shapes_g[lane];
    was_reset[lane] = 0;
    __syncthreads();

    if (lane < nenv) {
        const int env = env0 + lane;
        float *row = rows + lane * LL_STRIDE;
        float r, d;
        ll::step_row(row, cts + lane * LL_CSTRIDE, shapes, env, (int)actions[env], r, d);
        rewards[env] = r;
        dones[env] = d;
        if (AUTORESET && d > 0.5f) {
            ll::reset_row(row, ll::combined_seed(reset_seed, env));
            was_reset[lane] = 1;
        }
    }
    __syncthreads();

    // observation out: [nenv, 8] contiguous
    for (int i = lane; i < nenv * ll::OBS; i += EPB) {
        int r = i >> 3, c = i & 7;
        obs[(size_t)env0 * ll::OBS + i] = rows[r * LL_STRIDE + c];
    }
    stage_out_range(rows, gbase, nenv, lane, 0, LL_DYN, nullptr, 0);
    stage_out_range(rows, gbase, nenv, lane, ll::L::META_OFF, ll::STATE, nullptr, 0);
    if (AUTORESET) stage_out_range(rows, gbase, nenv, lane, LL_DYN, ll::L::META_OFF, was_reset, 1);
}

__global__ __launch_bounds__(EPB) void ll_reset_kernel(float *states, const float *dones, int batch,
                                                       uint64_t seed, int selective) {
    __shared__ float rows[EPB * LL_STRIDE];
    __shared__ int was_reset[EPB];
    const int lane = threadIdx.x;
    const int env0 = blockIdx.x * EPB;
    const int nenv = min(EPB, batch - env0);
    was_reset[lane] = 0;
    if (lane < nenv) {
        const int env = env0 + lane;
        if (!selective || dones[env] > 0.5f) {
            ll::reset_row(rows + lane * LL_STRIDE, ll::combined_seed(seed, env));
            was_reset[lane] = 1;
        }
    }
    __syncthreads();
    stage_out_range(rows, states + (size_t)env0 * ll::STATE, nenv, lane, 0, ll::STATE, was_reset, 1);
}

static int cartpole_side(mrl_ctx *ctx, const float *states, int batch, int32_t **out) {
    auto it = ctx->cartpole_steps.find(states);
    if (it != ctx->cartpole_steps.end() && it->second.batch >= batch) {
        *out = it->second.steps;
        return MRL_OK;
    }
    if (it != ctx->cartpole_steps.end()) {
        MRL_CHECK_HIP(hipStreamSynchronize(ctx->stream));
        MRL_CHECK_HIP(hipFree(it->second.steps));
        ctx->cartpole_steps.erase(it);
    }
    int32_t *p = nullptr;
    MRL_CHECK_HIP(hipMalloc(&p, sizeof(int32_t) * (size_t)batch));
    MRL_CHECK_HIP(hipMemsetAsync(p, 0, sizeof(int32_t) * (size_t)batch, ctx->stream));
    ctx->cartpole_steps[states] = {p, batch};
    *out = p;
    return MRL_OK;
}

}  // namespace mrl

using namespace mrl;

extern "C" {

int mrl_env_dims(int env_id, int *state_size, int *obs_dim, int *num_actions, int *action_dim) {
    int s, o, na, ad;
    switch (env_id) {
        case MRL_ENV_CARTPOLE: s = 4; o = 4; na = 2; ad = 0; break;
        case MRL_ENV_PENDULUM: s = 8; o = 3; na = 0; ad = 1; break;
        case MRL_ENV_LUNARLANDER: s = ll::STATE; o = ll::OBS; na = 4; ad = 0; break;
        default: return set_error(MRL_E_UNSUPPORTED, "mrl_env_dims: env_id %d is not built", env_id);
    }
    if (state_size) *state_size = s;
    if (obs_dim) *obs_dim = o;
    if (num_actions) *num_actions = na;
    if (action_dim) *action_dim = ad;
    return MRL_OK;
}

static int env_reset_impl(mrl_ctx *ctx, int env_id, int batch, float *states, float *dones,
                          uint64_t seed, int selective) {
    MRL_CHECK_ARG(ctx, "mrl_env_reset: NULL ctx");
    MRL_CHECK_ARG(batch >= 0, "mrl_env_reset: negative batch");
    if (batch == 0) return MRL_OK;
    MRL_CHECK_ARG(states, "mrl_env_reset: states is NULL");
    MRL_CHECK_ARG(!selective || dones, "mrl_env_selective_reset: dones is NULL");
    switch (env_id) {
        case MRL_ENV_CARTPOLE: {
            int32_t *steps;
            int rc = cartpole_side(ctx, states, batch, &steps);
            if (rc) return rc;
            // reset_kernel (non-selective) hard-wires seed 12345: envs/cartpole.mojo:803;
            // the launcher passes rng_seed only to the selective variant.
            uint32_t s32 = selective ? (uint32_t)seed : 12345u;
            hipLaunchKernelGGL(cartpole_reset_kernel, dim3(grid_for(batch, 256)), dim3(256), 0,
                               ctx->stream, states, steps, dones, batch, s32, selective);
            break;
        }
        case MRL_ENV_PENDULUM:
            hipLaunchKernelGGL(pendulum_reset_kernel, dim3(grid_for(batch, 256)), dim3(256), 0,
                               ctx->stream, states, dones, batch, seed, selective);
            break;
        case MRL_ENV_LUNARLANDER:
            hipLaunchKernelGGL(ll_reset_kernel, dim3(grid_for(batch, EPB)), dim3(EPB), 0,
                               ctx->stream, states, dones, batch, seed, selective);
            break;
        default:
            return set_error(MRL_E_UNSUPPORTED, "mrl_env_reset: env_id %d is not built", env_id);
    }
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_env_reset(mrl_ctx *ctx, int env_id, int batch, float *states, uint64_t seed) {
    return env_reset_impl(ctx, env_id, batch, states, nullptr, seed, 0);
}

int mrl_env_selective_reset(mrl_ctx *ctx, int env_id, int batch, float *states, float *dones,
                            uint64_t seed) {
    return env_reset_impl(ctx, env_id, batch, states, dones, seed, 1);
}

static int env_step_impl(mrl_ctx *ctx, int env_id, int batch, float *states, const float *actions,
                         float *rewards, float *dones, float *obs, uint64_t seed, bool autoreset,
                         uint64_t reset_seed) {
    (void)seed;  // none of the built envs consumes the step seed (their streams are keyed by env/step)
    MRL_CHECK_ARG(ctx, "mrl_env_step: NULL ctx");
    MRL_CHECK_ARG(batch >= 0, "mrl_env_step: negative batch");
    if (batch == 0) return MRL_OK;
    MRL_CHECK_ARG(states && actions && rewards && dones && obs, "mrl_env_step: NULL argument");
    switch (env_id) {
        case MRL_ENV_CARTPOLE: {
            int32_t *steps;
            int rc = cartpole_side(ctx, states, batch, &steps);
            if (rc) return rc;
            hipLaunchKernelGGL(cartpole_step_kernel, dim3(grid_for(batch, 256)), dim3(256), 0,
                               ctx->stream, states, steps, actions, rewards, dones, obs, batch);
            MRL_CHECK_LAUNCH();
            if (autoreset) return set_error(MRL_E_UNSUPPORTED, "autoreset: LunarLander only for now");
            break;
        }
        case MRL_ENV_PENDULUM:
            if (autoreset) return set_error(MRL_E_UNSUPPORTED, "autoreset: LunarLander only for now");
            hipLaunchKernelGGL(pendulum_step_kernel, dim3(grid_for(batch, 256)), dim3(256), 0,
                               ctx->stream, states, actions, rewards, dones, obs, batch);
            break;
        case MRL_ENV_LUNARLANDER:
            if (autoreset)
                hipLaunchKernelGGL(ll_step_kernel<true>, dim3(grid_for(batch, EPB)), dim3(EPB), 0,
                                   ctx->stream, states, actions, rewards, dones, obs, ctx->ll_shapes,
                                   batch, reset_seed);
            else
                hipLaunchKernelGGL(ll_step_kernel<false>, dim3(grid_for(batch, EPB)), dim3(EPB), 0,
                                   ctx->stream, states, actions, rewards, dones, obs, ctx->ll_shapes,
                                   batch, reset_seed);
            break;
        default:
            return set_error(MRL_E_UNSUPPORTED, "mrl_env_step: env_id %d is not built", env_id);
    }
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_env_step(mrl_ctx *ctx, int env_id, int batch, float *states, const float *actions,
                 float *rewards, float *dones, float *obs, uint64_t seed) {
    return env_step_impl(ctx, env_id, batch, states, actions, rewards, dones, obs, seed, false, 0);
}

int mrl_env_step_autoreset(mrl_ctx *ctx, int env_id, int batch, float *states, const float *actions,
                           float *rewards, float *dones, float *obs, uint64_t step_seed,
                           uint64_t reset_seed) {
    return env_step_impl(ctx, env_id, batch, states, actions, rewards, dones, obs, step_seed, true,
                         reset_seed);
}

}  // extern "C"
