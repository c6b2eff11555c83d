// Environment kernels and their C entry points.
//
// Physics envs: a workgroup handles EPB consecutive env rows.  The rows are contiguous in the
// reference's [B, STATE_SIZE] buffer, so all wavefronts of the block copy them HBM -> LDS with
// coalesced 16-byte loads, one lane of wavefront 0 per env then steps it entirely out of LDS
// (row stride odd => the lanes touch distinct banks for any field) while the other wavefronts
// detect its contacts where the env splits that off, and the fields that a step can change are
// copied back with coalesced stores.  HBM sees each row once in and the changed part once out;
// nothing is re-read.  (LunarLander above 8192 envs: one lane per env on rows left in global memory,
// phys_step_lane_kernel.)
#include <cmath>
#include "mrl_host.hpp"
#include "env_classic.hpp"
#include "env_block.hpp"
#include "env_cheetah_lanes.hpp"
#include "env_car.hpp"
#include "env_planar.hpp"

namespace mrl {

// ---------------------------------------------------------------- CartPole / Pendulum

// autoreset: a finished env is re-initialised with the selective-reset stream before its state and
// observation are written; rewards / dones still report the step that ended the episode
__global__ __launch_bounds__(256) void cartpole_step_kernel(float *states, int32_t *steps,
                                                            const float *actions, float *rewards,
                                                            float *dones, float *obs, int batch,
                                                            int autoreset, uint32_t reset_seed,
                                                            Accounting acc) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= batch) return;
    float4 v = reinterpret_cast<const float4 *>(states)[i];
    float s[4] = {v.x, v.y, v.z, v.w};
    int32_t st = steps[i];
    float r, d;
    cartpole::step(s, st, (int)actions[i], r, d);
    if (autoreset && d > 0.5f) cartpole::reset(s, st, i, reset_seed);
    float4 o = make_float4(s[0], s[1], s[2], s[3]);
    reinterpret_cast<float4 *>(states)[i] = o;
    reinterpret_cast<float4 *>(obs)[i] = o;
    steps[i] = st;
    rewards[i] = r;
    dones[i] = d;
    account(acc, i, r, d);
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
                                                            float *obs, int batch, int autoreset,
                                                            uint64_t reset_seed, Accounting acc) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= batch) return;
    float4 *row = reinterpret_cast<float4 *>(states) + 2 * (size_t)i;
    float4 a = row[0], b = row[1];
    float s[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float r, d;
    pendulum::step(s, actions[i], r, d);
    if (autoreset && d > 0.5f) pendulum::reset(s, i, reset_seed);
    row[0] = make_float4(s[0], s[1], s[2], s[3]);
    row[1] = make_float4(s[4], s[5], s[6], s[7]);
    obs[3 * (size_t)i + 0] = s[0];
    obs[3 * (size_t)i + 1] = s[1];
    obs[3 * (size_t)i + 2] = s[2];
    rewards[i] = r;
    dones[i] = d;
    account(acc, i, r, d);
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

// AUTORESET = false: step_kernel_gpu of the trait.  AUTORESET = true: step, then rows that
// finished are re-initialised in place (selective reset) before the observation is copied out.
template <class E, bool AUTORESET>
__device__ __forceinline__ void phys_step_body(float *states, const float *actions, float *rewards, float *dones,
                                               float *obs, const float *shapes_g, int batch, uint64_t reset_seed,
                                               Accounting acc) {
    using S = Stage<E>;
    __shared__ float rows[E::EPB * S::STRIDE];
    __shared__ float cts[E::EPB * S::CSTRIDE];
    __shared__ float shapes[E::NSHAPE];
    __shared__ unsigned long long was_reset;   // rows re-initialised by this launch, one bit each
    __shared__ float dlist[detect_list_floats<E>() + 1];
    __shared__ int dcount[detect_count_ints<E>()];
    const int tid = threadIdx.x;
    const int env0 = blockIdx.x * E::EPB;
    const int nenv = min(E::EPB, batch - env0);
    float *gbase = states + (size_t)env0 * E::STATE;

    S::in(rows, gbase, nenv, tid);
    for (int i = tid; i < E::NSHAPE; i += E::THREADS) shapes[i] = shapes_g[i];
    if (tid == 0) was_reset = 0;
    __syncthreads();

    phys_step_block<E, AUTORESET>(rows, cts, shapes, dlist, dcount, &was_reset,
                                  actions + (size_t)env0 * E::ACT_W, rewards + env0, dones + env0, env0, nenv,
                                  reset_seed, acc.at(env0));
    __syncthreads();

    for (int i = tid; i < nenv * E::OBS; i += E::THREADS) {   // observation out: [nenv, OBS] contiguous
        int r = i / E::OBS, c = i - r * E::OBS;
        obs[(size_t)env0 * E::OBS + i] = rows[r * S::STRIDE + c];
    }
    S::out(rows, gbase, nenv, tid, 0, E::DYN_END);
    S::out(rows, gbase, nenv, tid, E::L::META_OFF, E::STATE);
    if (AUTORESET) S::out_rows(rows, gbase, nenv, was_reset, tid, E::DYN_END, E::L::META_OFF);
}

template <class E, bool AUTORESET>
__global__ __launch_bounds__(E::THREADS) void phys_step_kernel(float *states, const float *actions,
                                                          float *rewards, float *dones, float *obs,
                                                          const float *shapes_g, int batch,
                                                          uint64_t reset_seed, Accounting acc) {
    phys_step_body<E, AUTORESET>(states, actions, rewards, dones, obs, shapes_g, batch, reset_seed, acc);
}

// The same step with one lane per ENV and the rows left in global memory (64 envs per single-wavefront
// workgroup, only the contact scratch in LDS): nothing is shared between lanes, so a batch that fills the
// chip runs at the rate of the vector units instead of at the latency of one workgroup's phase chain.
// Used from E::LANE_FROM envs on (LunarLander: one wavefront's step lasts 44 us whatever the batch, the
// 32-row workgroup's 33 us, but a CU holds five of these wavefronts and one such workgroup).
template <class E, bool AUTORESET>
__global__ __launch_bounds__(64) void phys_step_lane_kernel(float *states, const float *actions, float *rewards,
                                                            float *dones, float *obs, const float *shapes_g, int batch,
                                                            uint64_t reset_seed, Accounting acc) {
    using S = Stage<E>;
    __shared__ float cts[WAVE * S::CSTRIDE];
    __shared__ float shapes[E::NSHAPE];
    const int lane = threadIdx.x;
    const int env = blockIdx.x * WAVE + lane;
    for (int i = lane; i < E::NSHAPE; i += WAVE) shapes[i] = shapes_g[i];
    __syncthreads();
    if (env >= batch) return;
    float *row = states + (size_t)env * E::STATE;
    const EpisodeSums sums = account_before(acc, env);
    float r, d;
    E::step(row, cts + lane * S::CSTRIDE, shapes, env, actions + (size_t)env * E::ACT_W, r, d);
    rewards[env] = r;
    dones[env] = d;
    account(acc, env, r, d, sums);
    if (AUTORESET && d > 0.5f) E::reset(row, reset_seed, env);
#pragma unroll
    for (int k = 0; k < E::OBS; ++k) obs[(size_t)env * E::OBS + k] = row[k];
}

// HalfCheetah with one lane per body (env_cheetah_lanes.hpp): a workgroup is one wavefront with
// eight envs, so 4096 envs are 512 wavefronts spread over the chip instead of 64 long ones.  Rows
// are staged through LDS as in phys_step_kernel; a row whose wiring is not HalfCheetah's own is
// stepped by lane 0 of its group with the one-lane form.
struct HalfCheetahLanes : HalfCheetah {
    static constexpr int EPB = 8, THREADS = 64;
};

template <bool AUTORESET>
__global__ __launch_bounds__(64) void hc_lanes_step_kernel(float *states, const float *actions, float *rewards,
                                                          float *dones, float *obs, const float *shapes_g,
                                                          int batch, uint64_t reset_seed, Accounting acc) {
    using E = HalfCheetahLanes;
    using S = Stage<E>;
    __shared__ float rows[E::EPB * S::STRIDE];
    __shared__ float cts[E::EPB * S::CSTRIDE];   // contact scratch of the one-lane form
    __shared__ float shapes[E::NSHAPE];
    const int lane = threadIdx.x;
    const int env0 = blockIdx.x * E::EPB;
    const int nenv = min(E::EPB, batch - env0);
    float *gbase = states + (size_t)env0 * E::STATE;
    S::in(rows, gbase, nenv, lane);
    for (int i = lane; i < E::NSHAPE; i += E::THREADS) shapes[i] = shapes_g[i];
    __syncthreads();

    const int slot = lane >> 3, b = lane & 7;
    const bool live = slot < nenv;
    // groups beyond the batch work on LDS rows of their own that are never copied out
    float *row = rows + slot * S::STRIDE;
    const int env = env0 + (live ? slot : 0);
    const float *act = actions + (size_t)env * E::ACT_W;
    const bool ok = live && hc::lanes_row_ok(row, shapes);
    float r = 0.0f, d = 0.0f;
    if (ok) hc::step_lanes(row, shapes, act, lane, r, d);
    else if (live && b == 0) hc::step_row(row, cts + slot * S::CSTRIDE, shapes, env, act, r, d);
    bool finished = false;
    if (live && b == 0) {
        rewards[env] = r;
        dones[env] = d;
        account(acc.at(env0), slot, r, d);
        finished = d > 0.5f;
        if (AUTORESET && finished) E::reset(row, reset_seed, env);
    }
    const unsigned long long fin = __ballot(finished);
    unsigned long long was_reset = 0;
#pragma unroll
    for (int k = 0; k < E::EPB; ++k) was_reset |= ((fin >> (8 * k)) & 1ull) << k;
    __syncthreads();

    for (int i = lane; i < nenv * E::OBS; i += E::THREADS) {
        int rr = i / E::OBS, c = i - rr * E::OBS;
        obs[(size_t)env0 * E::OBS + i] = rows[rr * S::STRIDE + c];
    }
    S::out(rows, gbase, nenv, lane, 0, E::DYN_END);
    S::out(rows, gbase, nenv, lane, E::L::META_OFF, E::STATE);
    if (AUTORESET) S::out_rows(rows, gbase, nenv, was_reset, lane, E::DYN_END, E::L::META_OFF);
}

// CarRacingV2 (env_car.hpp): a wavefront per env for the step, sixteen lanes per env for a reset of
// its own (where one lane of the group walks the track); rows in global memory
constexpr int CAR_THREADS = 256, CAR_EPB = CAR_THREADS / cr::STEP_LANES;
constexpr int CAR_RESET_GROUP = 16, CAR_RESET_EPB = CAR_THREADS / CAR_RESET_GROUP;

template <bool AUTORESET>
__global__ __launch_bounds__(CAR_THREADS) void car_step_kernel(float *states, const float *actions, float *rewards,
                                                               float *dones, float *obs, int batch,
                                                               uint64_t reset_seed, Accounting acc, int trait_form) {
    __shared__ __align__(16) float tables[CAR_EPB][cr::TABLE];   // each wavefront's copy of its env's tile table
    const int sub = threadIdx.x & 63, wave = threadIdx.x / cr::STEP_LANES;
    const int env = blockIdx.x * CAR_EPB + wave;
    if (env >= batch) return;   // whole wavefronts leave together
    float *row = states + (size_t)env * cr::STATE;
    float r, d, ob[cr::OBS];
    cr::step_wave(row, row, tables[wave], actions + (size_t)env * cr::ACT, sub, r, d, ob, trait_form != 0);
    if (sub == 0) {
        rewards[env] = r;
        dones[env] = d;
        account(acc, env, r, d);
    }
    if (AUTORESET && d > 0.5f) {
        float sx, sy, sa;
        cr::reset_group<cr::STEP_LANES>(row, cr::combined_seed(reset_seed, env), sub, sx, sy, sa);
#pragma unroll
        for (int k = 3; k < cr::OBS; ++k) ob[k] = 0.0f;
        ob[0] = sx; ob[1] = sy; ob[2] = sa;
    }
    // the observation the row now starts with, straight from the registers (every lane holds all of it)
    float mine = ob[0];
#pragma unroll
    for (int k = 1; k < cr::OBS; ++k) mine = sub == k ? ob[k] : mine;
    if (sub < cr::OBS) obs[(size_t)env * cr::OBS + sub] = mine;
}

__global__ __launch_bounds__(CAR_THREADS) void car_reset_kernel(float *states, float *dones, int batch, uint64_t seed,
                                                                int selective) {
    const int lane = threadIdx.x & 63, sub = lane & (CAR_RESET_GROUP - 1);
    const int env = blockIdx.x * CAR_RESET_EPB + threadIdx.x / CAR_RESET_GROUP;
    if (env >= batch) return;
    if (selective) {
        if (!(dones[env] > 0.5f)) return;
    }
    float sx, sy, sa;
    cr::reset_group<CAR_RESET_GROUP>(states + (size_t)env * cr::STATE, cr::combined_seed(seed, env), lane, sx, sy, sa);
    if (selective && sub == 0) dones[env] = 0.0f;
}

// HopperPlanar / Walker2dPlanar (env_planar.hpp): one lane per env, the Float64 state in registers for the
// step.  Rows are 248 / 392 bytes: a workgroup's 128 rows are one contiguous range, copied to LDS and back
// with every lane moving 8 bytes next to its neighbour's; a lane then reads its own row out of LDS (a row is
// an odd number of doubles, so the lanes' reads of one field fall into different banks).
constexpr int PLANAR_ROWS = 128;
template <class M, bool AUTORESET>
__global__ __launch_bounds__(PLANAR_ROWS) void planar_step_kernel(float *states, const float *actions, float *rewards,
                                                                  float *dones, float *obs, int batch,
                                                                  uint64_t reset_seed, Accounting acc) {
    __shared__ __align__(16) float slab[PLANAR_ROWS * M::STATE];
    static_assert(M::STATE % 2 == 0 && (M::STATE / 2) % 2 == 1, "rows are whole doubles, an odd number of them");
    const int tid = threadIdx.x;
    const int env0 = blockIdx.x * PLANAR_ROWS;
    const int nenv = min(PLANAR_ROWS, batch - env0);
    float2 *g = reinterpret_cast<float2 *>(states + (size_t)env0 * M::STATE);
    float2 *l = reinterpret_cast<float2 *>(slab);
    constexpr int PER_LANE = M::STATE / 2;           // 8-byte pieces of the slab per lane when it is full
    if (nenv == PLANAR_ROWS) {
#pragma unroll
        for (int k = 0; k < PER_LANE; ++k) l[tid + k * PLANAR_ROWS] = g[tid + k * PLANAR_ROWS];
    } else {
        for (int i = tid; i < nenv * PER_LANE; i += PLANAR_ROWS) l[i] = g[i];
    }
    __syncthreads();
    if (tid < nenv) {
        const int i = env0 + tid;
        float *row = slab + tid * M::STATE;
        planar::State<M> s;
        s.load(row);
        float a[M::ACT];
#pragma unroll
        for (int k = 0; k < M::ACT; ++k) a[k] = actions[(size_t)i * M::ACT + k];
        const bool was_done = s.meta[1] > 0.5;       // such a row is left as it is
        float r, d;
        planar::step<M>(s, a, r, d);
        const bool fresh = AUTORESET && d > 0.5f;
        if (fresh) planar::reset<M>(s, planar::combined_seed(reset_seed, i));
        if (!was_done || fresh) s.store(row);
        rewards[i] = r;
        dones[i] = d;
        account(acc, i, r, d);
    }
    __syncthreads();
    if (nenv == PLANAR_ROWS) {
#pragma unroll
        for (int k = 0; k < PER_LANE; ++k) g[tid + k * PLANAR_ROWS] = l[tid + k * PLANAR_ROWS];
    } else {
        for (int i = tid; i < nenv * PER_LANE; i += PLANAR_ROWS) g[i] = l[i];
    }
    for (int i = tid; i < nenv * M::OBS; i += PLANAR_ROWS) {   // observation out: [nenv, OBS] contiguous
        const int r = i / M::OBS, c = i - r * M::OBS;
        obs[(size_t)env0 * M::OBS + i] = slab[r * M::STATE + c];
    }
}

template <class M>
__global__ __launch_bounds__(256) void planar_reset_kernel(float *states, float *dones, int batch, uint64_t seed,
                                                           int selective) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= batch) return;
    if (selective) {
        if (!(dones[i] > 0.5f)) return;
    }
    planar::State<M> s;
    planar::reset<M>(s, planar::combined_seed(seed, i));
    s.store(states + (size_t)i * M::STATE);
    if (selective) dones[i] = 0.0f;
}

template <class E>
__global__ __launch_bounds__(E::THREADS) void phys_reset_kernel(float *states, const float *dones, int batch,
                                                           uint64_t seed, int selective) {
    using S = Stage<E>;
    __shared__ float rows[E::EPB * S::STRIDE];
    __shared__ unsigned long long was_reset;   // rows re-initialised by this launch, one bit each
    const int tid = threadIdx.x;
    const int env0 = blockIdx.x * E::EPB;
    const int nenv = min(E::EPB, batch - env0);
    if (tid == 0) was_reset = 0;
    __syncthreads();
    if (tid < WAVE) {
        const bool want = tid < nenv && (!selective || dones[env0 + tid] > 0.5f);
        reset_rows<E>(rows, &was_reset, __ballot(want), seed, env0, tid);
    }
    __syncthreads();
    S::out_rows(rows, states + (size_t)env0 * E::STATE, nenv, was_reset, tid, 0, E::STATE);
}

template <class E>
static int launch_phys_reset(mrl_ctx *ctx, int batch, float *states, const float *dones, uint64_t seed,
                             int selective) {
    hipLaunchKernelGGL(phys_reset_kernel<E>, dim3(grid_for(batch, E::EPB)), dim3(E::THREADS), 0, ctx->stream,
                       states, dones, batch, seed, selective);
    return MRL_OK;
}

template <class E>
static int launch_phys_step(mrl_ctx *ctx, int batch, float *states, const float *actions, float *rewards,
                            float *dones, float *obs, const float *shapes, bool autoreset,
                            uint64_t reset_seed, const Accounting &acc) {
    if constexpr (E::LANE_FROM > 0) {
        if (batch >= E::LANE_FROM) {
            dim3 grid64(grid_for(batch, WAVE));
            if (autoreset)
                hipLaunchKernelGGL((phys_step_lane_kernel<E, true>), grid64, dim3(WAVE), 0, ctx->stream, states, actions,
                                   rewards, dones, obs, shapes, batch, reset_seed, acc);
            else
                hipLaunchKernelGGL((phys_step_lane_kernel<E, false>), grid64, dim3(WAVE), 0, ctx->stream, states, actions,
                                   rewards, dones, obs, shapes, batch, reset_seed, acc);
            return MRL_OK;
        }
    }
    dim3 grid(grid_for(batch, E::EPB));
    if (autoreset)
        hipLaunchKernelGGL((phys_step_kernel<E, true>), grid, dim3(E::THREADS), 0, ctx->stream, states, actions,
                           rewards, dones, obs, shapes, batch, reset_seed, acc);
    else
        hipLaunchKernelGGL((phys_step_kernel<E, false>), grid, dim3(E::THREADS), 0, ctx->stream, states, actions,
                           rewards, dones, obs, shapes, batch, reset_seed, acc);
    return MRL_OK;
}

int cartpole_side(mrl_ctx *ctx, const float *states, int batch, int32_t **out) {
    auto it = ctx->cartpole_steps.find(states);
    if (it != ctx->cartpole_steps.end() && it->second.batch >= batch) {
        *out = it->second.steps;
        return MRL_OK;
    }
    if (it != ctx->cartpole_steps.end()) {
        if (!it->second.owned)
            return set_error(MRL_E_ARG, "CartPole: the step counters bound to these states hold %d envs, the call has %d",
                             it->second.batch, batch);
        MRL_CHECK_HIP(hipStreamSynchronize(ctx->stream));
        MRL_CHECK_HIP(hipFree(it->second.steps));
        ctx->cartpole_steps.erase(it);
    }
    int32_t *p = nullptr;
    MRL_CHECK_HIP(hipMalloc(&p, sizeof(int32_t) * (size_t)batch));
    MRL_CHECK_HIP(hipMemsetAsync(p, 0, sizeof(int32_t) * (size_t)batch, ctx->stream));
    ctx->cartpole_steps[states] = {p, batch, true};
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
        case MRL_ENV_LUNARLANDER_CONTINUOUS: s = ll::STATE; o = ll::OBS; na = 0; ad = 2; break;
        case MRL_ENV_BIPEDAL: s = bw::STATE; o = bw::OBS; na = 0; ad = bw::ACT; break;
        case MRL_ENV_HALFCHEETAH: s = hc::STATE; o = hc::OBS; na = 0; ad = hc::ACT; break;
        case MRL_ENV_CARRACING: s = cr::STATE; o = cr::OBS; na = 0; ad = cr::ACT; break;
        case MRL_ENV_HOPPER_PLANAR: s = planar::Hopper::STATE; o = planar::Hopper::OBS; na = 0; ad = planar::Hopper::ACT; break;
        case MRL_ENV_WALKER2D_PLANAR: s = planar::Walker2d::STATE; o = planar::Walker2d::OBS; na = 0; ad = planar::Walker2d::ACT; break;
        default: return set_error(MRL_E_UNSUPPORTED, "mrl_env_dims: env_id %d is not built", env_id);
    }
    if (state_size) *state_size = s;
    if (obs_dim) *obs_dim = o;
    if (num_actions) *num_actions = na;
    if (action_dim) *action_dim = ad;
    return MRL_OK;
}

int mrl_cartpole_bind_steps(mrl_ctx *ctx, const float *states, int batch, int32_t *steps) {
    MRL_CHECK_ARG(ctx && states, "mrl_cartpole_bind_steps: NULL argument");
    MRL_CHECK_ARG(batch >= 0, "mrl_cartpole_bind_steps: negative batch");
    auto it = ctx->cartpole_steps.find(states);
    if (it != ctx->cartpole_steps.end()) {
        if (it->second.owned) {
            MRL_CHECK_HIP(hipStreamSynchronize(ctx->stream));
            MRL_CHECK_HIP(hipFree(it->second.steps));
        }
        ctx->cartpole_steps.erase(it);
    }
    if (steps != nullptr) ctx->cartpole_steps[states] = {steps, batch, false};
    return MRL_OK;
}

__global__ void lunar_wind_kernel(float *shapes, float on, float wind_power, float turbulence_power) {
    if (threadIdx.x == 0) {
        shapes[mrl::ll::WIND_OFF] = on;
        shapes[mrl::ll::WIND_OFF + 1] = wind_power;
        shapes[mrl::ll::WIND_OFF + 2] = turbulence_power;
    }
}

int mrl_car_racing_set_step_form(mrl_ctx *ctx, int form) {
    MRL_CHECK_ARG(ctx, "mrl_car_racing_set_step_form: NULL ctx");
    MRL_CHECK_ARG(form == MRL_CAR_STEP_CPU_ENV || form == MRL_CAR_STEP_GPU_TRAIT,
                  "mrl_car_racing_set_step_form: form %d is neither MRL_CAR_STEP_CPU_ENV nor MRL_CAR_STEP_GPU_TRAIT", form);
    ctx->car_trait_form = form;   // a kernel argument of the launches made from now on
    return MRL_OK;
}

int mrl_lunar_set_wind(mrl_ctx *ctx, int enable, double wind_power, double turbulence_power) {
    MRL_CHECK_ARG(ctx, "mrl_lunar_set_wind: NULL ctx");
    MRL_CHECK_ARG(std::isfinite(wind_power) && std::isfinite(turbulence_power),
                  "mrl_lunar_set_wind: powers must be finite");
    // on the context's stream: steps enqueued before the call keep the old setting, steps after it see the new one
    hipLaunchKernelGGL(lunar_wind_kernel, dim3(1), dim3(64), 0, ctx->stream, ctx->ll_shapes, enable ? 1.0f : 0.0f,
                       (float)wind_power, (float)turbulence_power);
    MRL_CHECK_LAUNCH();
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
        case MRL_ENV_LUNARLANDER_CONTINUOUS:
            launch_phys_reset<LunarLander>(ctx, batch, states, dones, seed, selective);
            break;
        case MRL_ENV_BIPEDAL: launch_phys_reset<BipedalWalker>(ctx, batch, states, dones, seed, selective); break;
        case MRL_ENV_HALFCHEETAH: launch_phys_reset<HalfCheetah>(ctx, batch, states, dones, seed, selective); break;
        case MRL_ENV_CARRACING:
            hipLaunchKernelGGL(car_reset_kernel, dim3(grid_for(batch, CAR_RESET_EPB)), dim3(CAR_THREADS), 0, ctx->stream, states,
                               dones, batch, seed, selective);
            break;
        case MRL_ENV_HOPPER_PLANAR:
            MRL_CHECK_ARG(reinterpret_cast<uintptr_t>(states) % 8 == 0, "mrl_env_reset: HopperPlanar rows hold doubles: states must be 8-byte aligned");
            hipLaunchKernelGGL(planar_reset_kernel<planar::Hopper>, dim3(grid_for(batch, 256)), dim3(256), 0, ctx->stream,
                               states, dones, batch, seed, selective);
            break;
        case MRL_ENV_WALKER2D_PLANAR:
            MRL_CHECK_ARG(reinterpret_cast<uintptr_t>(states) % 8 == 0, "mrl_env_reset: Walker2dPlanar rows hold doubles: states must be 8-byte aligned");
            hipLaunchKernelGGL(planar_reset_kernel<planar::Walker2d>, dim3(grid_for(batch, 256)), dim3(256), 0, ctx->stream,
                               states, dones, batch, seed, selective);
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
                         uint64_t reset_seed, const Accounting &acc) {
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
                               ctx->stream, states, steps, actions, rewards, dones, obs, batch,
                               autoreset ? 1 : 0, (uint32_t)reset_seed, acc);
            break;
        }
        case MRL_ENV_PENDULUM:
            hipLaunchKernelGGL(pendulum_step_kernel, dim3(grid_for(batch, 256)), dim3(256), 0,
                               ctx->stream, states, actions, rewards, dones, obs, batch,
                               autoreset ? 1 : 0, reset_seed, acc);
            break;
        case MRL_ENV_LUNARLANDER:
            launch_phys_step<LunarLander>(ctx, batch, states, actions, rewards, dones, obs, ctx->ll_shapes,
                                          autoreset, reset_seed, acc);
            break;
        case MRL_ENV_LUNARLANDER_CONTINUOUS:
            launch_phys_step<LunarLanderContinuous>(ctx, batch, states, actions, rewards, dones, obs, ctx->ll_shapes,
                                                    autoreset, reset_seed, acc);
            break;
        case MRL_ENV_BIPEDAL:
            launch_phys_step<BipedalWalker>(ctx, batch, states, actions, rewards, dones, obs, ctx->bw_shapes,
                                            autoreset, reset_seed, acc);
            break;
        case MRL_ENV_HALFCHEETAH: {
            const dim3 grid(grid_for(batch, HalfCheetahLanes::EPB)), block(HalfCheetahLanes::THREADS);
            if (autoreset)
                hipLaunchKernelGGL((hc_lanes_step_kernel<true>), grid, block, 0, ctx->stream, states, actions, rewards,
                                   dones, obs, ctx->hc_shapes, batch, reset_seed, acc);
            else
                hipLaunchKernelGGL((hc_lanes_step_kernel<false>), grid, block, 0, ctx->stream, states, actions, rewards,
                                   dones, obs, ctx->hc_shapes, batch, reset_seed, acc);
            break;
        }
        case MRL_ENV_CARRACING: {
            const dim3 grid(grid_for(batch, CAR_EPB)), block(CAR_THREADS);
            if (autoreset)
                hipLaunchKernelGGL((car_step_kernel<true>), grid, block, 0, ctx->stream, states, actions, rewards, dones,
                                   obs, batch, reset_seed, acc, ctx->car_trait_form);
            else
                hipLaunchKernelGGL((car_step_kernel<false>), grid, block, 0, ctx->stream, states, actions, rewards, dones,
                                   obs, batch, reset_seed, acc, ctx->car_trait_form);
            break;
        }
        case MRL_ENV_HOPPER_PLANAR:
        case MRL_ENV_WALKER2D_PLANAR: {
            MRL_CHECK_ARG(reinterpret_cast<uintptr_t>(states) % 8 == 0, "mrl_env_step: the planar envs' rows hold doubles: states must be 8-byte aligned");
            const dim3 grid(grid_for(batch, PLANAR_ROWS)), block(PLANAR_ROWS);
            const bool hopper = env_id == MRL_ENV_HOPPER_PLANAR;
            if (hopper && autoreset)
                hipLaunchKernelGGL((planar_step_kernel<planar::Hopper, true>), grid, block, 0, ctx->stream, states, actions,
                                   rewards, dones, obs, batch, reset_seed, acc);
            else if (hopper)
                hipLaunchKernelGGL((planar_step_kernel<planar::Hopper, false>), grid, block, 0, ctx->stream, states, actions,
                                   rewards, dones, obs, batch, reset_seed, acc);
            else if (autoreset)
                hipLaunchKernelGGL((planar_step_kernel<planar::Walker2d, true>), grid, block, 0, ctx->stream, states, actions,
                                   rewards, dones, obs, batch, reset_seed, acc);
            else
                hipLaunchKernelGGL((planar_step_kernel<planar::Walker2d, false>), grid, block, 0, ctx->stream, states, actions,
                                   rewards, dones, obs, batch, reset_seed, acc);
            break;
        }
        default:
            return set_error(MRL_E_UNSUPPORTED, "mrl_env_step: env_id %d is not built", env_id);
    }
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_env_step(mrl_ctx *ctx, int env_id, int batch, float *states, const float *actions,
                 float *rewards, float *dones, float *obs, uint64_t seed) {
    return env_step_impl(ctx, env_id, batch, states, actions, rewards, dones, obs, seed, false, 0,
                         Accounting{});
}

int mrl_env_step_autoreset(mrl_ctx *ctx, int env_id, int batch, float *states, const float *actions,
                           float *rewards, float *dones, float *obs, uint64_t step_seed,
                           uint64_t reset_seed) {
    return env_step_impl(ctx, env_id, batch, states, actions, rewards, dones, obs, step_seed, true,
                         reset_seed, Accounting{});
}

}  // extern "C"

int mrl::env_step_accounting(mrl_ctx *ctx, int env_id, int batch, float *states, const float *actions,
                             float *rewards, float *dones, float *obs, uint64_t step_seed,
                             uint64_t reset_seed, const Accounting &acc) {
    return env_step_impl(ctx, env_id, batch, states, actions, rewards, dones, obs, step_seed, true,
                         reset_seed, acc);
}
