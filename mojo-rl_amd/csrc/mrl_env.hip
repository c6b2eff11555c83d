// Environment kernels and their C entry points.
//
// Physics envs: a workgroup handles EPB consecutive env rows.  The rows are contiguous in the
// reference's [B, STATE_SIZE] buffer, so all wavefronts of the block copy them HBM -> LDS with
// coalesced 16-byte loads, one lane of wavefront 0 per env then steps it entirely out of LDS
// (row stride odd => the lanes touch distinct banks for any field) while the other wavefronts
// detect its contacts where the env splits that off, and the fields that a step can change are
// copied back with coalesced stores.  HBM sees each row once in and the changed part once out;
// nothing is re-read.
#include "mrl_host.hpp"
#include "env_classic.hpp"
#include "env_lunar.hpp"
#include "env_walkers.hpp"

namespace mrl {

// _store_post_step_kernel (deep_agents/ppo/ppo.mojo:692-708) + accumulate_rewards /
// increment_steps / extract_completed_episodes (deep_rl/gpu/rl_kernels.mojo:103-200) for one env
MRL_DEV void account(const Accounting &acc, int i, float r, float d) {
    if (acc.r_rewards == nullptr) return;
    acc.r_rewards[i] = r;
    acc.r_dones[i] = d;
    float er = acc.ep_return[i] + r;
    float el = acc.ep_length[i] + 1.0f;
    if (d > 0.5f) {
        int slot = atomicAdd(acc.done_count, 1);
        if (slot < acc.done_cap) {
            acc.done_returns[slot] = er;
            acc.done_lengths[slot] = el;
        }
        er = 0.0f;
        el = 0.0f;
    }
    acc.ep_return[i] = er;
    acc.ep_length[i] = el;
}

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

// ---------------------------------------------------------------- physics2d envs
// Per-env traits of the LDS-staged kernels.  EPB = env rows per workgroup (one wavefront; with
// 32 rows the upper half of the lanes only helps with the copies), DYN_END = first float of the
// row that a step never writes (everything before it, plus the metadata, is copied back).

struct LunarLander {
    using L = ll::L;
    static constexpr int STATE = ll::STATE, OBS = ll::OBS, ACT_W = 1, EPB = 32, THREADS = 512;
    static constexpr int DYN_END = L::JOINTS_OFF, NSHAPE = 3 * SHAPE_SIZE;
    static MRL_DEV void step(float *row, float *cts, const float *shapes, int env, const float *a,
                             float &r, float &d) {
        ll::step_row(row, cts, shapes, env, (int)a[0], r, d);
    }
    static MRL_DEV void reset(float *row, uint64_t seed, int env) {
        ll::reset_row(row, ll::combined_seed(seed, env));
    }
    static constexpr bool WAVE_RESET = true;
    static MRL_DEV void reset_wave(float *row, uint64_t seed, int env, int lane) {
        ll::reset_row_wave(row, ll::combined_seed(seed, env), lane);
    }
    // contact detection runs beside the engines of wavefront 0: every half of wavefronts 1 .. 7
    // takes one (body, vertex) pair of the block's 32 envs -- hull 6 vertices, legs 4 each
    static constexpr int DETECT_TASKS = 14;
    static MRL_DEV void detect_task(int k, int &body, int &vertex, int &max_verts) {
        if (k < 6) { body = 0; vertex = k; max_verts = 6; }
        else if (k < 10) { body = 1; vertex = k - 6; max_verts = 4; }
        else { body = 2; vertex = k - 10; max_verts = 4; }
    }
    using Carry = ll::StepCarry;
    static MRL_DEV Carry step_begin(float *row, int env, const float *a) { return ll::step_begin(row, env, (int)a[0]); }
    static MRL_DEV void step_finish(float *row, float *cts, int n, const float *shapes, const Carry &c, float &r,
                                    float &d) {
        ll::step_finish(row, cts, n, shapes, c, r, d);
    }
};

struct BipedalWalker {
    using L = bw::L;
    static constexpr int STATE = bw::STATE, OBS = bw::OBS, ACT_W = bw::ACT, EPB = 32, THREADS = 256;
    static constexpr int DYN_END = L::EDGES_OFF, NSHAPE = bw::NSHAPE_FLOATS;
    static MRL_DEV void step(float *row, float *cts, const float *shapes, int env, const float *a,
                             float &r, float &d) {
        bw::step_row(row, cts, shapes, env, a, r, d);
    }
    static MRL_DEV void reset(float *row, uint64_t seed, int env) { bw::reset_row(row, walker_seed(seed, env)); }
    static constexpr bool WAVE_RESET = false;
    static MRL_DEV void reset_wave(float *, uint64_t, int, int) {}
    static constexpr int DETECT_TASKS = 0;
    static MRL_DEV void detect_task(int, int &, int &, int &) {}
    struct Carry {};
    static MRL_DEV Carry step_begin(float *, int, const float *) { return Carry{}; }
    static MRL_DEV void step_finish(float *, float *, int, const float *, const Carry &, float &, float &) {}
};

struct HalfCheetah {
    using L = hc::L;
    static constexpr int STATE = hc::STATE, OBS = hc::OBS, ACT_W = hc::ACT, EPB = 64, THREADS = 256;
    static constexpr int DYN_END = L::EDGES_OFF, NSHAPE = hc::NSHAPE_FLOATS;
    static MRL_DEV void step(float *row, float *cts, const float *shapes, int env, const float *a,
                             float &r, float &d) {
        hc::step_row(row, cts, shapes, env, a, r, d);
    }
    static MRL_DEV void reset(float *row, uint64_t seed, int env) { hc::reset_row(row, walker_seed(seed, env)); }
    static constexpr bool WAVE_RESET = false;
    static MRL_DEV void reset_wave(float *, uint64_t, int, int) {}
    static constexpr int DETECT_TASKS = 0;
    static MRL_DEV void detect_task(int, int &, int &, int &) {}
    struct Carry {};
    static MRL_DEV Carry step_begin(float *, int, const float *) { return Carry{}; }
    static MRL_DEV void step_finish(float *, float *, int, const float *, const Carry &, float &, float &) {}
};

constexpr int WAVE = 64;    // the compute phase runs on one wavefront, one lane per env

template <class E>
struct Stage {
    static constexpr int STRIDE = E::STATE | 1;                            // odd => conflict-free lane access
    static constexpr int CSTRIDE = (E::L::MAX_CONTACTS * CONTACT_SCRATCH) | 1;

    // Copies run in batches of UNROLL independent elements per thread (all loads of a batch are
    // issued before the first store), so a thread waits for memory once per batch and not once
    // per element.
    static constexpr int UNROLL = 8;

    static MRL_DEV void in(float *lds, const float *g, int nenv, int lane) {
        if (E::STATE % 4 == 0) {   // rows are whole float4s, never straddled by a 16-byte load
            const float4 *src = reinterpret_cast<const float4 *>(g);
            const int total4 = nenv * (E::STATE / 4);
            for (int i0 = lane; i0 < total4; i0 += UNROLL * E::THREADS) {
                float4 v[UNROLL];
#pragma unroll
                for (int k = 0; k < UNROLL; ++k)
                    if (i0 + k * E::THREADS < total4) v[k] = src[i0 + k * E::THREADS];
#pragma unroll
                for (int k = 0; k < UNROLL; ++k) {
                    if (i0 + k * E::THREADS >= total4) continue;
                    const int f = (i0 + k * E::THREADS) * 4;
                    const int r = f / E::STATE, c = f - r * E::STATE;
                    float *d = lds + r * STRIDE + c;
                    d[0] = v[k].x; d[1] = v[k].y; d[2] = v[k].z; d[3] = v[k].w;
                }
            }
        } else {
            const int total = nenv * E::STATE;
            for (int i0 = lane; i0 < total; i0 += UNROLL * E::THREADS) {
                float v[UNROLL];
#pragma unroll
                for (int k = 0; k < UNROLL; ++k)
                    if (i0 + k * E::THREADS < total) v[k] = g[i0 + k * E::THREADS];
#pragma unroll
                for (int k = 0; k < UNROLL; ++k) {
                    const int i = i0 + k * E::THREADS;
                    if (i >= total) continue;
                    const int r = i / E::STATE, c = i - r * E::STATE;
                    lds[r * STRIDE + c] = v[k];
                }
            }
        }
    }

    // columns [c0, c1) of every row whose bit is set in `rows` (row r = bit r)
    static MRL_DEV void out(const float *lds, float *g, int nenv, int lane, int c0, int c1,
                            unsigned long long rows = ~0ull) {
        const int w = c1 - c0;
        const int total = nenv * w;
        for (int i0 = lane; i0 < total; i0 += UNROLL * E::THREADS) {
            float v[UNROLL];
            int at[UNROLL];
#pragma unroll
            for (int k = 0; k < UNROLL; ++k) {
                const int i = i0 + k * E::THREADS;
                at[k] = -1;
                if (i >= total) continue;
                const int r = i / w, c = c0 + (i - r * w);
                if (!((rows >> r) & 1ull)) continue;
                v[k] = lds[r * STRIDE + c];
                at[k] = r * E::STATE + c;
            }
#pragma unroll
            for (int k = 0; k < UNROLL; ++k)
                if (at[k] >= 0) g[at[k]] = v[k];
        }
    }

    // the same for a set of rows that is usually small: a few rows are copied one after the other
    static MRL_DEV void out_rows(const float *lds, float *g, int nenv, unsigned long long mask, int lane,
                                 int c0, int c1) {
        if (__popcll(mask) > 8) {
            out(lds, g, nenv, lane, c0, c1, mask);
            return;
        }
        while (mask) {
            const int r = __ffsll((long long)mask) - 1;
            mask &= mask - 1;
            for (int c = c0 + lane; c < c1; c += E::THREADS) g[(size_t)r * E::STATE + c] = lds[r * STRIDE + c];
        }
    }
};

// Resets the rows whose bit is set in `mask` (lanes of wavefront 0) and records the mask.  A handful of rows -- the
// usual case inside a step -- are rebuilt one after the other by all 64 lanes together; many rows
// (a full reset) are rebuilt by their own lanes in parallel.
template <class E>
MRL_DEV void reset_rows(float *rows, unsigned long long *was_reset, unsigned long long mask, uint64_t seed,
                        int env0, int lane) {
    using S = Stage<E>;
    if (lane == 0) *was_reset = mask;
    if (E::WAVE_RESET && __popcll(mask) <= 8) {
        while (mask) {
            const int src = __ffsll((long long)mask) - 1;
            mask &= mask - 1;
            E::reset_wave(rows + src * S::STRIDE, seed, env0 + src, lane);
        }
    } else if ((mask >> lane) & 1ull) {
        E::reset(rows + lane * S::STRIDE, seed, env0 + lane);
    }
}

// AUTORESET = false: step_kernel_gpu of the trait.  AUTORESET = true: step, then rows that
// finished are re-initialised in place (selective reset) before the observation is copied out.
template <class E, bool AUTORESET>
__global__ __launch_bounds__(E::THREADS) void phys_step_kernel(float *states, const float *actions,
                                                          float *rewards, float *dones, float *obs,
                                                          const float *shapes_g, int batch,
                                                          uint64_t reset_seed, Accounting acc) {
    using S = Stage<E>;
    __shared__ float rows[E::EPB * S::STRIDE];
    __shared__ float cts[E::EPB * S::CSTRIDE];
    __shared__ float shapes[E::NSHAPE];
    __shared__ unsigned long long was_reset;   // rows re-initialised by this launch, one bit each
    const int tid = threadIdx.x;
    const int env0 = blockIdx.x * E::EPB;
    const int nenv = min(E::EPB, batch - env0);
    float *gbase = states + (size_t)env0 * E::STATE;

    S::in(rows, gbase, nenv, tid);
    for (int i = tid; i < E::NSHAPE; i += E::THREADS) shapes[i] = shapes_g[i];
    if (tid == 0) was_reset = 0;
    __syncthreads();

    if constexpr (E::DETECT_TASKS > 0) {
        // wavefront 0: first half of the step (reads and writes velocities only); the halves of the
        // other wavefronts: contacts of one (body, vertex) pair each (read positions only), into
        // lists of their own.  A list holds DCAP records; a vertex that fills it, or a body whose
        // shape the task table does not cover, sends that env back to detection inside step_finish.
        constexpr int NT = E::DETECT_TASKS, HALF = WAVE / 2, DCAP = 4;
        constexpr int LSTRIDE = (DCAP * CONTACT_SIZE) | 1;
        __shared__ float dlist[NT * E::EPB * LSTRIDE];
        __shared__ int dcount[NT * E::EPB];
        static_assert(E::EPB <= HALF && (NT + 1) / 2 < E::THREADS / WAVE, "two tasks per wavefront besides wavefront 0");
        const int wave = tid / WAVE, lane = tid % WAVE;
        typename E::Carry carry{};
        if (wave == 0) {
            if (lane < nenv)
                carry = E::step_begin(rows + lane * S::STRIDE, env0 + lane, actions + (size_t)(env0 + lane) * E::ACT_W);
        } else {
            const int task = (wave - 1) * 2 + lane / HALF, e = lane % HALF;
            if (task < NT && e < nenv) {
                int body, vertex, max_verts;
                E::detect_task(task, body, vertex, max_verts);
                dcount[task * E::EPB + e] = edge_detect_vertex<typename E::L>(
                    rows + e * S::STRIDE, shapes, body, vertex, max_verts, dlist + (task * E::EPB + e) * LSTRIDE, DCAP);
            }
        }
        __syncthreads();
        if (wave == 0) {
            bool finished = false;
            if (lane < nenv) {
                // concatenate the lists in (body, vertex) order, cut at MAX_CONTACTS
                float *mine = cts + lane * S::CSTRIDE;
                int n = 0;
                bool redo = false;
                for (int k = 0; k < NT; ++k) {
                    const float *src = dlist + (k * E::EPB + lane) * LSTRIDE;
                    const int m = dcount[k * E::EPB + lane];
                    redo |= m < 0;
                    for (int c = 0; c < m && n < E::L::MAX_CONTACTS; ++c, ++n)
                        for (int f = 0; f < CONTACT_SIZE; ++f) mine[n * CONTACT_SIZE + f] = src[c * CONTACT_SIZE + f];
                }
                const int env = env0 + lane;
                float r, d;
                E::step_finish(rows + lane * S::STRIDE, mine, redo ? -1 : n, shapes, carry, r, d);
                rewards[env] = r;
                dones[env] = d;
                account(acc, env, r, d);
                finished = d > 0.5f;
            }
            if (AUTORESET) reset_rows<E>(rows, &was_reset, __ballot(finished), reset_seed, env0, lane);
        }
    } else {
        if (tid < WAVE) {
            bool finished = false;
            if (tid < nenv) {
                const int env = env0 + tid;
                float r, d;
                E::step(rows + tid * S::STRIDE, cts + tid * S::CSTRIDE, shapes, env,
                        actions + (size_t)env * E::ACT_W, r, d);
                rewards[env] = r;
                dones[env] = d;
                account(acc, env, r, d);
                finished = d > 0.5f;
            }
            if (AUTORESET) reset_rows<E>(rows, &was_reset, __ballot(finished), reset_seed, env0, tid);
        }
    }
    __syncthreads();

    for (int i = tid; i < nenv * E::OBS; i += E::THREADS) {   // observation out: [nenv, OBS] contiguous
        int r = i / E::OBS, c = i - r * E::OBS;
        obs[(size_t)env0 * E::OBS + i] = rows[r * S::STRIDE + c];
    }
    S::out(rows, gbase, nenv, tid, 0, E::DYN_END);
    S::out(rows, gbase, nenv, tid, E::L::META_OFF, E::STATE);
    if (AUTORESET) S::out_rows(rows, gbase, nenv, was_reset, tid, E::DYN_END, E::L::META_OFF);
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
    dim3 grid(grid_for(batch, E::EPB));
    if (autoreset)
        hipLaunchKernelGGL((phys_step_kernel<E, true>), grid, dim3(E::THREADS), 0, ctx->stream, states, actions,
                           rewards, dones, obs, shapes, batch, reset_seed, acc);
    else
        hipLaunchKernelGGL((phys_step_kernel<E, false>), grid, dim3(E::THREADS), 0, ctx->stream, states, actions,
                           rewards, dones, obs, shapes, batch, reset_seed, acc);
    return MRL_OK;
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
        case MRL_ENV_BIPEDAL: s = bw::STATE; o = bw::OBS; na = 0; ad = bw::ACT; break;
        case MRL_ENV_HALFCHEETAH: s = hc::STATE; o = hc::OBS; na = 0; ad = hc::ACT; break;
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
        case MRL_ENV_LUNARLANDER: launch_phys_reset<LunarLander>(ctx, batch, states, dones, seed, selective); break;
        case MRL_ENV_BIPEDAL: launch_phys_reset<BipedalWalker>(ctx, batch, states, dones, seed, selective); break;
        case MRL_ENV_HALFCHEETAH: launch_phys_reset<HalfCheetah>(ctx, batch, states, dones, seed, selective); break;
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
        case MRL_ENV_BIPEDAL:
            launch_phys_step<BipedalWalker>(ctx, batch, states, actions, rewards, dones, obs, ctx->bw_shapes,
                                            autoreset, reset_seed, acc);
            break;
        case MRL_ENV_HALFCHEETAH:
            launch_phys_step<HalfCheetah>(ctx, batch, states, actions, rewards, dones, obs, ctx->hc_shapes,
                                          autoreset, reset_seed, acc);
            break;
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
