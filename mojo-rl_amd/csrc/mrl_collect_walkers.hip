// Fused collection kernels of the continuous-control envs beyond the classic ones (BipedalWalker,
// HalfCheetah planar, CarRacingV2, HopperPlanar, Walker2dPlanar) with the agents' 256-wide Gaussian nets: many rollout steps of a
// block's 16 envs in ONE launch, like the kernels of mrl_collect.hip.  The env rows (CarRacing: the 40
// floats in front of the track) stay in LDS from the first step to the last; per step and block
//   policy   the actor  OBS -> 256 -> 256 -> A  on wavefronts 0 .. 3 and the critic  OBS -> 256 -> 256 -> 1
//            on four others, on the fp32 matrix cores (the 16-row tiles of mlp_tile16.hpp, 64 columns
//            per wavefront, weights streamed from L2), heads out of LDS.  The walkers: only the actor runs
//            ahead of the env step; the critic, whose value is only stored, runs beside the one-lane-per-
//            body solver on wavefronts 2, 3, 6 and 7 (the two SIMDs that the solver's wavefronts 0 and 1
//            do not use).  CarRacing, whose env step takes every wavefront: both nets side by side
//            (critic on wavefronts 4 .. 7) ahead of it;
//   sample   one lane per (env, action component): every component has a Philox stream of its own;
//   env step BipedalWalker: the workgroup-level step of env_block.hpp (contact detection on every
//            wavefront, solver with one lane per body on wavefronts 0 and 1, lidar rays on every
//            wavefront, wave-cooperative resets); HalfCheetah: one lane per body on wavefronts 0 and 1
//            (env_cheetah_lanes.hpp); CarRacing: a wavefront per env, two rounds of eight (env_car.hpp);
//            the tile tables stay in global memory and are staged through LDS every step (16 x 12 KB do
//            not fit beside the rest); HopperPlanar / Walker2dPlanar: one lane per env on wavefront 0
//            (Float64, env_planar.hpp), the critic beside it as for the walkers;
//   rollout row t of obs, action, log-prob, value, reward, done written on the way.
// With these envs the step is 70 - 80 % env step, a chain of one or two wavefronts' instructions: what the
// fusion buys is the launch gaps, the observation / action round trip through HBM, the staging of the rows
// in and out of LDS every step, and a policy forward of a 16-row tile on one CU.
//
// It gives what n_steps calls of mrl_rollout_step give (same per-env streams: seeds are affine in
// the step number), except that the finished-episode list is appended in the order in which blocks
// get there rather than step by step.
#include "mrl_host.hpp"
#include "mrl_device.hpp"
#include "mlp_tile.hpp"
#include "mlp_tile16.hpp"
#include "policy_sample.hpp"
#include "env_block.hpp"
#include "env_cheetah_lanes.hpp"
#include "env_car.hpp"
#include "env_planar.hpp"
#include "collect_args.hpp"

namespace mrl {

// HalfCheetah's traits with the block shape of this kernel
struct HalfCheetah16 : HalfCheetah {
    static constexpr int EPB = 16, THREADS = 512;
};

template <int A, int B>
constexpr int wmax() { return A > B ? A : B; }

// The policy half of a step, by all 512 threads: observation tile from `obs_at(row, column)` (also out to
// rollout row t), actor on wavefronts 0 .. 3 and critic on 4 .. 7 (tiles = 2 * H * HT16_LD floats of LDS),
// Gaussian sampling on one lane per (env, action component) -- the log-probability is the sum of the
// components' terms in component order --, rollout row t of action, log-prob and value.  Leaves the
// actions in act[env][AW]; ends with the block in step (everything above complete).
template <int IN, int AW, int ACT, class ObsAt>
MRL_DEV void policy16_gauss(const CollectArgs &a, ObsAt obs_at, int tid, int ne, int A, int zero, size_t row,
                            uint32_t sseed, int env0, float *xs, float *tiles, const float *w2a, const float *w2c,
                            float *logits, float *vals, float *act, float *part) {
    constexpr int H = 256, R = PR16, T = 512, KBA = 8;
    const int wave = tid / WAVE, lane = tid % WAVE;
    const int net = wave >> 2;                           // 0: actor, 1: critic
    {
        const float *p = (net ? a.critic_p : a.actor_p) + zero;
        float *tile = tiles + net * (H * HT16_LD);
        Hidden16Operands<H, IN, 4, KBA> ops;
        ops.load(p, 64 * (wave & 3), lane);
        for (int i = tid; i < R * IN; i += T) {
            const int r = i / IN, c = i - r * IN;
            float v = 0.0f;
            if (r < ne) {
                v = obs_at(r, c);
                a.r_obs[row * IN + i] = v;
            }
            xs[r * XS_LD + c] = v;
        }
        __syncthreads();
        BlockSync bs;
        hidden_stack16<H, IN, ACT, 4, KBA, true>(p, xs, tile, tile, ops, 64 * (wave & 3), lane, bs);
        if (net == 0) head16<H>(w2a, A, tile, logits, PA_MAX + 1, tid, T / 2);
        else head_rows16<H, 1, 1>(w2c, 1, tile, vals, 1, tid - T / 2, T / 2);
        __syncthreads();   // means and values complete; the tiles are dead from here on
    }
    for (int e = tid; e < ne * A; e += T) {
        const int r = e / A, j = e - r * A;
        float av;
        part[r * PA_MAX + j] = sample_gaussian_part(logits + r * (PA_MAX + 1) + j, w2a + HEAD_LOG_STD(H) + j, 1, A, j,
                                                    sseed, env0 + r, &av);
        act[r * AW + j] = av;
        a.r_actions[row * AW + e] = av;
    }
    if (tid < ne) a.r_values[row + tid] = vals[tid];
    __syncthreads();
    if (tid < ne) {
        float logp = 0.0f;
        for (int j = 0; j < A; ++j) logp = logp + part[tid * PA_MAX + j];
        a.r_logp[row + tid] = logp;
    }
}

// The actor's half of policy16_gauss by wavefronts 0 .. 3 alone (the observation tile xs is complete, every
// thread of the four passes its tid): hidden stack on `tile`, Gaussian sampling, rollout row t of action and
// log-prob; leaves the actions in act[env][AW].  The four wavefronts meet at `sync`, five rounds per call.
template <int IN, int AW, int ACT>
MRL_DEV void actor16_gauss(const CollectArgs &a, int tid, int ne, int A, int zero, size_t row, uint32_t sseed, int env0,
                           const float *xs, float *tile, const float *w2a, float *logits, float *act, float *part,
                           WaveGroupSync &sync) {
    constexpr int H = 256, KBA = 8, TA = 4 * WAVE;
    const int wave = tid / WAVE, lane = tid % WAVE;
    const float *p = a.actor_p + zero;
    Hidden16Operands<H, IN, 4, KBA> ops;
    ops.load(p, 64 * wave, lane);
    hidden_stack16<H, IN, ACT, 4, KBA, true>(p, xs, tile, tile, ops, 64 * wave, lane, sync);
    head16<H>(w2a, A, tile, logits, PA_MAX + 1, tid, TA);
    sync();   // means complete
    for (int e = tid; e < ne * A; e += TA) {
        const int r = e / A, j = e - r * A;
        float av;
        part[r * PA_MAX + j] = sample_gaussian_part(logits + r * (PA_MAX + 1) + j, w2a + HEAD_LOG_STD(H) + j, 1, A, j,
                                                    sseed, env0 + r, &av);
        act[r * AW + j] = av;
        a.r_actions[row * AW + e] = av;
    }
    sync();   // actions and the log-probability terms complete
    if (tid < ne) {
        float logp = 0.0f;
        for (int j = 0; j < A; ++j) logp = logp + part[tid * PA_MAX + j];
        a.r_logp[row + tid] = logp;
    }
}
constexpr unsigned ACTOR16_ROUNDS = 5, CRITIC16_ROUNDS = 3;

// The critic's half by wavefronts 2, 3, 6 and 7 (the two SIMDs that do not host wavefronts 0 and 1), on a
// barrier of their own: values of the block's rows into vals.
template <int IN, int ACT>
MRL_DEV void critic16_side(const CollectArgs &a, int zero, int k, int tid, const float *xs, float *tile, const float *w2c,
                           float *vals, unsigned *sync_word, unsigned *failed) {
    constexpr int H = 256, KBA = 8;
    const int wave = tid / WAVE, lane = tid % WAVE;
    if (!(wave & 2)) return;
    const int g = (wave & 1) + ((wave >> 2) << 1);   // 0 .. 3
    const float *p = a.critic_p + zero;
    WaveGroupSync sync{sync_word, (unsigned)k * CRITIC16_ROUNDS * 4u, 4u, failed, a.spin_limit};
    Hidden16Operands<H, IN, 4, KBA> ops;
    ops.load(p, 64 * g, lane);
    hidden_stack16<H, IN, ACT, 4, KBA, true>(p, xs, tile, tile, ops, 64 * g, lane, sync);
    head_rows16<H, 1, 1>(w2c, 1, tile, vals, 1, g * WAVE + lane, 4 * WAVE);
}

template <class E, int ACT, bool LANES>
__global__ __launch_bounds__(512) void collect_walker_kernel(CollectArgs a) {
    using S = Stage<E>;
    constexpr int H = 256, IN = E::OBS, AW = E::ACT_W, R = PR16, T = 512, KBA = 8;
    static_assert(E::EPB == R && E::THREADS == T && IN <= PIN_MAX && AW <= PA_MAX, "16 envs per workgroup of eight wavefronts");
    __shared__ float rows[R * S::STRIDE];
    __shared__ float xs[R * XS_LD];
    __shared__ __align__(16) float w2a[HEAD_LDS(H)];
    __shared__ float w2c[H + 1];                    // the critic's head: column of H weights, then the bias
    __shared__ float logits[R * (PA_MAX + 1)];
    __shared__ float vals[R];
    __shared__ float act[R * PA_MAX];               // [env][AW]
    __shared__ float part[R * PA_MAX];              // log-probability per (env, component)
    __shared__ float shapes[E::NSHAPE];
    __shared__ unsigned long long was_reset;
    __shared__ unsigned sync_actor, sync_critic, sync_failed;   // barriers of the actor's and the critic's wavefronts
    // the two activation tiles and the env step's scratch (contact lists) are never live together
    constexpr int LIST_F = detect_list_floats<E>() + 1;
    constexpr int ENV_F = R * S::CSTRIDE + LIST_F + detect_count_ints<E>();
    __shared__ float overlay[wmax<2 * H * HT16_LD, ENV_F>()];
    static_assert(R * S::CSTRIDE <= H * HT16_LD, "the solver's contact scratch stays below the critic's tile");
    float *cts = overlay, *dlist = cts + R * S::CSTRIDE;
    int *dcount = reinterpret_cast<int *>(dlist + LIST_F);

    const int t = threadIdx.x;
    const int env0 = blockIdx.x * R;
    const int nenv = min(R, a.n_envs - env0);
    const int N = a.n_envs;
    float *gbase = a.states + (size_t)env0 * E::STATE;

    S::in(rows, gbase, nenv, t);
    for (int i = t; i < E::NSHAPE; i += T) shapes[i] = a.shapes[i];
    stage_head(a.actor_p + IN * H + H + H * H + H, H, a.A, true, w2a, t, T);
    for (int i = t; i < H + 1; i += T) w2c[i] = a.critic_p[IN * H + H + H * H + H + i];
    if (t == 0) {
        was_reset = 0;
        sync_actor = 0;
        sync_critic = 0;
        sync_failed = 0;
    }
    __syncthreads();

    for (int k = 0; k < a.n_steps; ++k) {
        // nothing but the rows is carried from one step to the next (see collect16_kernel)
        int tid = t, ne = __builtin_amdgcn_readfirstlane(nenv), A = __builtin_amdgcn_readfirstlane(a.A), zero = 0;
        asm volatile("" : "+v"(tid), "+s"(zero), "+s"(ne), "+s"(A) : : "memory");
        const size_t row = (size_t)(a.t0 + k) * N + env0;   // this block's slice of rollout row t
        const uint32_t sseed = a.sample_seed + (uint32_t)k * a.sample_stride;
        const uint64_t rseed = a.reset_seed + (uint64_t)k * a.reset_stride;
        const int wave = tid / WAVE, lane = tid % WAVE;
        // The env step keeps wavefronts 0 and 1 busy for most of the step (the solver with one lane per body)
        // and the others for little or nothing: only the actor goes ahead of it (wavefronts 0 .. 3, one per
        // SIMD); the critic, whose value is only stored, runs beside the solver on wavefronts 2, 3, 6 and 7 --
        // the two SIMDs that do not host wavefronts 0 and 1.  Both groups meet at bounded barriers of their
        // own, rebuilt every step from the step number.
        for (int i = tid; i < R * IN; i += T) {
            const int r = i / IN, c = i - r * IN;
            float v = 0.0f;
            if (r < ne) {
                v = rows[r * S::STRIDE + c];
                a.r_obs[row * IN + i] = v;
            }
            xs[r * XS_LD + c] = v;
        }
        __syncthreads();
        if (wave < 4) {
            WaveGroupSync actor_sync{&sync_actor, (unsigned)k * ACTOR16_ROUNDS * 4u, 4u, &sync_failed, a.spin_limit};
            actor16_gauss<IN, AW, ACT>(a, tid, ne, A, zero, row, sseed, env0, xs, overlay, w2a, logits, act, part, actor_sync);
        }
        float *critic_tile = overlay + H * HT16_LD;   // (above the env step's contact scratch cts)
        // ---- env step with auto-reset, reward / done into rollout row t, episode accounting
        Accounting acc = a.acc;
        acc.r_rewards = a.r_rewards + (size_t)(a.t0 + k) * N;
        acc.r_dones = a.r_dones + (size_t)(a.t0 + k) * N;
        acc = acc.at(env0);
        if constexpr (!LANES) {
            // (the critic's tile lies over contact lists that are spent by the time the solver runs)
            auto side = [&](int th) {
                critic16_side<IN, ACT>(a, zero, k, th, xs, critic_tile, w2c, vals, &sync_critic, &sync_failed);
            };
            phys_step_block<E, true>(rows, cts, shapes, dlist, dcount, &was_reset, act, nullptr, nullptr, env0, ne,
                                     rseed, acc, tid, side);
        } else {
            // HalfCheetah: eight lanes per env, eight envs per wavefront, on wavefronts 0 and 1; a row
            // whose wiring is not HalfCheetah's own is stepped by lane 0 of its group in the one-lane form
            if (wave < 2) {
                const int slot = wave * 8 + (lane >> 3), b = lane & 7;
                const bool live = slot < ne;
                float *rowp = rows + slot * S::STRIDE;
                const int env = env0 + (live ? slot : 0);
                const float *ap = act + (live ? slot : 0) * AW;
                const bool ok = live && hc::lanes_row_ok(rowp, shapes);
                float r = 0.0f, d = 0.0f;
                if (ok) hc::step_lanes(rowp, shapes, ap, lane, r, d);
                else if (live && b == 0) hc::step_row(rowp, cts + slot * S::CSTRIDE, shapes, env, ap, r, d);
                if (live && b == 0) {
                    account(acc, slot, r, d);
                    if (d > 0.5f) E::reset(rowp, rseed, env);
                }
            } else {
                critic16_side<IN, ACT>(a, zero, k, tid, xs, critic_tile, w2c, vals, &sync_critic, &sync_failed);
            }
        }
        __syncthreads();   // env step done: the rows hold the next observation
        if (tid < ne) a.r_values[row + tid] = vals[tid];
        // a wait that gave up: the block's results are void from here on; leave the loop and end normally
        if (sync_failed != 0u) break;
    }
    if (sync_failed != 0u) {
        // a wait gave up: the step in progress ran on data that was never produced; the block's rows and
        // observations are not stored and keep the values from before the launch
        if (t == 0) *a.sync_error = 1;
        return;
    }

    for (int i = t; i < nenv * E::OBS; i += T) {
        const int r = i / E::OBS, c = i - r * E::OBS;
        a.obs[(size_t)env0 * E::OBS + i] = rows[r * S::STRIDE + c];
    }
    S::out(rows, gbase, nenv, t, 0, E::STATE);
}

// CarRacingV2: the rows stay in global memory (12 KB each, nearly all of it the track); the block keeps the
// 40 floats in front of the track -- observation, hull, wheels, controls, metadata -- of its 16 envs in LDS
// over the whole launch.  Env step: a wavefront per env in two rounds of eight; each wavefront stages its
// env's tile table through LDS (over the activation tiles, which are dead by then), steps, accounts, and
// rebuilds the env when it finished (one lane walks the new track: only this block waits for it).
template <int ACT>
__global__ __launch_bounds__(512) void collect_car_kernel(CollectArgs a) {
    constexpr int H = 256, IN = cr::OBS, AW = cr::ACT, R = PR16, T = 512, HEAD = cr::TRACK;
    static_assert(IN <= PIN_MAX && AW <= PA_MAX && cr::TABLE % 4 == 0, "tile limits");
    __shared__ float heads[R * (HEAD + 1)];
    __shared__ float xs[R * XS_LD];
    __shared__ __align__(16) float w2a[HEAD_LDS(H)];
    __shared__ float w2c[H + 1];
    __shared__ float logits[R * (PA_MAX + 1)];
    __shared__ float vals[R];
    __shared__ float act[R * PA_MAX];
    __shared__ float part[R * PA_MAX];
    __shared__ __align__(16) float overlay[wmax<2 * H * HT16_LD, 8 * cr::TABLE>()];

    const int t = threadIdx.x;
    const int env0 = blockIdx.x * R;
    const int nenv = min(R, a.n_envs - env0);
    const int N = a.n_envs;
    for (int i = t; i < nenv * HEAD; i += T) {
        const int r = i / HEAD, c = i - r * HEAD;
        heads[r * (HEAD + 1) + c] = a.states[(size_t)(env0 + r) * cr::STATE + c];
    }
    stage_head(a.actor_p + IN * H + H + H * H + H, H, a.A, true, w2a, t, T);
    for (int i = t; i < H + 1; i += T) w2c[i] = a.critic_p[IN * H + H + H * H + H + i];
    __syncthreads();

    for (int k = 0; k < a.n_steps; ++k) {
        int tid = t, ne = __builtin_amdgcn_readfirstlane(nenv), A = __builtin_amdgcn_readfirstlane(a.A), zero = 0;
        asm volatile("" : "+v"(tid), "+s"(zero), "+s"(ne), "+s"(A) : : "memory");
        const size_t row = (size_t)(a.t0 + k) * N + env0;
        const uint32_t sseed = a.sample_seed + (uint32_t)k * a.sample_stride;
        const uint64_t rseed = a.reset_seed + (uint64_t)k * a.reset_stride;
        const int wave = tid / WAVE, sub = tid % WAVE;
        policy16_gauss<IN, AW, ACT>(a, [&](int r, int c) { return heads[r * (HEAD + 1) + c]; }, tid, ne, A, zero, row, sseed,
                                    env0, xs, overlay, w2a, w2c, logits, vals, act, part);
        Accounting acc = a.acc;
        acc.r_rewards = a.r_rewards + (size_t)(a.t0 + k) * N;
        acc.r_dones = a.r_dones + (size_t)(a.t0 + k) * N;
        acc = acc.at(env0);
        __syncthreads();   // the sampling's reads of the means are done before the tables go over the tiles
#pragma unroll 1
        for (int round = 0; round < 2; ++round) {
            const int slot = round * 8 + wave;
            if (slot < ne) {
                const int env = env0 + slot;
                float *head = heads + slot * (HEAD + 1);
                float *grow = a.states + (size_t)env * cr::STATE;
                float r, d, ob[cr::OBS];
                cr::step_wave<true>(head, grow, overlay + wave * cr::TABLE, act + slot * AW, sub, r, d, ob,
                                    a.car_trait_form != 0);
                if (sub == 0) account(acc, slot, r, d);
                if (d > 0.5f) {
                    float sx, sy, sa;
                    const int nt = cr::reset_group<cr::STEP_LANES>(grow, cr::combined_seed(rseed, env), sub, sx, sy, sa);
                    if (sub < HEAD) {
                        float v = 0.0f;
                        if (sub == 0 || sub == cr::HULL + cr::H_X) v = sx;
                        else if (sub == 1 || sub == cr::HULL + cr::H_Y) v = sy;
                        else if (sub == 2 || sub == cr::HULL + cr::H_ANGLE) v = sa;
                        else if (sub == cr::META + cr::M_NUM_TILES) v = (float)nt;
                        head[sub] = v;
                    }
                    // the new track is read back by this wavefront at its next step: nothing older may
                    // linger in the vector cache
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
                }
            }
        }
        __syncthreads();   // env step done: the heads hold the next observation
    }

    for (int i = t; i < nenv * HEAD; i += T) {
        const int r = i / HEAD, c = i - r * HEAD;
        a.states[(size_t)(env0 + r) * cr::STATE + c] = heads[r * (HEAD + 1) + c];
    }
    for (int i = t; i < nenv * IN; i += T) {
        const int r = i / IN, c = i - r * IN;
        a.obs[(size_t)env0 * IN + i] = heads[r * (HEAD + 1) + c];
    }
}

// HopperPlanar / Walker2dPlanar (env_planar.hpp): the rows (248 / 392 bytes, Float64 state behind the fp32
// observation) stay in LDS over the whole launch; the actor runs on wavefronts 0 .. 3, then lanes 0 .. 15 of
// wavefront 0 step one env each (Float64, state in registers for the four sub-steps), account and rebuild
// finished rows in place, while the critic runs beside them on wavefronts 2, 3, 6 and 7.
template <class M, int ACT>
__global__ __launch_bounds__(512) void collect_planar_kernel(CollectArgs a) {
    constexpr int H = 256, IN = M::OBS, AW = M::ACT, R = PR16, T = 512;
    static_assert(IN <= PIN_MAX && AW <= PA_MAX && M::STATE % 2 == 0, "tile limits; rows are whole doubles");
    __shared__ __align__(16) float rows[R * M::STATE];
    __shared__ float xs[R * XS_LD];
    __shared__ __align__(16) float w2a[HEAD_LDS(H)];
    __shared__ float w2c[H + 1];
    __shared__ float logits[R * (PA_MAX + 1)];
    __shared__ float vals[R];
    __shared__ float act[R * PA_MAX];
    __shared__ float part[R * PA_MAX];
    __shared__ unsigned sync_actor, sync_critic, sync_failed;
    __shared__ __align__(16) float tiles[2 * H * HT16_LD];

    const int t = threadIdx.x;
    const int env0 = blockIdx.x * R;
    const int nenv = min(R, a.n_envs - env0);
    const int N = a.n_envs;
    float2 *g2 = reinterpret_cast<float2 *>(a.states + (size_t)env0 * M::STATE);
    float2 *l2 = reinterpret_cast<float2 *>(rows);
    for (int i = t; i < nenv * (M::STATE / 2); i += T) l2[i] = g2[i];
    stage_head(a.actor_p + IN * H + H + H * H + H, H, a.A, true, w2a, t, T);
    for (int i = t; i < H + 1; i += T) w2c[i] = a.critic_p[IN * H + H + H * H + H + i];
    if (t == 0) {
        sync_actor = 0;
        sync_critic = 0;
        sync_failed = 0;
    }
    __syncthreads();

    for (int k = 0; k < a.n_steps; ++k) {
        // nothing but the rows is carried from one step to the next (see collect16_kernel)
        int tid = t, ne = __builtin_amdgcn_readfirstlane(nenv), A = __builtin_amdgcn_readfirstlane(a.A), zero = 0;
        asm volatile("" : "+v"(tid), "+s"(zero), "+s"(ne), "+s"(A) : : "memory");
        const size_t row = (size_t)(a.t0 + k) * N + env0;
        const uint32_t sseed = a.sample_seed + (uint32_t)k * a.sample_stride;
        const uint64_t rseed = a.reset_seed + (uint64_t)k * a.reset_stride;
        const int wave = tid / WAVE, lane = tid % WAVE;
        for (int i = tid; i < R * IN; i += T) {
            const int r = i / IN, c = i - r * IN;
            float v = 0.0f;
            if (r < ne) {
                v = rows[r * M::STATE + c];
                a.r_obs[row * IN + i] = v;
            }
            xs[r * XS_LD + c] = v;
        }
        __syncthreads();
        if (wave < 4) {
            WaveGroupSync actor_sync{&sync_actor, (unsigned)k * ACTOR16_ROUNDS * 4u, 4u, &sync_failed, a.spin_limit};
            actor16_gauss<IN, AW, ACT>(a, tid, ne, A, zero, row, sseed, env0, xs, tiles, w2a, logits, act, part, actor_sync);
        }
        if (wave == 0) {
            if (lane < ne) {
                Accounting acc = a.acc;
                acc.r_rewards = a.r_rewards + (size_t)(a.t0 + k) * N;
                acc.r_dones = a.r_dones + (size_t)(a.t0 + k) * N;
                acc = acc.at(env0);
                float *rowp = rows + lane * M::STATE;
                planar::State<M> s;
                s.load(rowp);
                float r, d;
                planar::step<M>(s, act + lane * AW, r, d);
                account(acc, lane, r, d);
                if (d > 0.5f) planar::reset<M>(s, planar::combined_seed(rseed, env0 + lane));
                s.store(rowp);
            }
        } else {
            critic16_side<IN, ACT>(a, zero, k, tid, xs, tiles + H * HT16_LD, w2c, vals, &sync_critic, &sync_failed);
        }
        __syncthreads();   // env step done: the rows hold the next observation
        if (tid < ne) a.r_values[row + tid] = vals[tid];
        if (sync_failed != 0u) break;
    }
    if (sync_failed != 0u) {
        // a wait gave up: the block's rows and observations keep the values from before the launch
        if (t == 0) *a.sync_error = 1;
        return;
    }
    for (int i = t; i < nenv * IN; i += T) {
        const int r = i / IN, c = i - r * IN;
        a.obs[(size_t)env0 * IN + i] = rows[r * M::STATE + c];
    }
    for (int i = t; i < nenv * (M::STATE / 2); i += T) g2[i] = l2[i];
}

bool collect_walker_fusable(const mrl_rollout *r, int *act) {
    if (r->num_actions != 0) return false;
    int obs, aw;
    if (r->env_id == MRL_ENV_BIPEDAL) { obs = BipedalWalker::OBS; aw = BipedalWalker::ACT_W; }
    else if (r->env_id == MRL_ENV_HALFCHEETAH) { obs = HalfCheetah::OBS; aw = HalfCheetah::ACT_W; }
    else if (r->env_id == MRL_ENV_CARRACING) { obs = cr::OBS; aw = cr::ACT; }
    else if (r->env_id == MRL_ENV_HOPPER_PLANAR) { obs = planar::Hopper::OBS; aw = planar::Hopper::ACT; }
    else if (r->env_id == MRL_ENV_WALKER2D_PLANAR) { obs = planar::Walker2d::OBS; aw = planar::Walker2d::ACT; }
    else return false;
    // (the planar rows hold doubles)
    if (r->env_id >= MRL_ENV_HOPPER_PLANAR && reinterpret_cast<uintptr_t>(r->states) % 8 != 0) return false;
    const mrl_mlp_desc &a = r->actor, &c = r->critic;
    if (a.n_layers != 3 || c.n_layers != 3) return false;
    const int k0 = a.layers[0].kind;
    if (k0 != MRL_LINEAR_RELU && k0 != MRL_LINEAR_TANH) return false;
    for (const mrl_mlp_desc *d : {&a, &c}) {
        if (d->layers[0].kind != k0 || d->layers[1].kind != k0) return false;
        if (d->layers[0].in_dim != obs || d->layers[0].out_dim != 256 || d->layers[1].out_dim != 256) return false;
    }
    if (a.layers[2].kind != MRL_STOCHASTIC_ACTOR || a.layers[2].out_dim != aw) return false;
    if (c.layers[2].kind != MRL_LINEAR || c.layers[2].out_dim != 1) return false;
    // 16-byte loads of the weight rows
    if (reinterpret_cast<uintptr_t>(r->actor_params) % 16 != 0 || reinterpret_cast<uintptr_t>(r->critic_params) % 16 != 0)
        return false;
    *act = (k0 == MRL_LINEAR_RELU) ? 1 : 2;
    return true;
}

int launch_collect_walker(mrl_ctx *ctx, const mrl_rollout *r, const CollectArgs &args, int act) {
    CollectArgs a = args;
    const dim3 grid(grid_for(r->n_envs, PR16)), block(512);
    if (r->env_id == MRL_ENV_BIPEDAL) {
        a.shapes = ctx->bw_shapes;
        if (act == 1) hipLaunchKernelGGL((collect_walker_kernel<BipedalWalker, 1, false>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((collect_walker_kernel<BipedalWalker, 2, false>), grid, block, 0, ctx->stream, a);
    } else if (r->env_id == MRL_ENV_CARRACING) {
        if (act == 1) hipLaunchKernelGGL((collect_car_kernel<1>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((collect_car_kernel<2>), grid, block, 0, ctx->stream, a);
    } else if (r->env_id == MRL_ENV_HOPPER_PLANAR) {
        if (act == 1) hipLaunchKernelGGL((collect_planar_kernel<planar::Hopper, 1>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((collect_planar_kernel<planar::Hopper, 2>), grid, block, 0, ctx->stream, a);
    } else if (r->env_id == MRL_ENV_WALKER2D_PLANAR) {
        if (act == 1) hipLaunchKernelGGL((collect_planar_kernel<planar::Walker2d, 1>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((collect_planar_kernel<planar::Walker2d, 2>), grid, block, 0, ctx->stream, a);
    } else {
        a.shapes = ctx->hc_shapes;
        if (act == 1) hipLaunchKernelGGL((collect_walker_kernel<HalfCheetah16, 1, true>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((collect_walker_kernel<HalfCheetah16, 2, true>), grid, block, 0, ctx->stream, a);
    }
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

}  // namespace mrl
