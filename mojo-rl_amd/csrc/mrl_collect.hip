// Fused collection kernel: many rollout steps of a block's envs in ONE launch.
//
// Envs do not interact and the policy does not change during a rollout, so a workgroup can take
// its 32 envs through any number of steps on its own: the env rows stay in LDS from the first step
// to the last (HBM sees them once in and once out per launch, however many steps), the
// observation tile feeds the policy straight from those rows, and the sampled actions reach the
// env step through LDS.  Per step and block:
//   actor    OBS -> H -> H -> A on the fp32 matrix cores by all eight wavefronts (the 32 x H tiles
//            of mlp_tile.hpp, weights streamed from L2);
//   then, side by side,
//     wavefront 0        categorical / Gaussian sampling, then the env step of env_block.hpp (one
//                        env per lane), reward / done of rollout row t, episode accounting,
//                        in-place reset;
//     wavefronts 1 .. 7  contact detection for that env step;
//     all of these but   then the critic  OBS -> H -> H -> 1  (its value is only stored, so it does
//     wavefront 4        not hold up the env step; the six wavefronts meet at a barrier of their own,
//                        and wavefront 4, which shares wavefront 0's SIMD, stays out of its way);
//   rollout row t of obs, action, log-prob and value written on the way.
// No workgroup waits for another, so there is nothing between two steps but the block's own
// barriers; the launch ends when every block has done its n_steps.
//
// It gives what n_steps calls of mrl_rollout_step give (same per-env streams: seeds are affine
// in the step number), except that the finished-episode list is appended in the order in which
// blocks get there rather than step by step.
#include "mrl_host.hpp"
#include "mrl_device.hpp"
#include "mlp_tile.hpp"
#include "mlp_tile16.hpp"
#include "policy_sample.hpp"
#include "env_block.hpp"
#include "env_classic.hpp"
#include "collect_args.hpp"

namespace mrl {


template <int A, int B>
constexpr int cmax() { return A > B ? A : B; }

template <class E, int H, int ACT, bool GAUSS>
__global__ __launch_bounds__(E::THREADS) void collect_kernel(CollectArgs a) {
    using S = Stage<E>;
    constexpr int IN = E::OBS, AW = E::ACT_W, NW = E::THREADS / WAVE;
    // the critic runs on the six wavefronts that do not share a SIMD with wavefront 0 (1, 2, 3, 5, 6,
    // 7: two per SIMD, so that one's MFMAs cover the other's loads and epilogues; wavefront 0's solver
    // keeps its SIMD's issue slots to itself); its eight column tiles are dealt out 3 / 3 / 2 per SIMD
    constexpr int CRITIC_TPW = 2, CRITIC_WAVES = 6, CRITIC_T = CRITIC_WAVES * WAVE;
    static_assert(E::EPB == PR && E::THREADS == 2 * H && NW == 8 && H == 256, "one 32-row policy tile per block");
    static_assert(IN <= PIN_MAX && AW <= PA_MAX && E::DETECT_TASKS > 0, "policy tile limits; split-off detection");
    __shared__ float rows[PR * S::STRIDE];
    __shared__ float xs[PR * XS_LD];
    __shared__ __align__(16) float w2s[2][HEAD_LDS(H)];
    __shared__ float logits[PR * (PA_MAX + 1)];
    __shared__ float vals[PR];
    __shared__ float act[PR * PA_MAX];
    __shared__ float shapes[E::NSHAPE];
    __shared__ unsigned long long was_reset;
    __shared__ unsigned sync_critic, sync_detect, sync_failed;
    __shared__ int ncontacts[PR];   // an env's contact count after the merge of its lists (-1: detect again)
    __shared__ float hTc[H * HT_LD];   // the critic's activation tile (live during the env step)
    // the actor's activation tile and the env step's contact scratch are never live together
    constexpr int LIST_F = detect_list_floats<E>() + 1;
    constexpr int ENV_F = PR * S::CSTRIDE + LIST_F + detect_count_ints<E>();
    __shared__ float overlay[cmax<H * HT_LD, ENV_F>()];
    float *cts = overlay, *dlist = cts + PR * S::CSTRIDE;
    int *dcount = reinterpret_cast<int *>(dlist + LIST_F);

    const int t = threadIdx.x;
    const int env0 = blockIdx.x * PR;
    const int nenv = min(PR, a.n_envs - env0);
    const int N = a.n_envs;
    float *gbase = a.states + (size_t)env0 * E::STATE;

    S::in(rows, gbase, nenv, t);
    for (int i = t; i < E::NSHAPE; i += E::THREADS) shapes[i] = a.shapes[i];
    {
        const int net = t / H;
        const float *p = net ? a.critic_p : a.actor_p;
        stage_head(p + IN * H + H + H * H + H, H, net ? 1 : a.A, GAUSS && net == 0, w2s[net], t % H, H);
    }
    if (t == 0) {
        was_reset = 0;
        sync_critic = 0;
        sync_detect = 0;
        sync_failed = 0;
    }
    if (t < PR) ncontacts[t] = 0;   // read by the solver also when the detection's wait gave up
    __syncthreads();
    // wavefront 0, lane = env slot: the env's running episode return and length stay in registers
    const bool owner = t < nenv;
    float ep_return = owner ? a.acc.ep_return[env0 + t] : 0.0f;
    float ep_length = owner ? a.acc.ep_length[env0 + t] : 0.0f;
    static_assert((E::DETECT_TASKS + 1) / 2 <= NW - 1, "two detection tasks per wavefront besides wavefront 0");

    // Per step: every wavefront runs the actor (the action is what the env step waits for); then
    // wavefront 0 samples and steps the envs, wavefronts 1 .. 7 detect their contacts, and all of
    // these but wavefront 4 go on to run the critic, whose value is only stored -- off the critical path.
    for (int k = 0; k < a.n_steps; ++k) {
        // Nothing but the rows is carried from one step to the next: the thread index, the block's
        // env count and the parameter pointers pass through empty asm statements at the top of each
        // step, so the optimiser cannot keep what it derives from them (addresses, predicates, the
        // step-invariant operand values) live through the env step, whose solver needs the registers.
        int tid = t, ne = __builtin_amdgcn_readfirstlane(nenv), A = __builtin_amdgcn_readfirstlane(a.A), zero = 0;
        asm volatile("" : "+v"(tid), "+s"(zero), "+s"(ne), "+s"(A) : : "memory");
        const float *pa = a.actor_p + zero, *pc = a.critic_p + zero;
        const size_t row = (size_t)(a.t0 + k) * N + env0;   // this block's slice of rollout row t
        const uint32_t sseed = a.sample_seed + (uint32_t)k * a.sample_stride;
        const int wave = tid / WAVE, lane = tid % WAVE;
        // the barriers of the wavefront groups, rebuilt every step from the step number (the critic's
        // hidden stack meets three times per step, the detection once), so that nothing of them is
        // carried through the env step in registers
        WaveGroupSync critic_sync{&sync_critic, (unsigned)k * 3u * CRITIC_WAVES, (unsigned)CRITIC_WAVES, &sync_failed, a.spin_limit};
        WaveGroupSync detect_sync{&sync_detect, (unsigned)k * 2u * (NW - 1), (unsigned)(NW - 1), &sync_failed, a.spin_limit};
        // ---- actor, all wavefronts
        {
            HiddenOperands<H, 1, 32> ops;
            ops.load(pa, IN, tid);
            for (int i = tid; i < PR * IN; i += E::THREADS) {
                const int r = i / IN, c = i - r * IN;
                float v = 0.0f;
                if (r < ne) {
                    v = rows[r * S::STRIDE + c];
                    a.r_obs[row * IN + i] = v;
                }
                xs[r * XS_LD + c] = v;
            }
            __syncthreads();
            hidden_stack<H, ACT, 1, 32, true>(pa, IN, xs, overlay, overlay, TileCache{}, ops, tid);
            head<H>(w2s[0], A, overlay, logits, PA_MAX + 1, tid, E::THREADS);
            __syncthreads();   // logits complete; the actor's tile is dead from here on
        }
        if (wave == 0) {
            // ---- sample, then the env step of env_block.hpp with the contacts of wavefronts 1 .. 3
            typename E::Carry carry{};
            if (lane < ne) {
                const int i = env0 + lane;
                float logp;
                if (GAUSS) {
                    float av[PA_MAX];
                    logp = sample_gaussian(logits + lane * (PA_MAX + 1), w2s[0] + HEAD_LOG_STD(H), A, sseed, i, av);
                    for (int j = 0; j < A; ++j) {
                        act[lane * AW + j] = av[j];
                        a.r_actions[(row + lane) * AW + j] = av[j];
                    }
                } else {
                    int sel;
                    sample_categorical_few(logits + lane * (PA_MAX + 1), A, sseed, i, sel, logp);
                    act[lane] = (float)sel;
                    a.r_actions[row + lane] = (float)sel;
                }
                a.r_logp[row + lane] = logp;
                carry = E::step_begin(rows + lane * S::STRIDE, i, act + lane * AW, shapes);
            }
            // (the detecting wavefronts meet twice: lists complete, then every list moved to its place in its env's list)
            detect_sync.target += 2 * detect_sync.nwaves;
            detect_sync.wait_for(detect_sync.target);
            bool finished = false;
            int slot = 0;
            float fin_return = 0.0f, fin_length = 0.0f;
            if (lane < ne) {
                float *mine = cts + lane * S::CSTRIDE;
                const int n = ncontacts[lane];
                float r, d;
                E::step_finish(rows + lane * S::STRIDE, mine, n, shapes, carry, r, d);
                // rollout row t and the episode accounting of account(), on the running sums that
                // this lane carries for its env
                a.r_rewards[row + lane] = r;
                a.r_dones[row + lane] = d;
                ep_return = ep_return + r;
                ep_length = ep_length + 1.0f;
                finished = d > 0.5f;
                if (finished) {
                    // the slot in the finished-episode list comes back from L2 while the row is rebuilt
                    slot = atomicAdd(a.acc.done_count, 1);
                    fin_return = ep_return;
                    fin_length = ep_length;
                    ep_return = 0.0f;
                    ep_length = 0.0f;
                }
            }
            reset_rows<E>(rows, &was_reset, __ballot(finished), a.reset_seed + (uint64_t)k * a.reset_stride, env0, lane);
            if (finished && slot < a.acc.done_cap) {
                a.acc.done_returns[slot] = fin_return;
                a.acc.done_lengths[slot] = fin_length;
            }
        } else {
            // ---- contact detection: one (body, vertex) task per half of wavefronts 1 .. 7
            const int task = (wave - 1) * 2 + lane / (WAVE / 2), e = lane % (WAVE / 2);
            if (task < E::DETECT_TASKS && e < ne) detect_vertex_task<E>(rows, shapes, dlist, dcount, task, e);
            // the lists are merged by the lanes that made them, all at once, instead of one after the other by
            // the solver's wavefront: once every list of the block is in, each lane moves its own
            detect_sync();
            if (task < E::DETECT_TASKS && e < ne) {
                const int n = merge_vertex_list_of_task<E>(dlist, dcount, e, task, cts + e * S::CSTRIDE);
                if (task == 0) ncontacts[e] = n;
            }
            detect_sync.arrive();
            if (wave != 4) {
                // ---- critic, on its own barrier: member g = 0 .. 5 of the group is wavefront g + 1
                // (g < 3) or g + 2; members g and g + 3 share a SIMD and take tiles {2, 1}, {2, 1}, {1, 1}
                const int g = wave < 4 ? wave - 1 : wave - 2;
                const int tl = g * WAVE + lane;   // index among the critic's threads
                const int tile0 = g < 2 ? 2 * g : g + 2, tiles = g < 2 ? 2 : 1;
                HiddenOperands<H, CRITIC_TPW, 16> ops;
                ops.load(pc, IN, tl, tile0, tiles);
                hidden_stack<H, ACT, CRITIC_TPW, 16, true>(pc, IN, xs, hTc, hTc, TileCache{}, ops, tl, critic_sync);
                head<H>(w2s[1], 1, hTc, vals, 1, tl, CRITIC_T);
            }
        }
        __syncthreads();   // env step done, values complete
        if (tid < ne) a.r_values[row + tid] = vals[tid];
        // a wait that gave up: the block's results are void from here on; leave the loop (every
        // thread reads the same word after the barrier) and end normally
        if (sync_failed != 0u) break;
    }
    if (sync_failed != 0u) {
        // a wait gave up: the step in progress ran on data that was never produced.  Nothing of it is
        // stored: rows, observations and episode sums of this block keep the values from before the launch
        if (t == 0) *a.sync_error = 1;
        return;
    }

    if (owner) {
        a.acc.ep_return[env0 + t] = ep_return;
        a.acc.ep_length[env0 + t] = ep_length;
    }
    for (int i = t; i < nenv * E::OBS; i += E::THREADS) {
        const int r = i / E::OBS, c = i - r * E::OBS;
        a.obs[(size_t)env0 * E::OBS + i] = rows[r * S::STRIDE + c];
    }
    S::out(rows, gbase, nenv, t, 0, E::STATE);
}

// ---------------------------------------------------------------- 16 rows per workgroup
// The same step for a workgroup of four wavefronts and 16 envs, for launches with at most 16 envs
// per CU.  A step is a chain -- actor on the matrix cores, then sampling and the env step on ONE
// wavefront's vector unit -- and the env step costs the same whether 16 or 32 lanes carry an env,
// while the actor of 16 rows takes half the matrix time of 32 (v_mfma_f32_16x16x4_f32, same bits as
// the 32-row tiles): few envs are stepped faster spread 16 to a CU than packed 32 to half the CUs.
//   all four wavefronts     actor  OBS -> H -> H -> A, 64 columns each;
//   the solver wavefront    sampling, env step (one env per lane 0 .. 15), accounting, resets;
//   the other three         contact detection, then the critic (80 / 96 / 80 columns) at a barrier
//                           of their own.
// Two such workgroups fit a CU (LDS, registers), but running them side by side does not pay: on this
// hardware a SIMD issues either a matrix or a vector instruction, never both at once (a wavefront of
// dependent v_fma_f32 that shares its SIMD with a wavefront issuing v_mfma back to back takes the sum
// of both times), so one workgroup's env step does not hide behind the other's forward passes, and
// two solver wavefronts of 16 envs cost twice the vector time of one with 32.  With more than 16 envs
// per CU the 32-row kernel above is the faster one (8192 envs: 38.6 against 39.8 us per step).
// The solver wavefront is 0 in the lower half of the grid and 2 in the upper half: workgroups i and
// i + grid / 2 share a CU when the grid is twice the CU count, and their solvers then sit on
// different SIMDs.
template <class EB, int ACT, bool GAUSS>
__global__ __launch_bounds__(256, 2) void collect16_kernel(CollectArgs a) {
    using E = Rows16<EB>;
    using S = Stage<E>;
    constexpr int H = 256, IN = E::OBS, AW = E::ACT_W, R = PR16, T = E::THREADS;
    constexpr int CAP = 3;      // records per (body, vertex) list: two contacts, the third signals overflow
    constexpr int KBA = 8;      // k-steps of layer-1 weights fetched ahead
    static_assert(IN <= PIN_MAX && AW <= PA_MAX && E::DETECT_TASKS > 0 && E::DETECT_TASKS <= 24, "tile limits; split-off detection");
    __shared__ float rows[R * S::STRIDE];
    __shared__ float xs[R * XS_LD];
    __shared__ __align__(16) float w2a[HEAD_LDS(H)];
    __shared__ float w2c[H + 1];                    // the critic's head: column of H weights, then the bias
    __shared__ float logits[R * (PA_MAX + 1)];
    __shared__ float vals[R];
    __shared__ float act[R * PA_MAX];
    __shared__ float shapes[E::NSHAPE];
    __shared__ unsigned long long was_reset;
    __shared__ unsigned sync_critic, sync_detect, sync_failed;
    __shared__ float hTc[H * HT16_LD];              // the critic's activation tile (live during the env step)
    // the actor's activation tile and the env step's contact scratch are never live together
    constexpr int LIST_F = detect_list_floats<E, CAP>() + 1;
    constexpr int ENV_F = R * S::CSTRIDE + LIST_F + detect_count_ints<E>();
    __shared__ float overlay[cmax<H * HT16_LD, ENV_F>()];
    float *cts = overlay, *dlist = cts + R * S::CSTRIDE;
    int *dcount = reinterpret_cast<int *>(dlist + LIST_F);

    const int t = threadIdx.x;
    const int env0 = blockIdx.x * R;
    const int nenv = min(R, a.n_envs - env0);
    const int N = a.n_envs;
    const int sw = (2 * blockIdx.x >= gridDim.x && gridDim.x > 1) ? 2 : 0;   // the solver wavefront
    float *gbase = a.states + (size_t)env0 * E::STATE;

    S::in(rows, gbase, nenv, t);
    for (int i = t; i < E::NSHAPE; i += T) shapes[i] = a.shapes[i];
    stage_head(a.actor_p + IN * H + H + H * H + H, H, a.A, GAUSS, w2a, t, T);
    for (int i = t; i < H + 1; i += T) w2c[i] = a.critic_p[IN * H + H + H * H + H + i];
    if (t == 0) {
        was_reset = 0;
        sync_critic = 0;
        sync_detect = 0;
        sync_failed = 0;
    }
    __syncthreads();
    // solver wavefront, lane = env slot: the env's running episode return and length stay in registers
    const bool owner = (t >> 6) == sw && (t & 63) < nenv;
    float ep_return = owner ? a.acc.ep_return[env0 + (t & 63)] : 0.0f;
    float ep_length = owner ? a.acc.ep_length[env0 + (t & 63)] : 0.0f;

    for (int k = 0; k < a.n_steps; ++k) {
        // Nothing but the rows is carried from one step to the next: the thread index, the block's
        // env count and the parameter pointers pass through empty asm statements at the top of each
        // step, so the optimiser cannot keep what it derives from them live through the env step,
        // whose solver needs the registers.
        int tid = t, ne = __builtin_amdgcn_readfirstlane(nenv), A = __builtin_amdgcn_readfirstlane(a.A), zero = 0;
        asm volatile("" : "+v"(tid), "+s"(zero), "+s"(ne), "+s"(A) : : "memory");
        const float *pa = a.actor_p + zero, *pc = a.critic_p + zero;
        const size_t row = (size_t)(a.t0 + k) * N + env0;   // this block's slice of rollout row t
        const uint32_t sseed = a.sample_seed + (uint32_t)k * a.sample_stride;
        const int wave = tid / WAVE, lane = tid % WAVE;
        const int vw = (wave - sw) & 3;                     // 0: solver, 1 .. 3: helpers
        // the helpers' barriers, rebuilt every step from the step number (the critic's hidden stack meets
        // three times per step, the detection once): nothing of them stays in registers through the env step
        WaveGroupSync critic_sync{&sync_critic, (unsigned)k * 9u, 3u, &sync_failed, a.spin_limit};
        WaveGroupSync detect_sync{&sync_detect, (unsigned)k * 3u, 3u, &sync_failed, a.spin_limit};
        // ---- actor, all wavefronts
        {
            Hidden16Operands<H, IN, 4, KBA> ops;
            ops.load(pa, 64 * wave, lane);
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
            BlockSync bs;
            hidden_stack16<H, IN, ACT, 4, KBA, true>(pa, xs, overlay, overlay, ops, 64 * wave, lane, bs);
            head16<H>(w2a, A, overlay, logits, PA_MAX + 1, tid, T);
            __syncthreads();   // logits complete; the actor's tile is dead from here on
        }
        if (vw == 0) {
            // ---- sample, then the env step of env_block.hpp with the contacts the helpers detect
            typename E::Carry carry{};
            if (lane < ne) {
                const int i = env0 + lane;
                float logp;
                if (GAUSS) {
                    float av[PA_MAX];
                    logp = sample_gaussian(logits + lane * (PA_MAX + 1), w2a + HEAD_LOG_STD(H), A, sseed, i, av);
                    for (int j = 0; j < A; ++j) {
                        act[lane * AW + j] = av[j];
                        a.r_actions[(row + lane) * AW + j] = av[j];
                    }
                } else {
                    int sel;
                    sample_categorical_few(logits + lane * (PA_MAX + 1), A, sseed, i, sel, logp);
                    act[lane] = (float)sel;
                    a.r_actions[row + lane] = (float)sel;
                }
                a.r_logp[row + lane] = logp;
                carry = E::step_begin(rows + lane * S::STRIDE, i, act + lane * AW, shapes);
            }
            detect_sync.target += detect_sync.nwaves;
            detect_sync.wait_for(detect_sync.target);
            bool finished = false;
            if (lane < ne) {
                float *mine = cts + lane * S::CSTRIDE;
                const int n = merge_vertex_lists<E, CAP>(dlist, dcount, lane, mine);
                float r, d;
                E::step_finish(rows + lane * S::STRIDE, mine, n, shapes, carry, r, d);
                a.r_rewards[row + lane] = r;
                a.r_dones[row + lane] = d;
                ep_return = ep_return + r;
                ep_length = ep_length + 1.0f;
                finished = d > 0.5f;
                if (finished) {
                    const int slot = atomicAdd(a.acc.done_count, 1);
                    if (slot < a.acc.done_cap) {
                        a.acc.done_returns[slot] = ep_return;
                        a.acc.done_lengths[slot] = ep_length;
                    }
                    ep_return = 0.0f;
                    ep_length = 0.0f;
                }
            }
            reset_rows<E>(rows, &was_reset, __ballot(finished), a.reset_seed + (uint64_t)k * a.reset_stride, env0, lane);
        } else {
            // ---- contact detection: (body, vertex) task m * 4 + lane / 16 of env slot lane % 16, a
            // second pass on helper 0 for the tasks beyond twelve
            const int m = vw - 1, e = lane % R;
            if (e < ne)
                for (int task = m * 4 + lane / R; task < E::DETECT_TASKS; task += 12)
                    detect_vertex_task<E, CAP>(rows, shapes, dlist, dcount, task, e);
            detect_sync.arrive();
            // ---- critic on the three helpers, at their own barrier: helper 1 takes six column
            // tiles, helpers 0 (which had the second detection pass) and 2 five each
            const int tl = m * WAVE + lane;
            if (m == 1) {
                Hidden16Operands<H, IN, 6, KBA> ops;
                ops.load(pc, 80, lane);
                hidden_stack16<H, IN, ACT, 6, KBA, true>(pc, xs, hTc, hTc, ops, 80, lane, critic_sync);
            } else {
                const int c0 = m == 0 ? 0 : 176;
                Hidden16Operands<H, IN, 5, KBA> ops;
                ops.load(pc, c0, lane);
                hidden_stack16<H, IN, ACT, 5, KBA, true>(pc, xs, hTc, hTc, ops, c0, lane, critic_sync);
            }
            head_rows16<H, 1, 1>(w2c, 1, hTc, vals, 1, tl, 3 * WAVE);
        }
        __syncthreads();   // env step done, values complete
        if (tid < ne) a.r_values[row + tid] = vals[tid];
        // a wait that gave up: the block's results are void from here on; leave the loop (every
        // thread reads the same word after the barrier) and end normally
        if (sync_failed != 0u) break;
    }
    if (sync_failed != 0u) {   // as in collect_kernel: nothing of a block whose wait gave up is stored
        if (t == 0) *a.sync_error = 1;
        return;
    }

    if (owner) {
        a.acc.ep_return[env0 + (t & 63)] = ep_return;
        a.acc.ep_length[env0 + (t & 63)] = ep_length;
    }
    for (int i = t; i < nenv * E::OBS; i += T) {
        const int r = i / E::OBS, c = i - r * E::OBS;
        a.obs[(size_t)env0 * E::OBS + i] = rows[r * S::STRIDE + c];
    }
    S::out(rows, gbase, nenv, t, 0, E::STATE);
}

// ---------------------------------------------------------------- CartPole / Pendulum
// The same idea for the envs whose state is a handful of floats: a workgroup of four wavefronts
// (two on the actor, two on the critic, hidden width 64, one 32-column tile each) takes its 32
// envs through all the steps of the launch.  Each wavefront's share of the hidden layers' weights
// is loaded into registers once, before the first step; lanes 0 .. 31 of wavefront 0 carry one
// env each in registers -- state, step counter, episode sums -- and do sampling, step,
// accounting and reset in place.  A step is one dependent chain (observation -> two layers on
// the matrix cores -> head -> sample -> env step), so the time of a step does not depend on the
// number of envs until there are more workgroups than the chip holds at once.
struct CartPoleSlot {
    static constexpr int OBS = cartpole::OBS, ACT_W = 1;
    float s[4];
    int32_t steps;
    MRL_DEV void load(const float *states, const int32_t *side, int i) {
        const float4 v = reinterpret_cast<const float4 *>(states)[i];
        s[0] = v.x; s[1] = v.y; s[2] = v.z; s[3] = v.w;
        steps = side[i];
    }
    MRL_DEV void store(float *states, int32_t *side, int i) const {
        reinterpret_cast<float4 *>(states)[i] = make_float4(s[0], s[1], s[2], s[3]);
        side[i] = steps;
    }
    MRL_DEV float obs(int k) const { return s[k]; }
    MRL_DEV void step(const float *act, float &r, float &d) { cartpole::step(s, steps, (int)act[0], r, d); }
    MRL_DEV void reset(int i, uint64_t seed) { cartpole::reset(s, steps, i, (uint32_t)seed); }
};
struct PendulumSlot {
    static constexpr int OBS = pendulum::OBS, ACT_W = 1;
    float s[8];
    MRL_DEV void load(const float *states, const int32_t *, int i) {
        const float4 *row = reinterpret_cast<const float4 *>(states) + 2 * (size_t)i;
        const float4 a = row[0], b = row[1];
        s[0] = a.x; s[1] = a.y; s[2] = a.z; s[3] = a.w; s[4] = b.x; s[5] = b.y; s[6] = b.z; s[7] = b.w;
    }
    MRL_DEV void store(float *states, int32_t *, int i) const {
        float4 *row = reinterpret_cast<float4 *>(states) + 2 * (size_t)i;
        row[0] = make_float4(s[0], s[1], s[2], s[3]);
        row[1] = make_float4(s[4], s[5], s[6], s[7]);
    }
    MRL_DEV float obs(int k) const { return s[k]; }
    MRL_DEV void step(const float *act, float &r, float &d) { pendulum::step(s, act[0], r, d); }
    MRL_DEV void reset(int i, uint64_t seed) { pendulum::reset(s, i, seed); }
};

constexpr int CLASSIC_TPW = 1;   // accumulator tiles per wavefront: 1 = two wavefronts per net
constexpr int CLASSIC_THREADS = 2 * hidden_threads(64, CLASSIC_TPW);

template <class C, int ACT, bool GAUSS>
__global__ __launch_bounds__(CLASSIC_THREADS) void collect_classic_kernel(CollectArgs a, int32_t *side) {
    constexpr int H = 64, TPW = CLASSIC_TPW, TN = hidden_threads(H, TPW), IN = C::OBS, AW = C::ACT_W;
    constexpr int KB = H / 2;   // all of layer 1 in one block of k-steps: its weights stay in registers
    static_assert(IN <= PIN_MAX, "observation fits the input tile");
    __shared__ float xs[PR * XS_LD];
    __shared__ float hT[2][H * HT_LD];
    __shared__ float h2[2][PR * (H + 1)];
    __shared__ float logits[PR * (PA_MAX + 1)];
    __shared__ float vals[PR];
    __shared__ __align__(16) float w2s[2][HEAD_LDS(H)];
    const int t = threadIdx.x;
    const int env0 = blockIdx.x * PR;
    const int nenv = min(PR, a.n_envs - env0);
    const int N = a.n_envs;
    const bool owner = t < nenv;   // lanes 0 .. nenv - 1 of wavefront 0: one env each
    C slot{};
    float ep_return = 0.0f, ep_length = 0.0f;
    if (owner) {
        slot.load(a.states, side, env0 + t);
        ep_return = a.acc.ep_return[env0 + t];
        ep_length = a.acc.ep_length[env0 + t];
    }
    {
        const int net = t / TN;
        const float *p = net ? a.critic_p : a.actor_p;
        stage_head(p + IN * H + H + H * H + H, H, net ? 1 : a.A, GAUSS && net == 0, w2s[net], t % TN, TN);
    }
    for (int i = t; i < PR * XS_LD; i += CLASSIC_THREADS) xs[i] = 0.0f;
    // the hidden layers' weights of this wavefront's column tiles, loaded once for all the steps
    HiddenOperands<H, TPW, KB> ops;
    ops.load(t / TN ? a.critic_p : a.actor_p, IN, t);
    __syncthreads();
    // the policy does not change during the launch: exp(log_std) of the Gaussian head once for all the steps
    float stdv[PA_MAX];
#pragma unroll
    for (int j = 0; j < PA_MAX; ++j) stdv[j] = (GAUSS && owner && j < a.A) ? exp32(gaussian_log_std(w2s[0][HEAD_LOG_STD(H) + j])) : 1.0f;

    for (int k = 0; k < a.n_steps; ++k) {
        // (the empty asm keeps what the optimiser derives from these values inside the step)
        int tid = t, ne = __builtin_amdgcn_readfirstlane(nenv), A = __builtin_amdgcn_readfirstlane(a.A), zero = 0;
        asm volatile("" : "+v"(tid), "+s"(zero), "+s"(ne), "+s"(A) : : "memory");
        const int net = tid / TN;
        const float *p = (net ? a.critic_p : a.actor_p) + zero;
        const size_t row = (size_t)(a.t0 + k) * N + env0;   // this block's slice of rollout row t
        const uint32_t sseed = a.sample_seed + (uint32_t)k * a.sample_stride;
        if (tid < ne) {
#pragma unroll
            for (int c = 0; c < IN; ++c) {
                const float v = slot.obs(c);
                xs[tid * XS_LD + c] = v;
                a.r_obs[(row + tid) * IN + c] = v;
            }
        }
        __syncthreads();
        hidden_stack<H, ACT, TPW, KB>(p, IN, xs, hT[net], h2[net], TileCache{}, ops, tid);
        if (net == 0) head<H>(w2s[0], A, h2[0], logits, PA_MAX + 1, tid % TN, TN);
        else head<H>(w2s[1], 1, h2[1], vals, 1, tid % TN, TN);
        __syncthreads();
        if (tid < ne) {
            const int i = env0 + tid;
            float av[PA_MAX], logp;
            if (GAUSS) {
                logp = sample_gaussian(logits + tid * (PA_MAX + 1), w2s[0] + HEAD_LOG_STD(H), A, sseed, i, av, stdv);
                for (int j = 0; j < A; ++j) a.r_actions[(row + tid) * AW + j] = av[j];
            } else {
                int sel;
                sample_categorical_few(logits + tid * (PA_MAX + 1), A, sseed, i, sel, logp);
                av[0] = (float)sel;
                a.r_actions[row + tid] = av[0];
            }
            a.r_logp[row + tid] = logp;
            a.r_values[row + tid] = vals[tid];
            float r, d;
            slot.step(av, r, d);
            a.r_rewards[row + tid] = r;
            a.r_dones[row + tid] = d;
            ep_return = ep_return + r;
            ep_length = ep_length + 1.0f;
            if (d > 0.5f) {
                const int s = atomicAdd(a.acc.done_count, 1);
                if (s < a.acc.done_cap) {
                    a.acc.done_returns[s] = ep_return;
                    a.acc.done_lengths[s] = ep_length;
                }
                ep_return = 0.0f;
                ep_length = 0.0f;
                slot.reset(i, a.reset_seed + (uint64_t)k * a.reset_stride);
            }
        }
    }
    if (owner) {
        slot.store(a.states, side, env0 + t);
#pragma unroll
        for (int c = 0; c < IN; ++c) a.obs[(size_t)(env0 + t) * IN + c] = slot.obs(c);
        a.acc.ep_return[env0 + t] = ep_return;
        a.acc.ep_length[env0 + t] = ep_length;
    }
}

// true when mrl_rollout_steps can run the descriptor through collect_kernel
// (the wide kernel: LunarLander with hidden width 256; the two-wavefront kernel: CartPole and
// Pendulum with hidden width 64)
static bool collect_fusable(const mrl_rollout *r, bool gauss, int *act) {
    int obs, hidden;
    if (r->env_id == MRL_ENV_LUNARLANDER && !gauss) { obs = LunarLander::OBS; hidden = 256; }
    else if (r->env_id == MRL_ENV_LUNARLANDER_CONTINUOUS && gauss) { obs = LunarLander::OBS; hidden = 256; }
    else if (r->env_id == MRL_ENV_CARTPOLE && !gauss) { obs = cartpole::OBS; hidden = 64; }
    else if (r->env_id == MRL_ENV_PENDULUM && gauss) { obs = pendulum::OBS; hidden = 64; }
    else return false;
    const mrl_mlp_desc &a = r->actor, &c = r->critic;
    if (a.n_layers != 3 || c.n_layers != 3) return false;
    const int k0 = a.layers[0].kind;
    if (k0 != MRL_LINEAR_RELU && k0 != MRL_LINEAR_TANH) return false;
    for (const mrl_mlp_desc *d : {&a, &c}) {
        if (d->layers[0].kind != k0 || d->layers[1].kind != k0) return false;
        if (d->layers[0].in_dim != obs || d->layers[0].out_dim != hidden || d->layers[1].out_dim != hidden) return false;
    }
    if (a.layers[2].kind != (gauss ? MRL_STOCHASTIC_ACTOR : MRL_LINEAR) || c.layers[2].kind != MRL_LINEAR) return false;
    if (a.layers[2].out_dim > PA_MAX || c.layers[2].out_dim != 1) return false;
    *act = (k0 == MRL_LINEAR_RELU) ? 1 : 2;
    return true;
}

}  // namespace mrl

using namespace mrl;

extern "C" {

int mrl_rollout_fused(const mrl_rollout *r) {
    int act = 0;
    return r != nullptr && (collect_fusable(r, r->num_actions == 0, &act) || collect_walker_fusable(r, &act)) ? 1 : 0;
}

int mrl_rollout_steps(mrl_ctx *ctx, const mrl_rollout *r, int t0, int n_steps, uint32_t sample_seed,
                      uint32_t sample_stride, uint64_t step_seed, uint64_t step_stride, uint64_t reset_seed,
                      uint64_t reset_stride) {
    MRL_CHECK_ARG(ctx && r, "mrl_rollout_steps: NULL argument");
    MRL_CHECK_ARG(t0 >= 0 && n_steps >= 0, "mrl_rollout_steps: bad step range");
    if (n_steps == 0) return MRL_OK;
    const bool gauss = r->num_actions == 0;
    int act = 0;
    const bool walker = collect_walker_fusable(r, &act);
    if (!walker && !collect_fusable(r, gauss, &act)) {
        for (int k = 0; k < n_steps; ++k) {
            int rc = mrl_rollout_step(ctx, r, t0 + k, sample_seed + (uint32_t)k * sample_stride,
                                      step_seed + (uint64_t)k * step_stride, reset_seed + (uint64_t)k * reset_stride);
            if (rc) return rc;
        }
        return MRL_OK;
    }
    MRL_CHECK_ARG(r->n_envs > 0, "mrl_rollout_steps: bad sizes");
    MRL_CHECK_ARG(r->states && r->obs && r->actor_params && r->critic_params && r->r_obs && r->r_actions &&
                      r->r_log_probs && r->r_values && r->r_rewards && r->r_dones && r->ep_return &&
                      r->ep_length && r->done_returns && r->done_lengths && r->done_count,
                  "mrl_rollout_steps: NULL buffer in descriptor");
    int ss, od, na, ad;
    int rc = mrl_env_dims(r->env_id, &ss, &od, &na, &ad);
    if (rc) return rc;
    MRL_CHECK_ARG(od == r->obs_dim && (gauss ? (ad > 0 && mrl_mlp_out_dim(&r->actor) == 2 * ad)
                                             : (na == r->num_actions && mrl_mlp_out_dim(&r->actor) == na)),
                  "mrl_rollout_steps: descriptor does not match the env's observation / action space");
    const float *shapes = ctx->ll_shapes;
    CollectArgs a{};
    a.states = r->states; a.obs = r->obs;
    a.actor_p = r->actor_params; a.critic_p = r->critic_params; a.shapes = shapes;
    a.n_envs = r->n_envs; a.A = gauss ? ad : na; a.t0 = t0; a.n_steps = n_steps;
    a.sample_seed = sample_seed; a.sample_stride = sample_stride;
    a.reset_seed = reset_seed; a.reset_stride = reset_stride;
    a.r_obs = r->r_obs; a.r_actions = r->r_actions; a.r_logp = r->r_log_probs; a.r_values = r->r_values;
    a.r_rewards = r->r_rewards; a.r_dones = r->r_dones;
    a.acc = Accounting{r->r_rewards, r->r_dones, r->ep_return, r->ep_length, r->done_returns, r->done_lengths,
                       r->done_count, r->done_cap};
    a.spin_limit = ctx->spin_limit;
    a.sync_error = ctx->sync_error;
    a.car_trait_form = ctx->car_trait_form;
    // LunarLander: with at most 16 envs per CU the 16-row kernel (a shorter chain per step); beyond that
    // the 32-row kernel, whose single solver wavefront per CU steps twice the envs in the same time
    const bool lander = r->env_id == MRL_ENV_LUNARLANDER || r->env_id == MRL_ENV_LUNARLANDER_CONTINUOUS;
    const bool rows16 = lander && r->n_envs <= ctx->n_cus * PR16;
    const dim3 grid(grid_for(r->n_envs, rows16 ? PR16 : PR));
    int32_t *side = nullptr;
    if (r->env_id == MRL_ENV_CARTPOLE) {
        rc = cartpole_side(ctx, r->states, r->n_envs, &side);
        if (rc) return rc;
    }
    profile_step_begin(ctx);
    profile_mark(ctx, -1);
    if (walker) {
        rc = launch_collect_walker(ctx, r, a, act);
        if (rc) return rc;
    } else if (r->env_id == MRL_ENV_LUNARLANDER && rows16) {
        const dim3 block(Rows16<LunarLander>::THREADS);
        if (act == 1) hipLaunchKernelGGL((collect16_kernel<LunarLander, 1, false>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((collect16_kernel<LunarLander, 2, false>), grid, block, 0, ctx->stream, a);
    } else if (r->env_id == MRL_ENV_LUNARLANDER_CONTINUOUS && rows16) {
        const dim3 block(Rows16<LunarLander>::THREADS);
        if (act == 1) hipLaunchKernelGGL((collect16_kernel<LunarLanderContinuous, 1, true>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((collect16_kernel<LunarLanderContinuous, 2, true>), grid, block, 0, ctx->stream, a);
    } else if (r->env_id == MRL_ENV_LUNARLANDER) {
        const dim3 block(LunarLander::THREADS);
        if (act == 1) hipLaunchKernelGGL((collect_kernel<LunarLander, 256, 1, false>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((collect_kernel<LunarLander, 256, 2, false>), grid, block, 0, ctx->stream, a);
    } else if (r->env_id == MRL_ENV_LUNARLANDER_CONTINUOUS) {
        const dim3 block(LunarLander::THREADS);
        if (act == 1) hipLaunchKernelGGL((collect_kernel<LunarLanderContinuous, 256, 1, true>), grid, block, 0, ctx->stream, a);
        else hipLaunchKernelGGL((collect_kernel<LunarLanderContinuous, 256, 2, true>), grid, block, 0, ctx->stream, a);
    } else if (r->env_id == MRL_ENV_CARTPOLE) {
        if (act == 1) hipLaunchKernelGGL((collect_classic_kernel<CartPoleSlot, 1, false>), grid, dim3(CLASSIC_THREADS), 0, ctx->stream, a, side);
        else hipLaunchKernelGGL((collect_classic_kernel<CartPoleSlot, 2, false>), grid, dim3(CLASSIC_THREADS), 0, ctx->stream, a, side);
    } else {
        if (act == 1) hipLaunchKernelGGL((collect_classic_kernel<PendulumSlot, 1, true>), grid, dim3(CLASSIC_THREADS), 0, ctx->stream, a, side);
        else hipLaunchKernelGGL((collect_classic_kernel<PendulumSlot, 2, true>), grid, dim3(CLASSIC_THREADS), 0, ctx->stream, a, side);
    }
    MRL_CHECK_LAUNCH();
    profile_mark(ctx, MRL_PHASE_COLLECT);
    profile_step_end(ctx);
    return MRL_OK;
}

}  // extern "C"
