// Workgroup-level pieces of the physics2d env kernels, shared by the single-step kernels and the
// fused collection kernel: per-env traits, row staging between HBM and LDS, in-place resets and
// the step of a block's LDS-resident rows.
#pragma once
#include "mrl_host.hpp"
#include "env_lunar.hpp"
#include "env_walkers.hpp"
#include "env_bipedal_lanes.hpp"

namespace mrl {

// _store_post_step_kernel (deep_agents/ppo/ppo.mojo:692-708) + accumulate_rewards /
// increment_steps / extract_completed_episodes (deep_rl/gpu/rl_kernels.mojo:103-200) for one env
// `before` = env i's running (return, length) as they stood before the step; a caller with a long
// step reads them ahead of it (account_before) so that the step does not end on a memory round trip
struct EpisodeSums { float ret, len; };
MRL_DEV EpisodeSums account_before(const Accounting &acc, int i) {
    if (acc.r_rewards == nullptr) return EpisodeSums{0.0f, 0.0f};
    return EpisodeSums{acc.ep_return[i], acc.ep_length[i]};
}
MRL_DEV void account(const Accounting &acc, int i, float r, float d, const EpisodeSums &before) {
    if (acc.r_rewards == nullptr) return;
    acc.r_rewards[i] = r;
    acc.r_dones[i] = d;
    float er = before.ret + r;
    float el = before.len + 1.0f;
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
MRL_DEV void account(const Accounting &acc, int i, float r, float d) { account(acc, i, r, d, account_before(acc, i)); }

// ---------------------------------------------------------------- physics2d envs
// Per-env traits of the LDS-staged kernels.  EPB = env rows per workgroup (one wavefront; with
// 32 rows the upper half of the lanes only helps with the copies), DYN_END = first float of the
// row that a step never writes (everything before it, plus the metadata, is copied back).

struct LunarLander {
    using L = ll::L;
    static constexpr int STATE = ll::STATE, OBS = ll::OBS, ACT_W = 1, EPB = 32, THREADS = 512;
    static constexpr int LANE_FROM = 8193;   // batch from which the stand-alone step runs one lane per env
    static constexpr int DYN_END = L::JOINTS_OFF, NSHAPE = ll::NSHAPE_FLOATS;
    static MRL_DEV void step(float *row, float *cts, const float *shapes, int env, const float *a,
                             float &r, float &d) {
        ll::step_row(row, cts, shapes, env, (int)a[0], r, d);
    }
    static constexpr int POST_TASKS = 0, POST_WORDS = 0, POST_PARTS = 1;
    static MRL_DEV void post_share(const float *, int, unsigned *) {}
    static MRL_DEV float post_task(const float *, int, const unsigned *) { return 0.0f; }
    static MRL_DEV void post_join(float *, int, const float *) {}
    static MRL_DEV void reset(float *row, uint64_t seed, int env) {
        ll::reset_row(row, ll::combined_seed(seed, env));
    }
    static constexpr bool WAVE_RESET = true;
    static MRL_DEV void reset_wave(float *row, uint64_t seed, int env, int lane) {
        ll::reset_row_wave(row, ll::combined_seed(seed, env), lane);
    }
    // contact detection runs beside the engines of wavefront 0: every half of wavefronts 1 .. 7
    // takes one (body, vertex) pair of the block's 32 envs -- hull 6 vertices, legs 4 each
    static constexpr int DETECT_TASKS = 14, DETECT_WORDS = 0;
    static MRL_DEV void detect_share(const float *, const float *, int, unsigned *) {}
    static MRL_DEV void detect_task(int k, int &body, int &vertex, int &max_verts) {
        if (k < 6) { body = 0; vertex = k; max_verts = 6; }
        else if (k < 10) { body = 1; vertex = k - 6; max_verts = 4; }
        else { body = 2; vertex = k - 10; max_verts = 4; }
    }
    static constexpr bool LANES_PHYSICS = false;   // (BipedalWalker: the physics by one lane per body)
    using Carry = ll::StepCarry;
    static MRL_DEV Carry step_begin(float *row, int env, const float *a, const float *shapes) {
        return ll::step_begin(row, env, (int)a[0], shapes);
    }
    static MRL_DEV void step_finish(float *row, float *cts, int n, const float *shapes, const Carry &c, float &r,
                                    float &d) {
        ll::step_finish(row, cts, n, shapes, c, r, d);
    }
};

// LunarLanderV2 behind the continuous-action trait (the reference overloads step_kernel_gpu on
// the same struct, lunar_lander_v2.mojo:1520-1588): same rows, resets and contact detection,
// two action components per env
struct LunarLanderContinuous : LunarLander {
    static constexpr int ACT_W = 2;
    static MRL_DEV void step(float *row, float *cts, const float *shapes, int env, const float *a,
                             float &r, float &d) {
        const Carry c = ll::step_begin_continuous(row, env, a, shapes);
        ll::step_finish(row, cts, -1, shapes, c, r, d);
    }
    static MRL_DEV Carry step_begin(float *row, int env, const float *a, const float *shapes) {
        return ll::step_begin_continuous(row, env, a, shapes);
    }
};

struct BipedalWalker {
    using L = bw::L;
    static constexpr int STATE = bw::STATE, OBS = bw::OBS, ACT_W = bw::ACT, EPB = 16, THREADS = 512;
    static constexpr int LANE_FROM = 0;      // (never: the lane form is no faster for this env at any batch)
    static constexpr int DYN_END = L::EDGES_OFF, NSHAPE = bw::NSHAPE_FLOATS;
    // the ten lidar rays of the observation are left out of the step and run afterwards, spread
    // over all wavefronts of the block: task k = part k % 3 of the edges for ray k / 3; the parts of
    // a ray meet in LDS (post_join).
    static constexpr int POST_PARTS = 3, POST_TASKS = 10 * POST_PARTS;
    static MRL_DEV void step(float *row, float *cts, const float *shapes, int env, const float *a,
                             float &r, float &d) {
        bw::step_row<false>(row, cts, shapes, env, a, r, d);
    }
    // ahead of the rays, once per env and by all its lanes: the mask of the edges within lidar range of the hull
    static constexpr int POST_WORDS = EdgeMask<L>::WORDS;
    static MRL_DEV void post_share(const float *row, int slot, unsigned *words) {
        bw::lidar_near_share<THREADS / EPB, EPB>(row, slot, words);
    }
    static MRL_DEV float post_task(const float *row, int task, const unsigned *words) {
        return bw::lidar_value_part<POST_PARTS>(row, task / POST_PARTS, task % POST_PARTS, words);
    }
    // parts = the values of the env's tasks
    static MRL_DEV void post_join(float *row, int ray, const float *parts) {
        float t = parts[ray * POST_PARTS];
#pragma unroll
        for (int k = 1; k < POST_PARTS; ++k) {
            const float other = parts[ray * POST_PARTS + k];
            t = other < t ? other : t;
        }
        row[14 + ray] = t;
    }
    static MRL_DEV void reset(float *row, uint64_t seed, int env) { bw::reset_row(row, walker_seed(seed, env)); }
    static constexpr bool WAVE_RESET = true;
    static MRL_DEV void reset_wave(float *row, uint64_t seed, int env, int lane) {
        bw::reset_row_wave(row, walker_seed(seed, env), lane);
    }
    // contact detection ahead of the step, spread over all wavefronts: one (body, vertex) pair of
    // one env per lane -- hull 5 vertices, the four leg segments 4 each, against the 128 edges
    static constexpr int DETECT_TASKS = 21;
    // ahead of the pairs, once per env and by all its lanes: the mask of the edges near any of its bodies
    static constexpr int DETECT_WORDS = EdgeMask<L>::WORDS;
    static MRL_DEV void detect_share(const float *row, const float *shapes, int slot, unsigned *words) {
        bw::detect_near_share<THREADS / EPB, EPB>(row, shapes, slot, words);
    }
    static MRL_DEV void detect_task(int k, int &body, int &vertex, int &max_verts) {
        if (k < 5) { body = 0; vertex = k; max_verts = 5; }
        else { body = 1 + (k - 5) / 4; vertex = (k - 5) % 4; max_verts = 4; }
    }
    struct Carry { float act[bw::ACT]; };
    static MRL_DEV Carry step_begin(float *row, int, const float *a, const float *) {
        Carry c;
        bw::step_motors(row, a, c.act);
        return c;
    }
    static MRL_DEV void step_finish(float *row, float *cts, int n, const float *shapes, const Carry &c, float &r,
                                    float &d) {
        bw::step_finish<false>(row, cts, n, shapes, c.act, r, d);
    }
    // step_finish in two parts: the physics by the eight lanes of an env's group (env_bipedal_lanes.hpp),
    // then the rest by the env's lane
    static constexpr bool LANES_PHYSICS = true;
    static constexpr int LANES_PER_ENV = bw::LANES_PER_ENV;
    static MRL_DEV bool lanes_ok(const float *row) { return bw::lanes_row_ok(row); }
    static MRL_DEV void physics_lanes(float *row, float *cts, int n, int lane) { bw::physics_lanes(row, cts, n, lane); }
    static MRL_DEV void step_tail(float *row, const float *cts, int n, const Carry &c, float &r, float &d) {
        bw::step_tail<false, false>(row, cts, n, c.act, r, d);
    }
};

struct HalfCheetah {
    using L = hc::L;
    static constexpr int STATE = hc::STATE, OBS = hc::OBS, ACT_W = hc::ACT, EPB = 64, THREADS = 256;
    static constexpr int LANE_FROM = 0;      // (never: the lane form is no faster for this env at any batch)
    static constexpr int DYN_END = L::EDGES_OFF, NSHAPE = hc::NSHAPE_FLOATS;
    static MRL_DEV void step(float *row, float *cts, const float *shapes, int env, const float *a,
                             float &r, float &d) {
        hc::step_row(row, cts, shapes, env, a, r, d);
    }
    static constexpr bool LANES_PHYSICS = false;
    static constexpr int POST_TASKS = 0, POST_WORDS = 0, POST_PARTS = 1;
    static MRL_DEV void post_share(const float *, int, unsigned *) {}
    static MRL_DEV float post_task(const float *, int, const unsigned *) { return 0.0f; }
    static MRL_DEV void post_join(float *, int, const float *) {}
    static MRL_DEV void reset(float *row, uint64_t seed, int env) { hc::reset_row(row, walker_seed(seed, env)); }
    static constexpr bool WAVE_RESET = false;
    static MRL_DEV void reset_wave(float *, uint64_t, int, int) {}
    static constexpr int DETECT_TASKS = 0, DETECT_WORDS = 0;
    static MRL_DEV void detect_share(const float *, const float *, int, unsigned *) {}
    static MRL_DEV void detect_task(int, int &, int &, int &) {}
    struct Carry {};
    static MRL_DEV Carry step_begin(float *, int, const float *, const float *) { return Carry{}; }
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
        // The block's rows are one contiguous run that starts on a 16-byte boundary (EPB rows are a
        // multiple of 16 bytes), so it is read with 16-byte loads whatever STATE is; a load may
        // straddle two rows, each float finds its own (row, column).
        static_assert((E::EPB * E::STATE) % 4 == 0, "a block's rows start 16-byte aligned");
        const int total = nenv * E::STATE;
        const int total4 = total / 4;
        const float4 *src = reinterpret_cast<const float4 *>(g);
        for (int i0 = lane; i0 < total4; i0 += UNROLL * E::THREADS) {
            float4 v[UNROLL];
#pragma unroll
            for (int k = 0; k < UNROLL; ++k)
                if (i0 + k * E::THREADS < total4) v[k] = src[i0 + k * E::THREADS];
#pragma unroll
            for (int k = 0; k < UNROLL; ++k) {
                if (i0 + k * E::THREADS >= total4) continue;
                const int f = (i0 + k * E::THREADS) * 4;
                const float e[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
                if (E::STATE % 4 == 0) {   // never straddles
                    const int r = f / E::STATE, c = f - r * E::STATE;
                    float *d = lds + r * STRIDE + c;
                    d[0] = e[0]; d[1] = e[1]; d[2] = e[2]; d[3] = e[3];
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int r = (f + j) / E::STATE, c = (f + j) - r * E::STATE;
                        lds[r * STRIDE + c] = e[j];
                    }
                }
            }
        }
        for (int i = total4 * 4 + lane; i < total; i += E::THREADS) {   // at most three floats
            const int r = i / E::STATE, c = i - r * E::STATE;
            lds[r * STRIDE + c] = g[i];
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

// The same with every wavefront of the block taking part (all threads call it): wavefront w
// rebuilds the rows whose rank among the set bits is w modulo the number of wavefronts.
template <class E>
MRL_DEV void reset_rows_block(float *rows, unsigned long long mask, uint64_t seed, int env0, int tid) {
    using S = Stage<E>;
    constexpr int NW = E::THREADS / 64;
    const int wave = tid / 64, lane = tid % 64;
    if (E::WAVE_RESET && __popcll(mask) <= 8 * NW) {
        int rank = 0;
        while (mask) {
            const int src = __ffsll((long long)mask) - 1;
            mask &= mask - 1;
            if (rank % NW == wave) E::reset_wave(rows + src * S::STRIDE, seed, env0 + src, lane);
            ++rank;
        }
    } else if (wave == 0 && ((mask >> lane) & 1ull)) {
        E::reset(rows + lane * S::STRIDE, seed, env0 + lane);
    }
}

// Per-(body, vertex) contact lists of phys_step_block: CAP records per list (a vertex that fills
// its list sends the env back to detection inside step_finish), list stride in floats.
constexpr int DETECT_CAP = 4;
constexpr int detect_stride(int cap) { return (cap * CONTACT_SIZE) | 1; }
constexpr int DETECT_STRIDE = detect_stride(DETECT_CAP);

// task `task` of env slot e: detects into its list and records the count
template <class E, int CAP = DETECT_CAP>
MRL_DEV void detect_vertex_task(const float *rows, const float *shapes, float *dlist, int *dcount, int task, int e,
                                const unsigned *near = nullptr) {
    int body, vertex, max_verts;
    E::detect_task(task, body, vertex, max_verts);
    dcount[task * E::EPB + e] = edge_detect_vertex<typename E::L>(
        rows + e * Stage<E>::STRIDE, shapes, body, vertex, max_verts, dlist + (task * E::EPB + e) * detect_stride(CAP),
        CAP, near);
}

// concatenates env slot e's lists in (body, vertex) order into `mine`, cut at MAX_CONTACTS;
// returns the contact count, or -1 when some list asks for detection to be redone
template <class E, int CAP = DETECT_CAP>
MRL_DEV int merge_vertex_lists(const float *dlist, const int *dcount, int e, float *mine) {
    // all counts first (independent loads, one round trip), then only the lists that hold something:
    // most steps of most envs have no contact at all
    int m[E::DETECT_TASKS];
#pragma unroll
    for (int k = 0; k < E::DETECT_TASKS; ++k) m[k] = dcount[k * E::EPB + e];
    bool redo = false, any = false;
#pragma unroll
    for (int k = 0; k < E::DETECT_TASKS; ++k) {
        redo |= m[k] < 0;
        any |= m[k] > 0;
    }
    int n = 0;
    if (any) {
#pragma unroll
        for (int k = 0; k < E::DETECT_TASKS; ++k) {
            const float *src = dlist + (k * E::EPB + e) * detect_stride(CAP);
            for (int c = 0; c < m[k] && c < CAP && n < E::L::MAX_CONTACTS; ++c, ++n) {
                // a record is read whole before it is written (the two LDS ranges never overlap, which the
                // compiler cannot see: it would wait for every float on its own)
                float rec[CONTACT_SIZE];
#pragma unroll
                for (int f = 0; f < CONTACT_SIZE; ++f) rec[f] = src[c * CONTACT_SIZE + f];
#pragma unroll
                for (int f = 0; f < CONTACT_SIZE; ++f) mine[n * CONTACT_SIZE + f] = rec[f];
            }
        }
    }
    return redo ? -1 : n;
}

// merge_vertex_lists by the lanes that made the lists: the lane of (env slot e, task) moves its own list to
// its place in the env's merged list -- behind the contacts of the tasks before it -- so that all lists move
// at once.  Returns what merge_vertex_lists returns (every lane of the env gets the same value).
template <class E, int CAP = DETECT_CAP>
MRL_DEV int merge_vertex_list_of_task(const float *dlist, const int *dcount, int e, int task, float *mine) {
    int m[E::DETECT_TASKS];
#pragma unroll
    for (int k = 0; k < E::DETECT_TASKS; ++k) m[k] = dcount[k * E::EPB + e];
    bool redo = false;
    int before = 0, total = 0, own = 0;
#pragma unroll
    for (int k = 0; k < E::DETECT_TASKS; ++k) {
        redo |= m[k] < 0;
        const int c = m[k] < 0 ? 0 : (m[k] < CAP ? m[k] : CAP);
        before += k < task ? c : 0;
        own = k == task ? c : own;
        total += c;
    }
    const float *src = dlist + (task * E::EPB + e) * detect_stride(CAP);
    for (int c = 0; c < own && before + c < E::L::MAX_CONTACTS; ++c) {
        float rec[CONTACT_SIZE];
#pragma unroll
        for (int f = 0; f < CONTACT_SIZE; ++f) rec[f] = src[c * CONTACT_SIZE + f];
#pragma unroll
        for (int f = 0; f < CONTACT_SIZE; ++f) mine[(before + c) * CONTACT_SIZE + f] = rec[f];
    }
    return redo ? -1 : (total < E::L::MAX_CONTACTS ? total : E::L::MAX_CONTACTS);
}

// One step of the block's LDS-resident rows (all threads of the block call it, between two
// __syncthreads of the caller): wavefront 0 steps one env per lane, the other wavefronts detect
// contacts where the env splits that off.  `actions` = the actions of the block's envs
// ([nenv][ACT_W], global or LDS), rewards / dones = the block's slice of the per-step outputs
// (may be null), acc = rollout accounting with its pointers already offset to the block's first
// env.  AUTORESET: rows that finished are re-initialised in place and recorded in *was_reset.
// (what phys_step_block runs beside the one-lane-per-body solver when the caller has nothing for it)
struct NoSideJob {
    MRL_DEV void operator()(int) const {}
};

// `side`: work of the caller's that the wavefronts without a part in the one-lane-per-body solver (LANES_PHYSICS
// envs: wavefronts 2 and up) do while wavefronts 0 and 1 run it, called as side(tid) between the two block
// barriers around the solver; it must not touch the rows or the contact scratch `cts`.
template <class E, bool AUTORESET, class Side = NoSideJob>
MRL_DEV void phys_step_block(float *rows, float *cts, const float *shapes, float *dlist, int *dcount,
                             unsigned long long *was_reset, const float *actions, float *rewards,
                             float *dones, int env0, int nenv, uint64_t reset_seed, const Accounting &acc,
                             int tid = threadIdx.x, Side side = Side{}) {
    using S = Stage<E>;
    if constexpr (E::DETECT_TASKS > 0 && E::POST_TASKS == 0) {
        // wavefront 0: first half of the step (reads and writes velocities only); the halves of the
        // other wavefronts: contacts of one (body, vertex) pair each (read positions only), into
        // lists of their own.  A vertex that fills its list, or a body whose shape the task table
        // does not cover, sends that env back to detection inside step_finish.
        // (a wavefront holds WAVE / EPB tasks at a time; a block with fewer such groups than tasks takes turns)
        constexpr int NT = E::DETECT_TASKS, GROUP = E::EPB, PER_WAVE = WAVE / GROUP;
        constexpr int AT_ONCE = (E::THREADS / WAVE - 1) * PER_WAVE;
        static_assert((GROUP == 16 || GROUP == 32) && AT_ONCE > 0, "16 or 32 rows per workgroup, wavefront 0 and at least one more");
        const int wave = tid / WAVE, lane = tid % WAVE;
        typename E::Carry carry{};
        EpisodeSums sums{0.0f, 0.0f};
        if (wave == 0) {
            if (lane < nenv) sums = account_before(acc, lane);
            if (lane < nenv)
                carry = E::step_begin(rows + lane * S::STRIDE, env0 + lane, actions + (size_t)lane * E::ACT_W, shapes);
        } else {
            const int e = lane % GROUP;
#pragma unroll 1
            for (int task = (wave - 1) * PER_WAVE + lane / GROUP; task < NT; task += AT_ONCE)
                if (e < nenv) detect_vertex_task<E>(rows, shapes, dlist, dcount, task, e);
        }
        __syncthreads();
        if (wave == 0) {
            bool finished = false;
            if (lane < nenv) {
                float *mine = cts + lane * S::CSTRIDE;
                const int n = merge_vertex_lists<E>(dlist, dcount, lane, mine);
                const int env = env0 + lane;
                float r, d;
                E::step_finish(rows + lane * S::STRIDE, mine, n, shapes, carry, r, d);
                if (rewards != nullptr) {
                    rewards[env - env0] = r;
                    dones[env - env0] = d;
                }
                account(acc, env - env0, r, d, sums);
                finished = d > 0.5f;
            }
            if (AUTORESET) reset_rows<E>(rows, was_reset, __ballot(finished), reset_seed, env0, lane);
        }
    } else {
        typename E::Carry carry{};
        if constexpr (E::DETECT_TASKS > 0) {
            // first the contacts, by every wavefront: EPB lanes per (body, vertex) pair, as many
            // pairs at a time as the block has such lane groups; the lanes that will step the envs
            // put the action into the joint motors first (detection does not read the joints)
            static_assert(WAVE % E::EPB == 0 && E::EPB <= WAVE, "lane groups of EPB inside a wavefront");
            constexpr int SLOTS = E::THREADS / E::EPB;
            const int e = tid % E::EPB;
            if (tid < nenv) carry = E::step_begin(rows + tid * S::STRIDE, env0 + tid, actions + (size_t)tid * E::ACT_W, shapes);
            // (what the pairs of an env share goes behind the contact counts: detect_count_ints)
            const unsigned *near = nullptr;
            if constexpr (E::DETECT_WORDS > 0) {
                unsigned *words = reinterpret_cast<unsigned *>(dcount + E::DETECT_TASKS * E::EPB + 1) + e * E::DETECT_WORDS;
                if (e < nenv) E::detect_share(rows + e * S::STRIDE, shapes, tid / E::EPB, words);
                __syncthreads();
                near = words;
            }
            if (e < nenv)
                for (int task = tid / E::EPB; task < E::DETECT_TASKS; task += SLOTS)
                    detect_vertex_task<E>(rows, shapes, dlist, dcount, task, e, near);
            __syncthreads();
        }
        int lanes_n = 0;          // LANES_PHYSICS: the env's contact count; -1: the one-lane form steps this env
        if constexpr (E::LANES_PHYSICS) {
            // the physics of the step by one lane per body: the env's lane merges the contact lists, then
            // LANES_PER_ENV lanes per env (the first wavefronts of the block) run the solver, then the env's
            // lane goes on below with what follows the physics
            static_assert(E::DETECT_TASKS > 0 && E::EPB * E::LANES_PER_ENV <= E::THREADS, "a lane group per env");
            // (the env's contact count goes where its tasks' shared words were: they are spent, the counts are not yet)
            static_assert(E::DETECT_WORDS >= 1 && E::DETECT_TASKS <= E::THREADS / E::EPB, "a word per env, a lane per task");
            int *ncontacts = dcount + E::DETECT_TASKS * E::EPB + 1;
            {
                const int e = tid % E::EPB, task = tid / E::EPB;
                if (e < nenv && task < E::DETECT_TASKS) {
                    const int n = merge_vertex_list_of_task<E>(dlist, dcount, e, task, cts + e * S::CSTRIDE);
                    if (task == 0) ncontacts[e] = (n >= 0 && E::lanes_ok(rows + e * S::STRIDE)) ? n : -1;
                }
            }
            __syncthreads();
            const int slot = tid / E::LANES_PER_ENV;
            if (slot < nenv) {
                const int n = ncontacts[slot];
                if (n >= 0) E::physics_lanes(rows + slot * S::STRIDE, cts + slot * S::CSTRIDE, n, tid % WAVE);
            }
            static_assert(E::EPB * E::LANES_PER_ENV <= 2 * WAVE, "the solver's lanes are wavefronts 0 and 1");
            if (tid >= 2 * WAVE) side(tid);
            __syncthreads();
            if (tid < nenv) lanes_n = ncontacts[tid];
        }
        if (tid < WAVE) {
            bool finished = false;
            if (tid < nenv) {
                const int env = env0 + tid;
                const EpisodeSums sums = account_before(acc, tid);
                float r, d;
                if constexpr (E::LANES_PHYSICS) {
                    float *mine = cts + tid * S::CSTRIDE;
                    if (lanes_n >= 0) E::step_tail(rows + tid * S::STRIDE, mine, lanes_n, carry, r, d);
                    else E::step_finish(rows + tid * S::STRIDE, mine, -1, shapes, carry, r, d);
                } else if constexpr (E::DETECT_TASKS > 0) {
                    float *mine = cts + tid * S::CSTRIDE;
                    const int n = merge_vertex_lists<E>(dlist, dcount, tid, mine);
                    E::step_finish(rows + tid * S::STRIDE, mine, n, shapes, carry, r, d);
                } else {
                    E::step(rows + tid * S::STRIDE, cts + tid * S::CSTRIDE, shapes, env,
                            actions + (size_t)tid * E::ACT_W, r, d);
                }
                if (rewards != nullptr) {
                    rewards[env - env0] = r;
                    dones[env - env0] = d;
                }
                account(acc, env - env0, r, d, sums);
                finished = d > 0.5f;
            }
            if (E::POST_TASKS > 0) {
                const unsigned long long fin = __ballot(finished);
                if (tid == 0) *was_reset = AUTORESET ? fin : 0ull;
            } else if (AUTORESET) {
                reset_rows<E>(rows, was_reset, __ballot(finished), reset_seed, env0, tid);
            }
        }
        if constexpr (E::POST_TASKS > 0) {
            // what the step left for afterwards (rows that finished get it from their reset instead),
            // then the resets, both by all wavefronts
            __syncthreads();
            const unsigned long long fin = *was_reset;
            constexpr int SLOTS = E::THREADS / E::EPB;   // tasks in flight per env
            const int e = tid % E::EPB;
            // what the tasks of an env share is worked out first, by all its lanes, into the (spent)
            // contact counts; the tasks leave their values in the (spent) contact lists, where the
            // first lanes of the env put those of one result together
            const bool live = e < nenv && !((fin >> e) & 1ull);
            const int slot = tid / E::EPB;
            unsigned *words = reinterpret_cast<unsigned *>(dcount) + e * E::POST_WORDS;
            float *parts = dlist + e * E::POST_TASKS;
            static_assert(E::POST_WORDS <= E::DETECT_TASKS && E::POST_TASKS <= detect_stride(1) * E::DETECT_TASKS &&
                          E::POST_TASKS <= SLOTS, "words and task values fit the counts and lists, a task per lane");
            if constexpr (E::POST_WORDS > 0) {
                if (live) E::post_share(rows + e * S::STRIDE, slot, words);
                __syncthreads();
            }
            if (live && slot < E::POST_TASKS) parts[slot] = E::post_task(rows + e * S::STRIDE, slot, words);
            __syncthreads();
            if (live && slot < E::POST_TASKS / E::POST_PARTS) E::post_join(rows + e * S::STRIDE, slot, parts);
            if (AUTORESET) reset_rows_block<E>(rows, fin, reset_seed, env0, tid);
        }
    }
}

// LDS ints of phys_step_block's contact counts: one per list (and one spare), then what an env's tasks share
template <class E>
constexpr int detect_count_ints() { return E::DETECT_TASKS * E::EPB + 1 + E::DETECT_WORDS * E::EPB; }

// LDS floats of the per-task contact lists that phys_step_block needs (0: the env detects inline)
template <class E, int CAP = DETECT_CAP>
constexpr int detect_list_floats() { return E::DETECT_TASKS * E::EPB * detect_stride(CAP); }

// An env's traits with 16 rows per workgroup of four wavefronts (the fused collection kernel runs
// two such workgroups per CU, so that one's env step overlaps the other's policy forward)
template <class Base>
struct Rows16 : Base {
    static constexpr int EPB = 16, THREADS = 256;
};

}  // namespace mrl
