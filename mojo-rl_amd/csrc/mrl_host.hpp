// Host-side plumbing shared by the translation units of libmrl_hip.so: the context object,
// the thread-local error string and launch helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <algorithm>
#include <unordered_map>
#include <vector>
#include "../../include/mrl.h"

struct mrl_ctx {
    hipStream_t stream;
    int device;
    int n_cus;   // compute units of the device
    // CartPole keeps its per-env step counter (truncation at 500) outside the [B,4] state rows;
    // one int32[batch] array per states pointer, created on first use, freed with the context.
    struct Side { int32_t *steps; int batch; bool owned; };   // owned: allocated by the library
    std::unordered_map<const void *, Side> cartpole_steps;
    // device copy of the shape tables (filled at context creation)
    float *ll_shapes, *bw_shapes, *hc_shapes;
    // scratch for two-pass reductions (grad-norm partial sums, advantage statistics)
    float *reduce_scratch;
    int reduce_scratch_floats;
    // MLP workspace: activations between layers and split-batch partial gradients; grown on demand
    float *mlp_ws;
    size_t mlp_ws_floats;
    // per-step temporaries of the fused rollout step (logits, values, actions, log-probs,
    // rewards, dones for n_envs), grown on demand
    float *rollout_ws;
    size_t rollout_ws_floats;
    // scratch of the minibatch update: per-block KL partials [0, 1024), their arrival counter
    // (int, at float index 1024; zero between launches), sum-of-squares partials [2048, 4096),
    // advantage {mean, std} of up to 2048 minibatches [4096, 8192)
    float *upd_scratch;
    // Kernels whose wavefronts meet at barriers of their own (counters in LDS) bound every wait by
    // spin_limit polls; a wait that gives up raises *sync_error (pinned host memory that the device
    // writes directly) and the kernel ends normally.  mrl_ctx_synchronize reports and clears it.
    unsigned spin_limit;
    int *sync_error;
    // CarRacingV2: 0 = the CPU env's reward / termination arithmetic (default), 1 = the GPU trait's
    int car_trait_form;
    // phase timing: events recorded on `stream` at phase boundaries while armed
    bool profiling;
    std::vector<hipEvent_t> prof_events;
    std::vector<int> prof_tags;
    size_t prof_used;
    bool prof_chained;   // the last event recorded closes a phase and can open the next one
    int prof_every;      // rollout steps between two that are timed (1 = every step)
    long prof_step;      // rollout steps seen since profiling was armed
    bool prof_active;    // marks of the current rollout step are recorded
    bool prof_open_next; // the current rollout step ends with the event that opens the next one
};

namespace mrl {

int set_error(int code, const char *fmt, ...);

// makes *buf hold at least `need` floats (never shrinks); growing drains the stream first
int grow_workspace(mrl_ctx *ctx, float **buf, size_t *have, size_t need);

// Post-step bookkeeping of a collection step, done by the env-step kernel itself when the rollout
// step asks for it (all pointers null otherwise): rollout rows of reward / done, per-env episode
// return and length, and the device-side list of finished episodes.
struct Accounting {
    float *r_rewards, *r_dones;        // [N] row t of the time-major buffers
    float *ep_return, *ep_length;      // [N]
    float *done_returns, *done_lengths;
    int32_t *done_count;
    int32_t done_cap;
    // the same accounting seen from env i: per-env pointers advanced, the shared list untouched
    __host__ __device__ __forceinline__ Accounting at(int i) const {
        Accounting a = *this;
        if (r_rewards != nullptr) {
            a.r_rewards += i; a.r_dones += i; a.ep_return += i; a.ep_length += i;
        }
        return a;
    }
};

// mrl_env_step_autoreset with the bookkeeping folded into the same launch
int env_step_accounting(mrl_ctx *ctx, int env_id, int batch, float *states, const float *actions,
                        float *rewards, float *dones, float *obs, uint64_t step_seed, uint64_t reset_seed,
                        const Accounting &acc);

// CartPole's per-env step counters for the rows at `states` (created zeroed on first use)
int cartpole_side(mrl_ctx *ctx, const float *states, int batch, int32_t **out);

// resolves the device address of the file-scope scratch of mrl_clip_grad_norm_static for `device`
// (the current device); idempotent
int clip_static_setup(int device);

inline int grid_for(long n, int block) { return (int)((n + block - 1) / block); }

// Records a phase boundary: the time since the previous mark is charged to `tag`; tag < 0 opens
// a phase without charging anything.  An opening mark that directly follows a closing one reuses
// its event (two events per collection step instead of four), so work that the caller enqueues
// between two rollout steps is charged to the first phase of the second step.
inline void profile_mark(mrl_ctx *ctx, int tag) {
    if (!ctx->profiling || ctx->prof_used >= ctx->prof_events.size()) return;
    if (!ctx->prof_active) {
        ctx->prof_chained = false;
        return;
    }
    if (tag < 0 && ctx->prof_chained) return;
    if (hipEventRecord(ctx->prof_events[ctx->prof_used], ctx->stream) != hipSuccess) return;
    ctx->prof_tags[ctx->prof_used++] = tag;
    ctx->prof_chained = tag >= 0;
}

// Sampled timing (prof_every = k > 1): of every k rollout steps one is timed, and the step before
// it contributes one event, recorded after its last kernel, that opens the timed step's first
// phase.  (An opening event recorded straight after kernels that carry no event of their own is
// not a reliable start: the runtime may resolve it to a time before the last of them ran.)
inline void profile_step_begin(mrl_ctx *ctx) {
    ctx->prof_active = true;
    ctx->prof_open_next = false;
    if (!ctx->profiling || ctx->prof_every <= 1) return;
    const long phase = ctx->prof_step++ % ctx->prof_every;
    ctx->prof_active = phase == 0 && ctx->prof_chained;       // timed only if the step before opened it
    ctx->prof_open_next = phase == ctx->prof_every - 1;
}
inline void profile_step_end(mrl_ctx *ctx) {
    if (ctx->profiling && ctx->prof_open_next && ctx->prof_used < ctx->prof_events.size() &&
        hipEventRecord(ctx->prof_events[ctx->prof_used], ctx->stream) == hipSuccess) {
        ctx->prof_tags[ctx->prof_used++] = -1;
        ctx->prof_chained = true;
    }
    ctx->prof_open_next = false;
    ctx->prof_active = true;
}

}  // namespace mrl

#define MRL_CHECK_ARG(cond, ...)                                   \
    do {                                                           \
        if (!(cond)) return mrl::set_error(MRL_E_ARG, __VA_ARGS__); \
    } while (0)

#define MRL_CHECK_HIP(expr)                                                              \
    do {                                                                                 \
        hipError_t _e = (expr);                                                          \
        if (_e != hipSuccess)                                                            \
            return mrl::set_error(MRL_E_HIP, "%s failed: %s", #expr, hipGetErrorString(_e)); \
    } while (0)

#define MRL_CHECK_LAUNCH() MRL_CHECK_HIP(hipGetLastError())
