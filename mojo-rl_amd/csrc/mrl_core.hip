// Context lifetime and error reporting of libmrl_hip.so.
#include "mrl_host.hpp"
#include "env_lunar.hpp"
#include "env_walkers.hpp"

namespace mrl {

static thread_local char g_error[512] = "";

int set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int grow_workspace(mrl_ctx *ctx, float **buf, size_t *have, size_t need) {
    if (*have >= need) return MRL_OK;
    MRL_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    if (*buf) MRL_CHECK_HIP(hipFree(*buf));
    *buf = nullptr;
    *have = 0;
    MRL_CHECK_HIP(hipMalloc(buf, sizeof(float) * need));
    *have = need;
    return MRL_OK;
}

}  // namespace mrl

extern "C" {

int mrl_version(void) { return 100; }

const char *mrl_last_error(void) { return mrl::g_error; }

// a failed set-up step releases what the steps before it obtained
#define CTX_TRY(expr)                                                                             \
    do {                                                                                          \
        hipError_t _e = (expr);                                                                   \
        if (_e != hipSuccess) {                                                                   \
            mrl_ctx_destroy(c);                                                                   \
            return mrl::set_error(MRL_E_HIP, "mrl_ctx_create: %s failed: %s", #expr, hipGetErrorString(_e)); \
        }                                                                                         \
    } while (0)

int mrl_ctx_create(void *hip_stream, mrl_ctx **out) {
    MRL_CHECK_ARG(out != nullptr, "mrl_ctx_create: out is NULL");
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0)
        return mrl::set_error(MRL_E_HIP, "mrl_ctx_create: no HIP device (%s)", hipGetErrorString(e));
    mrl_ctx *c = new mrl_ctx();        // value-initialised: every pointer starts out null
    c->stream = (hipStream_t)hip_stream;
    c->reduce_scratch_floats = 4096;
    c->prof_every = 1;
    c->prof_active = true;
    c->spin_limit = MRL_DEFAULT_SPIN_LIMIT;
    CTX_TRY(hipGetDevice(&c->device));
    CTX_TRY(hipDeviceGetAttribute(&c->n_cus, hipDeviceAttributeMultiprocessorCount, c->device));
    mrl::ll::Shapes sh = mrl::ll::make_shapes();
    CTX_TRY(hipMalloc(&c->ll_shapes, sizeof(sh)));
    CTX_TRY(hipMemcpy(c->ll_shapes, &sh, sizeof(sh), hipMemcpyHostToDevice));
    mrl::bw::Shapes bs = mrl::bw::make_shapes();
    CTX_TRY(hipMalloc(&c->bw_shapes, sizeof(bs)));
    CTX_TRY(hipMemcpy(c->bw_shapes, &bs, sizeof(bs), hipMemcpyHostToDevice));
    mrl::hc::Shapes hs = mrl::hc::make_shapes();
    CTX_TRY(hipMalloc(&c->hc_shapes, sizeof(hs)));
    CTX_TRY(hipMemcpy(c->hc_shapes, &hs, sizeof(hs), hipMemcpyHostToDevice));
    CTX_TRY(hipMalloc(&c->reduce_scratch, sizeof(float) * c->reduce_scratch_floats));
    CTX_TRY(hipMalloc(&c->upd_scratch, sizeof(float) * 8192));
    CTX_TRY(hipMemset(c->upd_scratch, 0, sizeof(float) * 8192));
    CTX_TRY(hipHostMalloc((void **)&c->sync_error, 64, hipHostMallocDefault));
    *c->sync_error = 0;
    {
        int rc = mrl::clip_static_setup(c->device);
        if (rc != MRL_OK) { mrl_ctx_destroy(c); return rc; }
    }
    *out = c;
    return MRL_OK;
}
#undef CTX_TRY

int mrl_ctx_destroy(mrl_ctx *ctx) {
    if (!ctx) return MRL_OK;
    hipStreamSynchronize(ctx->stream);
    for (auto &kv : ctx->cartpole_steps)
        if (kv.second.owned) hipFree(kv.second.steps);
    if (ctx->ll_shapes) hipFree(ctx->ll_shapes);
    if (ctx->bw_shapes) hipFree(ctx->bw_shapes);
    if (ctx->hc_shapes) hipFree(ctx->hc_shapes);
    if (ctx->reduce_scratch) hipFree(ctx->reduce_scratch);
    if (ctx->upd_scratch) hipFree(ctx->upd_scratch);
    if (ctx->sync_error) hipHostFree(ctx->sync_error);
    if (ctx->mlp_ws) hipFree(ctx->mlp_ws);
    if (ctx->rollout_ws) hipFree(ctx->rollout_ws);
    for (hipEvent_t e : ctx->prof_events) hipEventDestroy(e);
    delete ctx;
    return MRL_OK;
}

int mrl_ctx_synchronize(mrl_ctx *ctx) {
    MRL_CHECK_ARG(ctx != nullptr, "mrl_ctx_synchronize: ctx is NULL");
    MRL_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    if (*(volatile int *)ctx->sync_error != 0) {
        *ctx->sync_error = 0;
        return mrl::set_error(MRL_E_SYNC, "mrl_ctx_synchronize: a kernel gave up waiting at one of its internal "
                              "barriers (limit %u polls); the results of the calls since the last synchronize are void",
                              ctx->spin_limit);
    }
    return MRL_OK;
}

int mrl_ctx_workspace(mrl_ctx *ctx, uint64_t *mlp_floats, uint64_t *rollout_floats) {
    MRL_CHECK_ARG(ctx != nullptr, "mrl_ctx_workspace: ctx is NULL");
    if (mlp_floats) *mlp_floats = ctx->mlp_ws_floats;
    if (rollout_floats) *rollout_floats = ctx->rollout_ws_floats;
    return MRL_OK;
}

int mrl_ctx_reserve(mrl_ctx *ctx, uint64_t mlp_floats, uint64_t rollout_floats) {
    MRL_CHECK_ARG(ctx != nullptr, "mrl_ctx_reserve: ctx is NULL");
    int rc = mrl::grow_workspace(ctx, &ctx->mlp_ws, &ctx->mlp_ws_floats, (size_t)mlp_floats);
    if (rc != MRL_OK) return rc;
    return mrl::grow_workspace(ctx, &ctx->rollout_ws, &ctx->rollout_ws_floats, (size_t)rollout_floats);
}

int mrl_ctx_set_spin_limit(mrl_ctx *ctx, unsigned polls) {
    MRL_CHECK_ARG(ctx != nullptr, "mrl_ctx_set_spin_limit: ctx is NULL");
    ctx->spin_limit = polls == 0 ? MRL_DEFAULT_SPIN_LIMIT : polls;
    return MRL_OK;
}

int mrl_profile_begin(mrl_ctx *ctx, int max_marks) {
    MRL_CHECK_ARG(ctx != nullptr && max_marks > 0, "mrl_profile_begin: bad arguments");
    while ((int)ctx->prof_events.size() < max_marks) {
        hipEvent_t e;
        MRL_CHECK_HIP(hipEventCreate(&e));
        ctx->prof_events.push_back(e);
    }
    ctx->prof_tags.assign(ctx->prof_events.size(), -1);
    ctx->prof_used = 0;
    ctx->prof_chained = false;
    ctx->prof_step = 0;
    ctx->prof_active = true;
    ctx->profiling = true;
    return MRL_OK;
}

int mrl_profile_sample_every(mrl_ctx *ctx, int every) {
    MRL_CHECK_ARG(ctx != nullptr && every >= 1, "mrl_profile_sample_every: bad arguments");
    ctx->prof_every = every;
    return MRL_OK;
}

int mrl_profile_end(mrl_ctx *ctx, int n_phases, double *total_ms, int *counts) {
    MRL_CHECK_ARG(ctx && total_ms && counts && n_phases > 0, "mrl_profile_end: bad arguments");
    ctx->profiling = false;
    MRL_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    for (int i = 0; i < n_phases; ++i) { total_ms[i] = 0.0; counts[i] = 0; }
    for (size_t i = 1; i < ctx->prof_used; ++i) {
        int tag = ctx->prof_tags[i];
        if (tag < 0 || tag >= n_phases) continue;
        float ms = 0.0f;
        MRL_CHECK_HIP(hipEventElapsedTime(&ms, ctx->prof_events[i - 1], ctx->prof_events[i]));
        total_ms[tag] += ms;
        counts[tag] += 1;
    }
    ctx->prof_used = 0;
    return MRL_OK;
}

}  // extern "C"
