// One PPO minibatch update -- the body of the minibatch loop of train_gpu
// (deep_agents/ppo/ppo.mojo:2438-2727, deep_agents/ppo/ppo_continuous.mojo:3000-3260) -- as one
// call that only enqueues: gather, per-minibatch advantage normalisation, actor and critic
// forward, loss gradients, KL test, backward, global-norm clip, Adam (and the log_std clamp).
// The actor and the critic do not depend on each other inside a minibatch, so when both have one
// of the fused shapes they run side by side in every launch, and a row tile never leaves its
// workgroup between the forward pass and the way back: 4 launches per minibatch (forward + loss
// gradients + KL test + backward dx; dW; sum; clip + Adam) instead of about 40.  The minibatch is
// not gathered: the forward reads its rows from the rollout through the indices and the loss
// normalises the advantage with statistics computed ahead (once per epoch for all minibatches).
// Other net shapes go layer by layer: gather + normalise, forward, loss gradients + KL test,
// backward, clip + Adam.
//
// KL early stop: the reference copies the per-sample KL to the host after the actor's loss
// gradient and breaks out of the minibatch and epoch loops when its mean exceeds target_kl.
// Here the mean is tested on the device, by the kernel that applies the update (from the per-tile
// sums that the loss gradients leave; kl_flag[0] is raised and stays raised), and that kernel
// does nothing once the flag is up: the parameters end exactly where
// the reference's break leaves them, without a host round trip.  kl_flag[2] counts the updates
// that were applied, for the host's optimiser step counters.
#include "mrl_host.hpp"
#include "mrl_device.hpp"
#include "mlp3.hpp"
#include "ppo_grads.hpp"

namespace mrl {

constexpr int UTPB = 256;

MRL_DEV float u_wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
template <int NW>
MRL_DEV float u_block_sum(float v, float *smem) {
    v = u_wave_sum(v);
    if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = 0.0f;
#pragma unroll
    for (int k = 0; k < NW; ++k) t += smem[k];
    __syncthreads();
    return t;
}

// ppo_gather_minibatch_kernel (ppo.mojo:135-191) with the per-minibatch advantage normalisation
// (ppo.mojo:2478-2511) done by one extra workgroup: that one gathers the advantages itself and
// writes them normalised, the others copy the remaining fields.
struct GatherArgs {
    const int32_t *idx;
    const float *r_obs, *r_act, *r_adv, *r_ret, *r_logp, *r_val;
    float *mb_obs, *mb_act, *mb_adv, *mb_ret, *mb_logp, *mb_val;
    int mb, obs_dim, act_dim, normalize;
};

__global__ __launch_bounds__(UTPB) void gather_norm_kernel(GatherArgs g) {
    __shared__ float smem[4];
    if (blockIdx.x == gridDim.x - 1) {
        constexpr int PER = 32;   // minibatches up to 8192 samples stay in registers
        if (g.mb <= PER * UTPB) {
            int src[PER];
            float v[PER];
#pragma unroll
            for (int k = 0; k < PER; ++k) {
                const int i = threadIdx.x + k * UTPB;
                src[k] = i < g.mb ? g.idx[i] : -1;
            }
#pragma unroll
            for (int k = 0; k < PER; ++k) v[k] = src[k] >= 0 ? g.r_adv[src[k]] : 0.0f;
            if (g.normalize) {
                float s = 0.0f;
#pragma unroll
                for (int k = 0; k < PER; ++k) s += v[k];
                const float mean = u_block_sum<4>(s, smem) / (float)g.mb;
                float q = 0.0f;
#pragma unroll
                for (int k = 0; k < PER; ++k) {
                    const float d = v[k] - mean;
                    q += src[k] >= 0 ? d * d : 0.0f;
                }
                const float variance = u_block_sum<4>(q, smem) / (float)g.mb;
                const float std = sqrtf(variance + 1e-8f);
#pragma unroll
                for (int k = 0; k < PER; ++k) v[k] = (v[k] - mean) / (std + 1e-8f);
            }
#pragma unroll
            for (int k = 0; k < PER; ++k)
                if (src[k] >= 0) g.mb_adv[threadIdx.x + k * UTPB] = v[k];
            return;
        }
        float s = 0.0f;
        for (int i = threadIdx.x; i < g.mb; i += UTPB) s += g.r_adv[g.idx[i]];
        if (!g.normalize) {
            for (int i = threadIdx.x; i < g.mb; i += UTPB) g.mb_adv[i] = g.r_adv[g.idx[i]];
            return;
        }
        const float mean = u_block_sum<4>(s, smem) / (float)g.mb;
        float q = 0.0f;
        for (int i = threadIdx.x; i < g.mb; i += UTPB) {
            const float d = g.r_adv[g.idx[i]] - mean;
            q += d * d;
        }
        const float variance = u_block_sum<4>(q, smem) / (float)g.mb;
        const float std = sqrtf(variance + 1e-8f);
        for (int i = threadIdx.x; i < g.mb; i += UTPB) g.mb_adv[i] = (g.r_adv[g.idx[i]] - mean) / (std + 1e-8f);
        return;
    }
    const long i = (long)blockIdx.x * UTPB + threadIdx.x;
    const int w = g.obs_dim;
    if (i >= (long)g.mb * w) return;
    const int b = (int)(i / w), c = (int)(i - (long)b * w);
    const long src = g.idx[b];
    g.mb_obs[i] = g.r_obs[src * g.obs_dim + c];
    if (c < g.act_dim) g.mb_act[(long)b * g.act_dim + c] = g.r_act[src * g.act_dim + c];
    if (c == 0) {
        g.mb_ret[b] = g.r_ret[src];
        g.mb_logp[b] = g.r_logp[src];
        g.mb_val[b] = g.r_val[src];
    }
}

// Mean and standard deviation of the advantages of minibatch blockIdx.x (rows idx[k * mb ..]), with
// the arithmetic of the normalising workgroup of gather_norm_kernel: stats[2k] = mean,
// stats[2k + 1] = sqrt(variance + 1e-8).  The fused forward normalises with them on the fly.
__global__ __launch_bounds__(UTPB) void adv_stats_kernel(const int32_t *__restrict__ idx,
                                                         const float *__restrict__ r_adv, int mb,
                                                         float *__restrict__ stats) {
    __shared__ float smem[4];
    constexpr int PER = 32;
    const int32_t *my = idx + (size_t)blockIdx.x * mb;
    float mean, variance;
    if (mb <= PER * UTPB) {
        float v[PER];
        bool in[PER];
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const int i = threadIdx.x + k * UTPB;
            in[k] = i < mb;
            v[k] = in[k] ? r_adv[my[i]] : 0.0f;
        }
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < PER; ++k) s += v[k];
        mean = u_block_sum<4>(s, smem) / (float)mb;
        float q = 0.0f;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const float d = v[k] - mean;
            q += in[k] ? d * d : 0.0f;
        }
        variance = u_block_sum<4>(q, smem) / (float)mb;
    } else {
        float s = 0.0f;
        for (int i = threadIdx.x; i < mb; i += UTPB) s += r_adv[my[i]];
        mean = u_block_sum<4>(s, smem) / (float)mb;
        float q = 0.0f;
        for (int i = threadIdx.x; i < mb; i += UTPB) {
            const float d = r_adv[my[i]] - mean;
            q += d * d;
        }
        variance = u_block_sum<4>(q, smem) / (float)mb;
    }
    if (threadIdx.x == 0) {
        stats[2 * blockIdx.x] = mean;
        stats[2 * blockIdx.x + 1] = sqrtf(variance + 1e-8f);
    }
}

// Actor and critic loss gradients in one launch (grid.y = 0: actor, 1: critic) and the KL test:
// every actor workgroup leaves the sum of its samples' KL estimates, the last one to arrive adds
// them up in workgroup order, compares the mean with target_kl and re-arms the counter.
struct LossArgs {
    const float *actor_out, *mb_logp, *mb_adv, *mb_act, *values, *mb_val, *mb_ret;
    float *g_actor_out, *g_values, *kl;
    float *kl_part;      // [grid.x]
    int *arrived;        // zero between launches
    int32_t *kl_flag;    // nullable: no test
    int mb, A, continuous, clip_value;
    float clip_eps, ent_coef, value_coef, target_kl;
};

__global__ __launch_bounds__(UTPB) void loss_grads_kernel(LossArgs a) {
    __shared__ float smem[4];
    __shared__ int last;
    const int b = blockIdx.x * UTPB + threadIdx.x;
    if (blockIdx.y == 1) {
        if (b < a.mb)
            a.g_values[b] = critic_grad_one(b, a.values, a.mb_val, a.mb_ret, a.mb, a.continuous, a.clip_value,
                                            a.value_coef, a.clip_eps);
        return;
    }
    float kl = 0.0f;
    if (b < a.mb) {
        kl = a.continuous ? actor_grad_gaussian_one(b, a.actor_out, a.mb_logp, a.mb_adv, a.mb_act, a.mb, a.A,
                                                    a.clip_eps, a.ent_coef, a.g_actor_out)
                          : actor_grad_discrete_one(b, a.actor_out, a.mb_logp, a.mb_adv, a.mb_act, a.mb, a.A,
                                                    a.clip_eps, a.ent_coef, a.g_actor_out);
        a.kl[b] = kl;
    }
    if (a.kl_flag == nullptr) return;
    const float s = u_block_sum<4>(kl, smem);
    if (threadIdx.x == 0) {
        __hip_atomic_store(&a.kl_part[blockIdx.x], s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __threadfence();
        last = atomicAdd(a.arrived, 1) == (int)gridDim.x - 1;
    }
    __syncthreads();
    if (!last) return;
    __threadfence();
    float t = 0.0f;
    for (int i = threadIdx.x; i < (int)gridDim.x; i += UTPB)
        t += __hip_atomic_load(&a.kl_part[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    t = u_block_sum<4>(t, smem);
    if (threadIdx.x == 0) {
        const float mean = t / (float)a.mb;
        a.kl_flag[1] = __float_as_int(mean);
        if (mean > a.target_kl) a.kl_flag[0] = 1;
        *a.arrived = 0;
    }
}

struct AdamNet {
    float *p, *g;
    float2 *state;
    int n;
    float lr, bc1, bc2;
    int clamp_off, clamp_n;   // log_std slice to clamp to [-5, 2] after the step (clamp_n = 0: none)
};
struct AdamNets { AdamNet n[2]; };

// partial[net][block] = sum of g^2 over the block's grid-stride slice; grid = (nb, nets)
__global__ __launch_bounds__(UTPB) void sq_partial2_kernel(AdamNets nets, float *__restrict__ partial) {
    __shared__ float smem[4];
    const AdamNet &a = nets.n[blockIdx.y];
    float s = 0.0f;
    for (long i = (long)blockIdx.x * UTPB + threadIdx.x; i < a.n; i += (long)gridDim.x * UTPB) s += a.g[i] * a.g[i];
    s = u_block_sum<4>(s, smem);
    if (threadIdx.x == 0) partial[blockIdx.y * gridDim.x + blockIdx.x] = s;
}

// global-norm clip (ppo.mojo:382-534; actor and critic separately) + Adam (adam.mojo:52-105)
// + log_std clamp (kernels.mojo:842-873); grid = (blocks, nets).  Does nothing once stop[0] != 0.
// kl_part != nullptr: the KL early-stop test of this minibatch has not been made yet: kl_part[0 .. kl_n)
// hold the row tiles' sums of the per-sample estimates.  Every workgroup adds them up in the same order,
// so all of them come to the same verdict; workgroup (0, 0) records it (stop[0] raised and sticky,
// stop[1] = the mean's bits).
__global__ __launch_bounds__(UTPB) void clip_adam2_kernel(AdamNets nets, const float *__restrict__ partial,
                                                          int nb, int part_stride, float max_norm, float beta1,
                                                          float beta2,
                                                          float omb1, float omb2, float eps,
                                                          int32_t *__restrict__ stop,
                                                          const float *__restrict__ kl_part, int kl_n, int kl_mb,
                                                          float target_kl) {
    __shared__ float smem[4];
    __shared__ float scale_s;
    __shared__ int stop_s;
    if (stop != nullptr && stop[0] != 0) return;
    if (stop != nullptr && kl_part != nullptr) {
        if (threadIdx.x < 64) {
            float sum = 0.0f;
            for (int i = threadIdx.x; i < kl_n; i += 64) sum += kl_part[i];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
            if (threadIdx.x == 0) {
                const float mean = sum / (float)kl_mb;
                stop_s = mean > target_kl;
                if (blockIdx.x == 0 && blockIdx.y == 0) {
                    stop[1] = __float_as_int(mean);
                    if (mean > target_kl) stop[0] = 1;
                }
            }
        }
        __syncthreads();
        if (stop_s) return;
    }
    const AdamNet &a = nets.n[blockIdx.y];
    float scale = 1.0f;
    if (max_norm > 0.0f) {
        float s = 0.0f;
        for (int i = threadIdx.x; i < nb; i += UTPB) s += partial[blockIdx.y * part_stride + i];
        s = u_block_sum<4>(s, smem);
        if (threadIdx.x == 0) {
            const float norm = sqrtf(s);
            scale_s = norm > max_norm ? max_norm / (norm + 1e-8f) : 1.0f;
        }
        __syncthreads();
        scale = scale_s;
    }
    if (stop != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) stop[2] = stop[2] + 1;
    const int i = blockIdx.x * UTPB + threadIdx.x;
    if (i >= a.n) return;
    const float gi = a.g[i] * scale;
    a.g[i] = gi;
    const float2 mv = a.state[i];
    const float m_new = beta1 * mv.x + omb1 * gi;
    const float v_new = beta2 * mv.y + omb2 * gi * gi;
    a.state[i] = make_float2(m_new, v_new);
    const float m_hat = m_new / a.bc1, v_hat = v_new / a.bc2;
    float p = a.p[i] - a.lr * m_hat / (sqrtf(v_hat) + eps);
    if (i >= a.clamp_off && i < a.clamp_off + a.clamp_n) {
        if (p < -5.0f) p = -5.0f;
        else if (p > 2.0f) p = 2.0f;
    }
    a.p[i] = p;
}

}  // namespace mrl

using namespace mrl;

extern "C" {

static int update_check(const mrl_update *u, const char *who) {
    MRL_CHECK_ARG(u != nullptr, "%s: descriptor is NULL", who);
    MRL_CHECK_ARG(u->minibatch > 0 && u->obs_dim > 0 && u->act_width > 0, "%s: bad sizes", who);
    MRL_CHECK_ARG(u->actor_params && u->critic_params && u->actor_grads && u->critic_grads && u->actor_state &&
                      u->critic_state, "%s: NULL parameter / gradient / optimiser buffer", who);
    MRL_CHECK_ARG(u->r_obs && u->r_actions && u->r_log_probs && u->r_values && u->advantages && u->returns,
                  "%s: NULL rollout buffer", who);
    MRL_CHECK_ARG(u->mb_obs && u->mb_actions && u->mb_adv && u->mb_ret && u->mb_logp && u->mb_val &&
                      u->actor_out && u->values && u->g_actor_out && u->g_values && u->kl && u->actor_cache &&
                      u->critic_cache, "%s: NULL minibatch buffer", who);
    MRL_CHECK_ARG(u->target_kl <= 0.0f || u->kl_flag != nullptr, "%s: target_kl needs kl_flag", who);
    const int head = mrl_mlp_out_dim(&u->actor);
    MRL_CHECK_ARG(head > 0 && mrl_mlp_out_dim(&u->critic) == 1, "%s: bad actor / critic description", who);
    const bool gauss = u->actor.layers[u->actor.n_layers - 1].kind == MRL_STOCHASTIC_ACTOR;
    MRL_CHECK_ARG(gauss == (u->continuous != 0), "%s: a continuous agent needs a StochasticActor head (and only it)",
                  who);
    MRL_CHECK_ARG(!gauss || head == 2 * u->act_width, "%s: act_width does not match the actor head", who);
    MRL_CHECK_ARG(gauss || u->act_width == 1, "%s: a discrete agent stores one float per action", who);
    MRL_CHECK_ARG(u->actor.layers[0].in_dim == u->obs_dim && u->critic.layers[0].in_dim == u->obs_dim,
                  "%s: nets do not read obs_dim inputs", who);
    return MRL_OK;
}

// floats of ctx->upd_scratch: KL partials, their arrival counter, sum-of-squares partials, and the
// advantage statistics of up to STATS_MAX minibatches
constexpr int SCR_KL = 0, SCR_ARRIVED = 1024, SCR_SQ = 2048, SCR_STATS = 4096, STATS_MAX = 2048;

static bool update_paired(const mrl_update *u) {
    return mlp3_pair_fusable(u->actor, u->critic) && reinterpret_cast<uintptr_t>(u->actor_params) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(u->critic_params) % 16 == 0 && (u->minibatch + 31) / 32 <= 1024;
}

// stats: {mean, std} of this minibatch's advantages on the device, already enqueued (paired nets
// only); null: worked out here
static int update_minibatch(mrl_ctx *ctx, const mrl_update *u, const int32_t *indices, int actor_t, int critic_t,
                            const float *stats) {
    int rc;
    const int mb = u->minibatch, head = mrl_mlp_out_dim(&u->actor);
    const int Pa = mrl_mlp_param_size(&u->actor), Pc = mrl_mlp_param_size(&u->critic);
    const bool cont = u->continuous != 0;
    const bool paired = update_paired(u);

    if (paired && u->norm_adv_per_minibatch && stats == nullptr) {
        float *st = ctx->upd_scratch + SCR_STATS;
        hipLaunchKernelGGL(adv_stats_kernel, dim3(1), dim3(UTPB), 0, ctx->stream, indices, u->advantages, mb, st);
        MRL_CHECK_LAUNCH();
        stats = st;
    }
    if (!paired) {
        GatherArgs g{indices, u->r_obs, u->r_actions, u->advantages, u->returns, u->r_log_probs, u->r_values,
                     u->mb_obs, u->mb_actions, u->mb_adv, u->mb_ret, u->mb_logp, u->mb_val,
                     mb, u->obs_dim, u->act_width, u->norm_adv_per_minibatch};
        MRL_CHECK_ARG(u->act_width <= u->obs_dim, "mrl_ppo_update_minibatch: action wider than observation");
        hipLaunchKernelGGL(gather_norm_kernel, dim3(grid_for((long)mb * u->obs_dim, UTPB) + 1), dim3(UTPB), 0,
                           ctx->stream, g);
        MRL_CHECK_LAUNCH();
    }

    const mrl_mlp_desc *descs[2] = {&u->actor, &u->critic};
    Mlp3Nets io{};
    io.n[0].x = u->mb_obs; io.n[0].params = u->actor_params; io.n[0].out = u->actor_out; io.n[0].cache = u->actor_cache;
    io.n[1].x = u->mb_obs; io.n[1].params = u->critic_params; io.n[1].out = u->values; io.n[1].cache = u->critic_cache;
    FwdLoss fl{};
    if (paired) {
        // both nets go forward straight from the rollout rows, on to their loss gradients and the KL
        // test and back again in one launch per row tile (mlp3_backward_n below)
        fl.idx = indices;
        fl.r_obs = u->r_obs; fl.r_act = u->r_actions; fl.r_adv = u->advantages; fl.r_ret = u->returns;
        fl.r_logp = u->r_log_probs; fl.r_val = u->r_values;
        fl.adv_stats = u->norm_adv_per_minibatch ? stats : nullptr;
        fl.g_actor_out = u->g_actor_out; fl.g_values = u->g_values; fl.kl = u->kl;
        fl.kl_part = ctx->upd_scratch + SCR_KL;
        fl.kl_flag = u->target_kl > 0.0f ? u->kl_flag : nullptr;
        fl.mb = mb; fl.A = cont ? u->act_width : head; fl.continuous = cont ? 1 : 0;
        fl.clip_value = u->clip_value ? 1 : 0;
        fl.clip_eps = u->clip_epsilon; fl.ent_coef = u->entropy_coef; fl.value_coef = u->value_loss_coef;
        fl.target_kl = u->target_kl;
    } else {
        rc = mrl_mlp_forward(ctx, &u->actor, mb, u->mb_obs, u->actor_params, u->actor_out, u->actor_cache);
        if (rc) return rc;
        rc = mrl_mlp_forward(ctx, &u->critic, mb, u->mb_obs, u->critic_params, u->values, u->critic_cache);
        if (rc) return rc;
    }

    if (!paired) {
        const int nblk = grid_for(mb, UTPB);
        const bool test = u->target_kl > 0.0f && nblk <= 1024;
        LossArgs a{u->actor_out, u->mb_logp, u->mb_adv, u->mb_actions, u->values, u->mb_val, u->mb_ret,
                   u->g_actor_out, u->g_values, u->kl, ctx->upd_scratch,
                   reinterpret_cast<int *>(ctx->upd_scratch + 1024), test ? u->kl_flag : nullptr,
                   mb, cont ? u->act_width : head, cont ? 1 : 0, u->clip_value ? 1 : 0,
                   u->clip_epsilon, u->entropy_coef, u->value_loss_coef, u->target_kl};
        hipLaunchKernelGGL(loss_grads_kernel, dim3(nblk, 2), dim3(UTPB), 0, ctx->stream, a);
        MRL_CHECK_LAUNCH();
        if (u->target_kl > 0.0f && !test) {
            rc = mrl_kl_check(ctx, u->kl, mb, u->target_kl, u->kl_flag);
            if (rc) return rc;
        }
    }

    io.n[0].grad_out = u->g_actor_out;
    io.n[1].grad_out = u->g_values;
    float *grads[2] = {u->actor_grads, u->critic_grads};
    int sq_blocks = 0;   // > 0: the backward pass already left the sum-of-squares partials
    if (paired) {
        float *ws = nullptr;
        rc = mlp_ensure_ws(ctx, mlp3_backward_ws(descs, 2, mb), &ws);
        if (rc) return rc;
        rc = mlp3_backward_n(ctx, descs, 2, mb, io, grads, ws,
                             u->max_grad_norm > 0.0f ? ctx->upd_scratch + SCR_SQ : nullptr, &sq_blocks, &fl);
        if (rc) return rc;
    } else {
        rc = mrl_mlp_backward(ctx, &u->actor, mb, u->g_actor_out, u->actor_params, u->actor_cache, u->actor_grads,
                              nullptr);
        if (rc) return rc;
        rc = mrl_mlp_backward(ctx, &u->critic, mb, u->g_values, u->critic_params, u->critic_cache, u->critic_grads,
                              nullptr);
        if (rc) return rc;
    }

    AdamNets an{};
    auto fill = [&](AdamNet &a, float *p, float *g, float *st, int n, double lr, int t) {
        a.p = p; a.g = g; a.state = reinterpret_cast<float2 *>(st); a.n = n; a.lr = (float)lr;
        // bias corrections in fp64 then rounded, as the host code of the reference does
        a.bc1 = (float)(1.0 - pow(u->beta1, (double)t));
        a.bc2 = (float)(1.0 - pow(u->beta2, (double)t));
        a.clamp_off = 0; a.clamp_n = 0;
    };
    fill(an.n[0], u->actor_params, u->actor_grads, u->actor_state, Pa, u->actor_lr, actor_t);
    fill(an.n[1], u->critic_params, u->critic_grads, u->critic_state, Pc, u->critic_lr, critic_t);
    if (cont) { an.n[0].clamp_off = Pa - u->act_width; an.n[0].clamp_n = u->act_width; }
    const int nmax = std::max(Pa, Pc);
    int nb = sq_blocks, stride = 1024;
    const float *part = ctx->upd_scratch + 2048;
    if (u->max_grad_norm > 0.0f && sq_blocks == 0) {
        nb = std::min(256, grid_for(nmax, UTPB));
        stride = nb;
        float *p2 = ctx->reduce_scratch + 1024;   // [2][nb], nb <= 256
        hipLaunchKernelGGL(sq_partial2_kernel, dim3(nb, 2), dim3(UTPB), 0, ctx->stream, an, p2);
        part = p2;
    }
    hipLaunchKernelGGL(clip_adam2_kernel, dim3(grid_for(nmax, UTPB), 2), dim3(UTPB), 0, ctx->stream, an, part, nb,
                       stride, u->max_grad_norm, (float)u->beta1, (float)u->beta2, (float)(1.0 - u->beta1),
                       (float)(1.0 - u->beta2), (float)u->eps, u->target_kl > 0.0f ? u->kl_flag : nullptr,
                       paired && u->target_kl > 0.0f ? ctx->upd_scratch + SCR_KL : nullptr, grid_for(mb, 32), mb,
                       u->target_kl);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_ppo_update_minibatch(mrl_ctx *ctx, const mrl_update *u, const int32_t *indices, int actor_t,
                             int critic_t) {
    MRL_CHECK_ARG(ctx != nullptr, "mrl_ppo_update_minibatch: ctx is NULL");
    int rc = update_check(u, "mrl_ppo_update_minibatch");
    if (rc) return rc;
    MRL_CHECK_ARG(indices != nullptr && actor_t >= 1 && critic_t >= 1,
                  "mrl_ppo_update_minibatch: need indices and step counts >= 1");
    return update_minibatch(ctx, u, indices, actor_t, critic_t, nullptr);
}

int mrl_minibatch_adv_stats(mrl_ctx *ctx, const int32_t *indices, const float *advantages, int minibatch,
                            int n_minibatches, float *stats) {
    MRL_CHECK_ARG(ctx != nullptr, "mrl_minibatch_adv_stats: ctx is NULL");
    MRL_CHECK_ARG(minibatch > 0 && n_minibatches >= 0, "mrl_minibatch_adv_stats: bad sizes");
    if (n_minibatches == 0) return MRL_OK;
    MRL_CHECK_ARG(indices && advantages && stats, "mrl_minibatch_adv_stats: NULL buffer");
    // the launch mrl_ppo_update_epoch makes ahead of its minibatches, into the caller's buffer
    hipLaunchKernelGGL(adv_stats_kernel, dim3(n_minibatches), dim3(UTPB), 0, ctx->stream, indices, advantages,
                       minibatch, stats);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mrl_ppo_update_epoch(mrl_ctx *ctx, const mrl_update *u, const int32_t *indices, int n_minibatches,
                         int actor_t0, int critic_t0) {
    MRL_CHECK_ARG(ctx != nullptr, "mrl_ppo_update_epoch: ctx is NULL");
    int rc = update_check(u, "mrl_ppo_update_epoch");
    if (rc) return rc;
    MRL_CHECK_ARG(n_minibatches >= 0 && actor_t0 >= 0 && critic_t0 >= 0, "mrl_ppo_update_epoch: negative count");
    MRL_CHECK_ARG(n_minibatches == 0 || indices != nullptr, "mrl_ppo_update_epoch: indices is NULL");
    const bool ahead = update_paired(u) && u->norm_adv_per_minibatch;
    for (int k0 = 0; k0 < n_minibatches; k0 += STATS_MAX) {
        const int n = std::min(STATS_MAX, n_minibatches - k0);
        float *stats = ctx->upd_scratch + SCR_STATS;
        if (ahead) {   // the advantage statistics of all these minibatches in one launch
            hipLaunchKernelGGL(adv_stats_kernel, dim3(n), dim3(UTPB), 0, ctx->stream,
                               indices + (size_t)k0 * u->minibatch, u->advantages, u->minibatch, stats);
            MRL_CHECK_LAUNCH();
        }
        for (int k = k0; k < k0 + n; ++k) {
            rc = update_minibatch(ctx, u, indices + (size_t)k * u->minibatch, actor_t0 + k + 1, critic_t0 + k + 1,
                                  ahead ? stats + 2 * (k - k0) : nullptr);
            if (rc) return rc;
        }
    }
    return MRL_OK;
}

}  // extern "C"
