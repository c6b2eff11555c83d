// Host-side interface of the fused three-layer MLP kernels (mrl_mlp3.hip).
#pragma once
#include "mrl_host.hpp"

namespace mrl {

// one net's buffers for the fused kernels; fields a call does not need stay null
struct Mlp3Net {
    const float *x;          // forward: input [B, IN]
    const float *params;
    float *out;              // forward: [B, A] or [B, 2A]
    float *cache;            // forward: written when non-null; backward: read
    const float *grad_out;   // backward
    float *g1, *g0, *ls_part, *db_part, *thin_part;  // backward workspace (set by the host function)
    int A, gauss;            // set by the host function from the description
    int thin_stride;         // floats per row tile in thin_part: IN H + H A, + H H where the tiles carry dW1 too
};
struct Mlp3Nets { Mlp3Net n[2]; };

// PPO tail of a paired forward (net 0 = actor, net 1 = critic) over minibatch rows that are still
// where the rollout left them: the forward reads its input rows through `idx`, and every row tile
// goes straight on to its loss gradients (deep_agents/ppo/ppo.mojo:285-378, 538-633;
// kernels.mojo:230-486) and to its share of the KL early-stop test, so that neither a gather nor a
// loss launch is needed.  enabled = 0: plain forward.
struct FwdLoss {
    int enabled;
    const int32_t *idx;                                   // [mb] rollout rows of the minibatch
    const float *r_obs, *r_act, *r_adv, *r_ret, *r_logp, *r_val;
    const float *adv_stats;                               // {mean, std} of the minibatch's advantages; null: as they are
    float *g_actor_out, *g_values, *kl;                   // [mb, head], [mb], [mb]
    float *kl_part;                                       // [row tiles] sums of the tiles' KL estimates, for the test
    int32_t *kl_flag;                                     // null: no test (nothing is left in kl_part)
    int mb, A, continuous, clip_value;                    // A = actions (discrete) or action width (continuous)
    float clip_eps, ent_coef, value_coef, target_kl;
};

bool mlp3_fusable(const mrl_mlp_desc &d, int *H, int *act, bool *gauss);
bool mlp3_pair_fusable(const mrl_mlp_desc &a, const mrl_mlp_desc &b);
int mlp3_forward(mrl_ctx *ctx, const mrl_mlp_desc &d, int batch, const float *in, const float *params,
                 float *out, float *cache);
int mlp3_forward_n(mrl_ctx *ctx, const mrl_mlp_desc *const *descs, int n_nets, int batch, Mlp3Nets io,
                   const FwdLoss *loss = nullptr);
size_t mlp3_backward_ws(const mrl_mlp_desc *const *descs, int n_nets, int batch);
int mlp3_backward(mrl_ctx *ctx, const mrl_mlp_desc &d, int batch, const float *grad_out, const float *params,
                  const float *cache, float *grads, float *ws);
// sq_part (nullable): receives per-block sums of squares of the gradients, [net * 1024 + block];
// *sq_blocks = number of blocks written (0 when none were)
// fused (nullable): the nets have not gone forward yet -- one kernel per row tile runs forward
// (inputs read through fused->idx, io.n[i].out written, h1 into the cache's c1 rows), loss
// gradients and the way back, in place of a forward launch, a loss launch and the dx launch
int mlp3_backward_n(mrl_ctx *ctx, const mrl_mlp_desc *const *descs, int n_nets, int batch, Mlp3Nets io,
                    float *const *grads, float *ws, float *sq_part, int *sq_blocks, const FwdLoss *fused = nullptr);
// grows the context's MLP workspace to at least `floats`
int mlp_ensure_ws(mrl_ctx *ctx, size_t floats, float **out);

}  // namespace mrl
