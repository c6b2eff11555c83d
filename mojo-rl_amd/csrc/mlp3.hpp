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
};
struct Mlp3Nets { Mlp3Net n[2]; };

bool mlp3_fusable(const mrl_mlp_desc &d, int *H, int *act, bool *gauss);
bool mlp3_pair_fusable(const mrl_mlp_desc &a, const mrl_mlp_desc &b);
int mlp3_forward(mrl_ctx *ctx, const mrl_mlp_desc &d, int batch, const float *in, const float *params,
                 float *out, float *cache);
int mlp3_forward_n(mrl_ctx *ctx, const mrl_mlp_desc *const *descs, int n_nets, int batch, Mlp3Nets io);
size_t mlp3_backward_ws(const mrl_mlp_desc *const *descs, int n_nets, int batch);
int mlp3_backward(mrl_ctx *ctx, const mrl_mlp_desc &d, int batch, const float *grad_out, const float *params,
                  const float *cache, float *grads, float *ws);
// sq_part (nullable): receives per-block sums of squares of the gradients, [net * 1024 + block];
// *sq_blocks = number of blocks written (0 when none were)
int mlp3_backward_n(mrl_ctx *ctx, const mrl_mlp_desc *const *descs, int n_nets, int batch, Mlp3Nets io,
                    float *const *grads, float *ws, float *sq_part, int *sq_blocks);
// grows the context's MLP workspace to at least `floats`
int mlp_ensure_ws(mrl_ctx *ctx, size_t floats, float **out);

}  // namespace mrl
