// MLP forward / backward on the fp32 matrix cores (v_mfma_f32_32x32x2_f32).
//
// One layer of the reference (deep_rl/model/{linear,linear_relu,linear_tanh,
// stochastic_actor}.mojo) is  y = act(x W + b)  with W row-major [in, out] followed by b in
// the flat parameter vector, and its backward is
//     g' = g * act'(cache),  dx = g' W^T,  dW = x^T g',  db = sum_b g'.
// Three kernels cover it for any sizes (edges are zero-padded into the 32x32 tiles):
//   linear_fwd_kernel    Y[M,N]   = act(X[M,K] W[K,N] + b)         (+ cache writes)
//   linear_bwd_dx_kernel dX[M,K]  = G'[M,N] W^T
//   linear_bwd_dw_kernel [dW; db] = [X | 1]^T G'    split over the batch, then summed
// The last one appends a column of ones to X, so that the bias gradient falls out as row K of
// the product and [dW | db] is written as one contiguous [(K+1), N] block -- exactly the
// reference's gradient layout.
//
// Block = 256 lanes = 4 wavefronts; block tile 64x64, each wavefront owns one 32x32
// accumulator tile; operands go HBM/L2 -> LDS in k-chunks of 32, stored k-major so that the
// 64 lanes of an MFMA operand read are consecutive words.
#include "mrl_host.hpp"
#include "mrl_device.hpp"
#include "mlp3.hpp"

namespace mrl {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BM = 64, BN = 64, KC = 32;
constexpr int LDS_LD = 65;  // odd leading dimension: transposed stores spread over banks

enum { ACT_NONE = 0, ACT_RELU = 1, ACT_TANH = 2 };

MRL_DEV void mfma_chunk(const float *As, const float *Bs, int wr, int wc, int lane, floatx16 &acc) {
    const int half = lane >> 5, l31 = lane & 31;
#pragma unroll
    for (int kk = 0; kk < KC; kk += 2) {
        float a = As[(kk + half) * LDS_LD + 32 * wr + l31];
        float b = Bs[(kk + half) * LDS_LD + 32 * wc + l31];
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
    }
}

// accumulator element v of lane `lane` sits at (row, col) of the 32x32 tile:
MRL_DEV int acc_row(int v, int lane) { return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3); }
MRL_DEV int acc_col(int lane) { return lane & 31; }

// derivative of the layer's own activation, from what the forward cached at [.. | K + n]
template <int ACT>
MRL_DEV float act_mask(const float *cache, int cs, int k_in, long row, int n) {
    if (ACT == ACT_RELU) return cache[row * cs + k_in + n] > 0.0f ? 1.0f : 0.0f;
    if (ACT == ACT_TANH) {
        float y = cache[row * cs + k_in + n];
        return 1.0f - y * y;
    }
    return 1.0f;
}

// Y = act(X W + b).  cache (nullable), row stride cs: [x (K) | pre-activation (ReLU) or
// output (tanh) (N)]; for ACT_NONE only x is cached.
template <int ACT>
__global__ __launch_bounds__(256) void linear_fwd_kernel(const float *__restrict__ X, int ldx,
                                                         const float *__restrict__ W,
                                                         const float *__restrict__ bias,
                                                         float *__restrict__ Y, int ldy,
                                                         float *__restrict__ cache, int cs, int M,
                                                         int K, int N) {
    __shared__ float As[KC * LDS_LD];
    __shared__ float Bs[KC * LDS_LD];
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wr = w >> 1, wc = w & 1;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    floatx16 acc = {0};
    const int arow = t >> 2, akseg = (t & 3) * 8;
    const int bk = t >> 3, bnseg = (t & 7) * 8;
    for (int k0 = 0; k0 < K; k0 += KC) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int k = k0 + akseg + i;
            long row = m0 + arow;
            float v = (row < M && k < K) ? X[row * ldx + k] : 0.0f;
            As[(akseg + i) * LDS_LD + arow] = v;
            if (cache != nullptr && blockIdx.x == 0 && row < M && k < K) cache[row * cs + k] = v;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int k = k0 + bk, n = n0 + bnseg + i;
            Bs[bk * LDS_LD + bnseg + i] = (k < K && n < N) ? W[(long)k * N + n] : 0.0f;
        }
        __syncthreads();
        mfma_chunk(As, Bs, wr, wc, lane, acc);
        __syncthreads();
    }
    const int col = n0 + 32 * wc + acc_col(lane);
    if (col < N) {
        const float b = bias[col];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            long row = m0 + 32 * wr + acc_row(v, lane);
            if (row >= M) continue;
            float pre = acc[v] + b;
            float y = pre;
            if (ACT == ACT_RELU) y = pre > 0.0f ? pre : 0.0f;
            if (ACT == ACT_TANH) y = tanh_mlp(pre);
            Y[row * ldy + col] = y;
            if (cache != nullptr) {
                if (ACT == ACT_RELU) cache[row * cs + K + col] = pre;
                if (ACT == ACT_TANH) cache[row * cs + K + col] = y;
            }
        }
    }
}

// state-independent log_std of the Gaussian head, clamped to [-5, 2], broadcast to every row
__global__ __launch_bounds__(256) void actor_log_std_kernel(const float *__restrict__ log_std,
                                                            float *__restrict__ Y, int M, int A) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long)M * A) return;
    long row = i / A;
    int j = (int)(i - row * A);
    float v = log_std[j];
    if (v < -5.0f) v = -5.0f;
    else if (v > 2.0f) v = 2.0f;
    Y[row * 2 * A + A + j] = v;
}

// dX[M,K] = (G * act')[M,N] W^T
template <int ACT>
__global__ __launch_bounds__(256) void linear_bwd_dx_kernel(const float *__restrict__ G, int ldg,
                                                            const float *__restrict__ W,
                                                            const float *__restrict__ cache, int cs,
                                                            float *__restrict__ dX, int M, int K,
                                                            int N) {
    __shared__ float As[KC * LDS_LD];
    __shared__ float Bs[KC * LDS_LD];
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wr = w >> 1, wc = w & 1;
    const int m0 = blockIdx.y * BM, j0 = blockIdx.x * BN;  // j: column of dX = input index
    floatx16 acc = {0};
    const int arow = t >> 2, anseg = (t & 3) * 8;
    const int bj = t >> 2, bnseg = (t & 3) * 8;
    for (int n0 = 0; n0 < N; n0 += KC) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int n = n0 + anseg + i;
            long row = m0 + arow;
            float v = 0.0f;
            if (row < M && n < N) v = G[row * ldg + n] * act_mask<ACT>(cache, cs, K, row, n);
            As[(anseg + i) * LDS_LD + arow] = v;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int n = n0 + bnseg + i, j = j0 + bj;
            Bs[(bnseg + i) * LDS_LD + bj] = (j < K && n < N) ? W[(long)j * N + n] : 0.0f;
        }
        __syncthreads();
        mfma_chunk(As, Bs, wr, wc, lane, acc);
        __syncthreads();
    }
    const int col = j0 + 32 * wc + acc_col(lane);
    if (col < K) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            long row = m0 + 32 * wr + acc_row(v, lane);
            if (row < M) dX[row * K + col] = acc[v];
        }
    }
}

// partial[z][(K+1), N] = [X | 1]^T (G * act') over the rows of batch slice z
template <int ACT>
__global__ __launch_bounds__(256) void linear_bwd_dw_kernel(const float *__restrict__ Xc, int cs,
                                                            const float *__restrict__ G, int ldg,
                                                            float *__restrict__ partial, int M,
                                                            int K, int N, int rows_per_split) {
    __shared__ float As[KC * LDS_LD];
    __shared__ float Bs[KC * LDS_LD];
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wr = w >> 1, wc = w & 1;
    const int i0 = blockIdx.y * BM, j0 = blockIdx.x * BN, z = blockIdx.z;
    const long b_begin = (long)z * rows_per_split;
    long b_end = b_begin + rows_per_split;
    if (b_end > M) b_end = M;
    floatx16 acc = {0};
    const int bb = t >> 3, seg = (t & 7) * 8;
    for (long b0 = b_begin; b0 < b_end; b0 += KC) {
        const long b = b0 + bb;
        const bool inb = b < b_end;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int ii = i0 + seg + i;
            float v = 0.0f;
            if (inb) {
                if (ii < K) v = Xc[b * cs + ii];
                else if (ii == K) v = 1.0f;
            }
            As[bb * LDS_LD + seg + i] = v;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int j = j0 + seg + i;
            float v = 0.0f;
            if (inb && j < N) v = G[b * ldg + j] * act_mask<ACT>(Xc, cs, K, b, j);
            Bs[bb * LDS_LD + seg + i] = v;
        }
        __syncthreads();
        mfma_chunk(As, Bs, wr, wc, lane, acc);
        __syncthreads();
    }
    const int col = j0 + 32 * wc + acc_col(lane);
    if (col < N) {
        float *out = partial + (long)z * (K + 1) * N;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            int row = i0 + 32 * wr + acc_row(v, lane);
            if (row <= K) out[(long)row * N + col] = acc[v];
        }
    }
}

__global__ __launch_bounds__(256) void sum_partials_kernel(const float *__restrict__ partial,
                                                           float *__restrict__ out, int n,
                                                           int splits) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = 0.0f;
    for (int z = 0; z < splits; ++z) s += partial[(long)z * n + i];
    out[i] = s;
}

// d_log_std[j] = sum_b G[b, A + j]
__global__ __launch_bounds__(256) void column_sum_kernel(const float *__restrict__ G, int ldg,
                                                         int col0, int M, float *__restrict__ out) {
    __shared__ float red[256];
    const int j = blockIdx.x, t = threadIdx.x;
    float s = 0.0f;
    for (long b = t; b < M; b += 256) s += G[b * ldg + col0 + j];
    red[t] = s;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) {
        if (t < st) red[t] += red[t + st];
        __syncthreads();
    }
    if (t == 0) out[j] = red[0];
}

// ----------------------------------------------------------------------------- host side

static int layer_out_dim(const mrl_layer &l) {
    return l.kind == MRL_STOCHASTIC_ACTOR ? 2 * l.out_dim : l.out_dim;
}
static int layer_param_size(const mrl_layer &l) {
    int p = l.in_dim * l.out_dim + l.out_dim;
    return l.kind == MRL_STOCHASTIC_ACTOR ? p + l.out_dim : p;
}
static int layer_cache_size(const mrl_layer &l) {
    return (l.kind == MRL_LINEAR || l.kind == MRL_STOCHASTIC_ACTOR) ? l.in_dim : l.in_dim + l.out_dim;
}

static int check_desc(const mrl_mlp_desc *d, const char *who) {
    MRL_CHECK_ARG(d != nullptr, "%s: desc is NULL", who);
    MRL_CHECK_ARG(d->n_layers >= 1 && d->n_layers <= MRL_MAX_LAYERS, "%s: n_layers %d out of range",
                  who, d->n_layers);
    for (int i = 0; i < d->n_layers; ++i) {
        const mrl_layer &l = d->layers[i];
        MRL_CHECK_ARG(l.kind >= MRL_LINEAR && l.kind <= MRL_STOCHASTIC_ACTOR, "%s: layer %d kind %d",
                      who, i, l.kind);
        MRL_CHECK_ARG(l.in_dim > 0 && l.out_dim > 0, "%s: layer %d has a non-positive size", who, i);
        if (i > 0)
            MRL_CHECK_ARG(l.in_dim == layer_out_dim(d->layers[i - 1]),
                          "%s: layer %d in_dim %d != previous out_dim %d", who, i, l.in_dim,
                          layer_out_dim(d->layers[i - 1]));
        MRL_CHECK_ARG(l.kind != MRL_STOCHASTIC_ACTOR || i == d->n_layers - 1,
                      "%s: the stochastic actor head must be the last layer", who);
    }
    return MRL_OK;
}

// grows the context's MLP workspace (activations between layers, split-K partials)
static int ensure_ws(mrl_ctx *ctx, size_t floats, float **out) {
    int rc = grow_workspace(ctx, &ctx->mlp_ws, &ctx->mlp_ws_floats, floats);
    *out = ctx->mlp_ws;
    return rc;
}

template <int ACT>
static void launch_fwd(hipStream_t s, const float *X, int ldx, const float *W, const float *b,
                       float *Y, int ldy, float *cache, int cs, int M, int K, int N) {
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    hipLaunchKernelGGL(linear_fwd_kernel<ACT>, grid, dim3(256), 0, s, X, ldx, W, b, Y, ldy, cache, cs,
                       M, K, N);
}

int mlp_ensure_ws(mrl_ctx *ctx, size_t floats, float **out) { return ensure_ws(ctx, floats, out); }

}  // namespace mrl

using namespace mrl;

extern "C" {

int mrl_mlp_param_size(const mrl_mlp_desc *d) {
    int rc = check_desc(d, "mrl_mlp_param_size");
    if (rc) return rc;
    int s = 0;
    for (int i = 0; i < d->n_layers; ++i) s += layer_param_size(d->layers[i]);
    return s;
}

int mrl_mlp_cache_size(const mrl_mlp_desc *d) {
    int rc = check_desc(d, "mrl_mlp_cache_size");
    if (rc) return rc;
    int s = 0;
    for (int i = 0; i < d->n_layers; ++i) s += layer_cache_size(d->layers[i]);
    return s;
}

int mrl_mlp_out_dim(const mrl_mlp_desc *d) {
    int rc = check_desc(d, "mrl_mlp_out_dim");
    if (rc) return rc;
    return layer_out_dim(d->layers[d->n_layers - 1]);
}

int mrl_mlp_forward(mrl_ctx *ctx, const mrl_mlp_desc *d, int batch, const float *in,
                    const float *params, float *out, float *cache) {
    MRL_CHECK_ARG(ctx != nullptr, "mrl_mlp_forward: ctx is NULL");
    int rc = check_desc(d, "mrl_mlp_forward");
    if (rc) return rc;
    MRL_CHECK_ARG(batch >= 0, "mrl_mlp_forward: negative batch");
    if (batch == 0) return MRL_OK;
    MRL_CHECK_ARG(in && params && out, "mrl_mlp_forward: NULL buffer");
    rc = mlp3_forward(ctx, *d, batch, in, params, out, cache);
    if (rc != MRL_E_UNSUPPORTED) return rc;
    // two ping-pong activation buffers of the widest hidden size
    int widest = 0;
    for (int i = 0; i + 1 < d->n_layers; ++i) widest = std::max(widest, layer_out_dim(d->layers[i]));
    float *ws = nullptr;
    if (widest > 0) {
        rc = ensure_ws(ctx, (size_t)2 * batch * widest, &ws);
        if (rc) return rc;
    }
    const float *cur = in;
    const float *p = params;
    float *c = cache;
    for (int i = 0; i < d->n_layers; ++i) {
        const mrl_layer &l = d->layers[i];
        const bool last = i == d->n_layers - 1;
        float *dst = last ? out : ws + (size_t)(i & 1) * batch * widest;
        const int K = l.in_dim, N = l.out_dim, cs = layer_cache_size(l);
        const float *W = p, *b = p + (size_t)K * N;
        switch (l.kind) {
            case MRL_LINEAR: launch_fwd<ACT_NONE>(ctx->stream, cur, K, W, b, dst, N, c, cs, batch, K, N); break;
            case MRL_LINEAR_RELU: launch_fwd<ACT_RELU>(ctx->stream, cur, K, W, b, dst, N, c, cs, batch, K, N); break;
            case MRL_LINEAR_TANH: launch_fwd<ACT_TANH>(ctx->stream, cur, K, W, b, dst, N, c, cs, batch, K, N); break;
            case MRL_STOCHASTIC_ACTOR:
                launch_fwd<ACT_NONE>(ctx->stream, cur, K, W, b, dst, 2 * N, c, cs, batch, K, N);
                hipLaunchKernelGGL(actor_log_std_kernel, dim3(grid_for((long)batch * N, 256)), dim3(256),
                                   0, ctx->stream, b + N, dst, batch, N);
                break;
        }
        MRL_CHECK_LAUNCH();
        p += layer_param_size(l);
        if (c) c += (size_t)batch * cs;
        cur = dst;
    }
    return MRL_OK;
}

int mrl_mlp_backward(mrl_ctx *ctx, const mrl_mlp_desc *d, int batch, const float *grad_out,
                     const float *params, const float *cache, float *grads, float *grad_in) {
    MRL_CHECK_ARG(ctx != nullptr, "mrl_mlp_backward: ctx is NULL");
    int rc = check_desc(d, "mrl_mlp_backward");
    if (rc) return rc;
    MRL_CHECK_ARG(batch > 0, "mrl_mlp_backward: batch must be positive");
    MRL_CHECK_ARG(grad_out && params && cache && grads, "mrl_mlp_backward: NULL buffer");
    {
        int fh, fa;
        bool fg;
        if (grad_in == nullptr && mlp3_fusable(*d, &fh, &fa, &fg)) {
            float *fws = nullptr;
            const mrl_mlp_desc *ds[1] = {d};
            rc = ensure_ws(ctx, mlp3_backward_ws(ds, 1, batch), &fws);
            if (rc) return rc;
            rc = mlp3_backward(ctx, *d, batch, grad_out, params, cache, grads, fws);
            if (rc != MRL_E_UNSUPPORTED) return rc;
        }
    }

    size_t poff[MRL_MAX_LAYERS], coff[MRL_MAX_LAYERS];
    size_t p = 0, c = 0;
    int widest = 1, max_p = 0;
    for (int i = 0; i < d->n_layers; ++i) {
        poff[i] = p; coff[i] = c;
        p += layer_param_size(d->layers[i]);
        c += (size_t)batch * layer_cache_size(d->layers[i]);
        widest = std::max(widest, d->layers[i].in_dim);
        max_p = std::max(max_p, (d->layers[i].in_dim + 1) * d->layers[i].out_dim);
    }
    // batch split so that the dW launches fill the chip; slices are multiples of the k-chunk
    int splits = std::max(1, std::min(32, batch / 128));
    int rows_per = ((batch + splits - 1) / splits + KC - 1) / KC * KC;
    splits = (batch + rows_per - 1) / rows_per;
    float *ws = nullptr;
    rc = ensure_ws(ctx, (size_t)2 * batch * widest + (size_t)splits * max_p, &ws);
    if (rc) return rc;
    float *partial = ws + (size_t)2 * batch * widest;

    const float *g = grad_out;
    for (int i = d->n_layers - 1; i >= 0; --i) {
        const mrl_layer &l = d->layers[i];
        const int K = l.in_dim, N = l.out_dim, cs = layer_cache_size(l);
        const int ldg = (l.kind == MRL_STOCHASTIC_ACTOR) ? 2 * N : N;
        const float *W = params + poff[i];
        const float *ca = cache + coff[i];
        float *dst_dx = (i == 0) ? grad_in : ws + (size_t)(i & 1) * batch * widest;
        dim3 gdw((N + BN - 1) / BN, (K + 1 + BM - 1) / BM, splits);
        dim3 gdx((K + BN - 1) / BN, (batch + BM - 1) / BM);
        const int act = l.kind == MRL_LINEAR_RELU ? ACT_RELU : (l.kind == MRL_LINEAR_TANH ? ACT_TANH : ACT_NONE);
#define MRL_BWD(ACT)                                                                                  \
    do {                                                                                              \
        hipLaunchKernelGGL(linear_bwd_dw_kernel<ACT>, gdw, dim3(256), 0, ctx->stream, ca, cs, g, ldg,  \
                           partial, batch, K, N, rows_per);                                           \
        if (dst_dx)                                                                                   \
            hipLaunchKernelGGL(linear_bwd_dx_kernel<ACT>, gdx, dim3(256), 0, ctx->stream, g, ldg, W,   \
                               ca, cs, dst_dx, batch, K, N);                                          \
    } while (0)
        if (act == ACT_RELU) MRL_BWD(ACT_RELU);
        else if (act == ACT_TANH) MRL_BWD(ACT_TANH);
        else MRL_BWD(ACT_NONE);
#undef MRL_BWD
        MRL_CHECK_LAUNCH();
        const int np = (K + 1) * N;
        hipLaunchKernelGGL(sum_partials_kernel, dim3(grid_for(np, 256)), dim3(256), 0, ctx->stream,
                           partial, grads + poff[i], np, splits);
        if (l.kind == MRL_STOCHASTIC_ACTOR)
            hipLaunchKernelGGL(column_sum_kernel, dim3(N), dim3(256), 0, ctx->stream, g, ldg, N, batch,
                               grads + poff[i] + np);
        MRL_CHECK_LAUNCH();
        g = dst_dx;
    }
    return MRL_OK;
}

}  // extern "C"
