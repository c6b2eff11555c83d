// Fused kernels for the update path of three-layer nets  IN -> H -> H -> out  (H in {64, 256},
// IN <= 32, out <= 8 or a StochasticActor head of <= 8 actions): the shapes of every actor and
// critic the PPO agents build (deep_agents/ppo/ppo.mojo:779-817, ppo_continuous.mojo:171-194).
//
//   mlp3_fwd_kernel     the whole forward of a 32-row tile in one launch (hidden activations
//                       stay in LDS), writing the reference's per-layer cache on the way;
//   mlp3_bwd_dx_kernel  the chain  g2 -> g1 = (g2 W2^T) * act' -> g0 = (g1 W1^T) * act'  of a
//                       32-row tile in one launch; g1 and g0 go to a workspace;
//   dw3_kernel          [dW | db] of all three layers in one launch, split over the batch;
//   sum3_kernel         sum of the splits straight into the flat gradient vector (+ log_std).
// They replace 3 + 2 + 3 + 3 launches of the per-layer kernels (which remain the path for any
// other shape, and for callers that ask for the gradient with respect to the input).
#include "mrl_host.hpp"
#include "mrl_device.hpp"
#include "mlp_tile.hpp"

namespace mrl {

template <int H, int ACT, bool GAUSS>
__global__ __launch_bounds__(H) void mlp3_fwd_kernel(const float *__restrict__ x, int B, int IN, int A,
                                                     const float *__restrict__ params,
                                                     float *__restrict__ out, float *__restrict__ cache) {
    __shared__ float xs[PR * XS_LD];
    __shared__ float hT[H * HT_LD];
    __shared__ float h2[PR * (H + 1)];
    __shared__ float ys[PR * (PA_MAX + 1)];
    const int t = threadIdx.x;
    const long row0 = (long)blockIdx.x * PR;
    const int nrow = (int)min((long)PR, B - row0);
    TileCache tc{nullptr, nullptr, nullptr, row0, nrow};
    if (cache != nullptr) {
        tc.c0 = cache;
        tc.c1 = cache + (size_t)B * (IN + H);
        tc.c2 = tc.c1 + (size_t)B * 2 * H;
    }
    for (int i = t; i < PR * IN; i += H) {
        const int r = i / IN, k = i - r * IN;
        float v = 0.0f;
        if (r < nrow) {
            v = x[row0 * IN + i];
            if (cache != nullptr) tc.c0[(row0 + r) * (IN + H) + k] = v;
        }
        xs[r * XS_LD + k] = v;
    }
    __syncthreads();
    hidden_stack<H, ACT>(params, IN, xs, hT, h2, tc);
    const float *W2 = params + IN * H + H + H * H + H;
    head<H>(W2, A, h2, ys, PA_MAX + 1);
    __syncthreads();
    const int ld = GAUSS ? 2 * A : A;
    for (int i = t; i < nrow * ld; i += H) {
        const int r = i / ld, a = i - r * ld;
        float v;
        if (a < A) {
            v = ys[r * (PA_MAX + 1) + a];
        } else {   // state-independent log_std, clamped (deep_rl/model/stochastic_actor.mojo:260-275)
            v = W2[H * A + A + (a - A)];
            if (v < -5.0f) v = -5.0f;
            else if (v > 2.0f) v = 2.0f;
        }
        out[(row0 + r) * ld + a] = v;
    }
}

template <int ACT>
MRL_DEV float act_deriv(float cached) {
    if (ACT == 1) return cached > 0.0f ? 1.0f : 0.0f;
    if (ACT == 2) return 1.0f - cached * cached;
    return 1.0f;
}

// grad_out [B, ld] (ld = A, or 2A for the Gaussian head: mean gradients first); g1, g0 [B, H];
// ls_part [tiles, A]: per-tile sums of the log_std gradient columns
template <int H, int ACT, bool GAUSS>
__global__ __launch_bounds__(H) void mlp3_bwd_dx_kernel(const float *__restrict__ grad_out, int B, int IN,
                                                        int A, const float *__restrict__ params,
                                                        const float *__restrict__ cache,
                                                        float *__restrict__ g1, float *__restrict__ g0,
                                                        float *__restrict__ ls_part) {
    constexpr int KCH = 32;                       // k-chunk of W1 staged per round
    __shared__ float g2s[PR * (2 * PA_MAX + 1)];
    __shared__ float gT[H * HT_LD];               // g1 of the tile, k-major
    __shared__ float wT[KCH * (H + 1)];           // W1[i][o0 + k] stored as [k][i]
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, half = lane >> 5, l31 = lane & 31;
    const long row0 = (long)blockIdx.x * PR;
    const int nrow = (int)min((long)PR, B - row0);
    const int ld = GAUSS ? 2 * A : A;
    const float *c0 = cache, *c1 = cache + (size_t)B * (IN + H);
    const float *W1 = params + IN * H + H;
    const float *W2 = W1 + H * H + H;
    for (int i = t; i < PR * ld; i += H) {
        const int r = i / ld, a = i - r * ld;
        g2s[r * (2 * PA_MAX + 1) + a] = r < nrow ? grad_out[row0 * ld + i] : 0.0f;
    }
    __syncthreads();
    if (GAUSS && t < A) {
        float s = 0.0f;
        for (int r = 0; r < PR; ++r) s += g2s[r * (2 * PA_MAX + 1) + A + t];
        ls_part[(long)blockIdx.x * A + t] = s;
    }
    {   // g1[r][n] = (sum_a g2[r][a] W2[n][a]) * act'(layer 1); thread t owns column n = t
        float wrow[PA_MAX];
#pragma unroll
        for (int a = 0; a < PA_MAX; ++a) wrow[a] = a < A ? W2[t * A + a] : 0.0f;
        for (int r = 0; r < PR; ++r) {
            float s = 0.0f;
#pragma unroll
            for (int a = 0; a < PA_MAX; ++a)
                if (a < A) s = fmaf(g2s[r * (2 * PA_MAX + 1) + a], wrow[a], s);
            float g = 0.0f;
            if (r < nrow) {
                g = s * act_deriv<ACT>(c1[(row0 + r) * (2 * H) + H + t]);
                g1[(row0 + r) * H + t] = g;
            }
            gT[t * HT_LD + r] = g;
        }
    }
    // dh1 = g1 W1^T: wavefront w owns input columns [64w, 64w + 64)
    floatx16 acc0 = {0}, acc1 = {0};
    const int col0 = 64 * w + l31, col1 = col0 + 32;
    for (int o0 = 0; o0 < H; o0 += KCH) {
        __syncthreads();   // gT complete (first round) / previous chunk consumed
        {   // thread t copies W1[t][o0 .. o0 + 32) -> wT[k][t]
            const float4 *src = reinterpret_cast<const float4 *>(W1 + (size_t)t * H + o0);
#pragma unroll
            for (int q = 0; q < KCH / 4; ++q) {
                const float4 v = src[q];
                wT[(4 * q + 0) * (H + 1) + t] = v.x;
                wT[(4 * q + 1) * (H + 1) + t] = v.y;
                wT[(4 * q + 2) * (H + 1) + t] = v.z;
                wT[(4 * q + 3) * (H + 1) + t] = v.w;
            }
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KCH / 2; ++kk) {
            const int k = 2 * kk + half;
            const float a = gT[(o0 + k) * HT_LD + l31];
            const float b0 = wT[k * (H + 1) + col0];
            const float b1 = wT[k * (H + 1) + col1];
            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b0, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b1, acc1, 0, 0, 0);
        }
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int row = 8 * (v >> 2) + 4 * half + (v & 3);
        if (row >= nrow) continue;
        const float *q = c0 + (row0 + row) * (IN + H) + IN;
        float *o = g0 + (row0 + row) * H;
        o[col0] = acc0[v] * act_deriv<ACT>(q[col0]);
        o[col1] = acc1[v] * act_deriv<ACT>(q[col1]);
    }
}

// ---------------------------------------------------------------- [dW | db] of the three layers
constexpr int DBM = 64, DBN = 64, DKC = 32, DLD = 65;

struct DwProblem {
    const float *X;   // layer input per batch row (row stride xs)
    const float *G;   // gradient at the layer's pre-activation (row stride gs)
    int xs, gs, K, N; // K inputs, N outputs: the block written is [(K + 1), N] (last row = bias)
    int poff;         // offset of the layer in the flat parameter vector
    int tiles_n, tiles;   // tiles_n = ceil(N / 64); tiles = tiles_n * ceil((K + 1) / 64)
};
struct Dw3 { DwProblem p[3]; };

// grid.x = sum of the layers' tiles, grid.y = batch splits; partial[z][P]
__global__ __launch_bounds__(256) void dw3_kernel(Dw3 d, int M, int rows_per_split, int P,
                                                  float *__restrict__ partial) {
    __shared__ float As[DKC * DLD];
    __shared__ float Bs[DKC * DLD];
    int tile = blockIdx.x, li = 0;
    while (li < 2 && tile >= d.p[li].tiles) { tile -= d.p[li].tiles; ++li; }
    const DwProblem &pr = d.p[li];
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wr = w >> 1, wc = w & 1;
    const int half = lane >> 5, l31 = lane & 31;
    const int j0 = (tile % pr.tiles_n) * DBN, i0 = (tile / pr.tiles_n) * DBM, z = blockIdx.y;
    const long b_begin = (long)z * rows_per_split;
    long b_end = b_begin + rows_per_split;
    if (b_end > M) b_end = M;
    floatx16 acc = {0};
    const int bb = t >> 3, seg = (t & 7) * 8;
    for (long b0 = b_begin; b0 < b_end; b0 += DKC) {
        const long b = b0 + bb;
        const bool inb = b < b_end;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int ii = i0 + seg + i;
            float v = 0.0f;
            if (inb) {
                if (ii < pr.K) v = pr.X[b * pr.xs + ii];
                else if (ii == pr.K) v = 1.0f;
            }
            As[bb * DLD + seg + i] = v;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int j = j0 + seg + i;
            Bs[bb * DLD + seg + i] = (inb && j < pr.N) ? pr.G[b * pr.gs + j] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < DKC; kk += 2) {
            const float a = As[(kk + half) * DLD + 32 * wr + l31];
            const float bv = Bs[(kk + half) * DLD + 32 * wc + l31];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bv, acc, 0, 0, 0);
        }
        __syncthreads();
    }
    const int col = j0 + 32 * wc + l31;
    if (col < pr.N) {
        float *out = partial + (size_t)z * P + pr.poff;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = i0 + 32 * wr + 8 * (v >> 2) + 4 * half + (v & 3);
            if (row <= pr.K) out[(size_t)row * pr.N + col] = acc[v];
        }
    }
}

// grads[i] = sum_z partial[z][i] for the [W | b] blocks; the log_std tail (Gaussian head) sums the
// per-tile column sums of the backward-dx kernel
__global__ __launch_bounds__(256) void sum3_kernel(const float *__restrict__ partial, int splits, int P,
                                                   int n_wb, const float *__restrict__ ls_part, int tiles,
                                                   int A, float *__restrict__ grads) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= P) return;
    float s = 0.0f;
    if (i < n_wb) {
        for (int z = 0; z < splits; ++z) s += partial[(size_t)z * P + i];
    } else {
        const int j = i - n_wb;
        for (int q = 0; q < tiles; ++q) s += ls_part[(size_t)q * A + j];
    }
    grads[i] = s;
}

// ---------------------------------------------------------------- host side

bool mlp3_fusable(const mrl_mlp_desc &d, int *H, int *act, bool *gauss) {
    if (d.n_layers != 3) return false;
    const int k0 = d.layers[0].kind;
    if ((k0 != MRL_LINEAR_RELU && k0 != MRL_LINEAR_TANH) || d.layers[1].kind != k0) return false;
    const int k2 = d.layers[2].kind;
    if (k2 != MRL_LINEAR && k2 != MRL_STOCHASTIC_ACTOR) return false;
    const int h = d.layers[0].out_dim;
    if ((h != 64 && h != 256) || d.layers[1].out_dim != h) return false;
    if (d.layers[0].in_dim > PIN_MAX || d.layers[2].out_dim > PA_MAX) return false;
    *H = h;
    *act = k0 == MRL_LINEAR_RELU ? 1 : 2;
    *gauss = k2 == MRL_STOCHASTIC_ACTOR;
    return true;
}

int mlp3_forward(mrl_ctx *ctx, const mrl_mlp_desc &d, int batch, const float *in, const float *params,
                 float *out, float *cache) {
    int H = 0, act = 0;
    bool gauss = false;
    if (!mlp3_fusable(d, &H, &act, &gauss)) return MRL_E_UNSUPPORTED;
    const int IN = d.layers[0].in_dim, A = d.layers[2].out_dim;
    dim3 grid((batch + PR - 1) / PR);
#define MRL_F(HH, AA, GG)                                                                          \
    hipLaunchKernelGGL((mlp3_fwd_kernel<HH, AA, GG>), grid, dim3(HH), 0, ctx->stream, in, batch, IN, A, \
                       params, out, cache)
#define MRL_F2(HH, AA) do { if (gauss) MRL_F(HH, AA, true); else MRL_F(HH, AA, false); } while (0)
    if (H == 256 && act == 1) MRL_F2(256, 1);
    else if (H == 256) MRL_F2(256, 2);
    else if (act == 1) MRL_F2(64, 1);
    else MRL_F2(64, 2);
#undef MRL_F2
#undef MRL_F
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mlp3_backward(mrl_ctx *ctx, const mrl_mlp_desc &d, int batch, const float *grad_out, const float *params,
                  const float *cache, float *grads, float *ws) {
    int H = 0, act = 0;
    bool gauss = false;
    if (!mlp3_fusable(d, &H, &act, &gauss)) return MRL_E_UNSUPPORTED;
    const int IN = d.layers[0].in_dim, A = d.layers[2].out_dim;
    // the W1 rows are staged with 16-byte loads
    if (reinterpret_cast<uintptr_t>(params + IN * H + H) % 16 != 0) return MRL_E_UNSUPPORTED;
    const int tiles = (batch + PR - 1) / PR;
    const int n_wb = (IN + 1) * H + (H + 1) * H + (H + 1) * A;
    const int P = n_wb + (gauss ? A : 0);
    int splits = std::max(1, std::min(32, batch / 128));
    int rows_per = ((batch + splits - 1) / splits + DKC - 1) / DKC * DKC;
    splits = (batch + rows_per - 1) / rows_per;
    // workspace: g1 [B, H] | g0 [B, H] | ls_part [tiles, A] | partial [splits, P]
    float *g1 = ws, *g0 = g1 + (size_t)batch * H, *ls_part = g0 + (size_t)batch * H;
    float *partial = ls_part + (size_t)tiles * PA_MAX;
#define MRL_B(HH, AA, GG)                                                                               \
    hipLaunchKernelGGL((mlp3_bwd_dx_kernel<HH, AA, GG>), dim3(tiles), dim3(HH), 0, ctx->stream, grad_out,    \
                       batch, IN, A, params, cache, g1, g0, ls_part)
#define MRL_B2(HH, AA) do { if (gauss) MRL_B(HH, AA, true); else MRL_B(HH, AA, false); } while (0)
    if (H == 256 && act == 1) MRL_B2(256, 1);
    else if (H == 256) MRL_B2(256, 2);
    else if (act == 1) MRL_B2(64, 1);
    else MRL_B2(64, 2);
#undef MRL_B2
#undef MRL_B
    MRL_CHECK_LAUNCH();
    const float *c0 = cache, *c1 = cache + (size_t)batch * (IN + H), *c2 = c1 + (size_t)batch * 2 * H;
    Dw3 dw;
    auto fill = [](DwProblem &p, const float *X, int xs, const float *G, int gs, int K, int N, int poff) {
        p.X = X; p.G = G; p.xs = xs; p.gs = gs; p.K = K; p.N = N; p.poff = poff;
        p.tiles_n = (N + DBN - 1) / DBN;
        p.tiles = p.tiles_n * ((K + 1 + DBM - 1) / DBM);
    };
    fill(dw.p[0], c0, IN + H, g0, H, IN, H, 0);
    fill(dw.p[1], c1, 2 * H, g1, H, H, H, (IN + 1) * H);
    fill(dw.p[2], c2, H, grad_out, gauss ? 2 * A : A, H, A, (IN + 1) * H + (H + 1) * H);
    dim3 gdw(dw.p[0].tiles + dw.p[1].tiles + dw.p[2].tiles, splits);
    hipLaunchKernelGGL(dw3_kernel, gdw, dim3(256), 0, ctx->stream, dw, batch, rows_per, P, partial);
    hipLaunchKernelGGL(sum3_kernel, dim3(grid_for(P, 256)), dim3(256), 0, ctx->stream, partial, splits, P,
                       n_wb, ls_part, tiles, A, grads);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

// floats of workspace mlp3_backward needs
size_t mlp3_backward_ws(const mrl_mlp_desc &d, int batch) {
    const int H = d.layers[0].out_dim, IN = d.layers[0].in_dim, A = d.layers[2].out_dim;
    const size_t P = (size_t)(IN + 1) * H + (size_t)(H + 1) * H + (size_t)(H + 1) * A + A;
    return (size_t)2 * batch * H + (size_t)((batch + PR - 1) / PR) * PA_MAX + (size_t)32 * P;
}

}  // namespace mrl
