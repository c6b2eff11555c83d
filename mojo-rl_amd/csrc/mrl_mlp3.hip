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
#include "mlp3.hpp"
#include "ppo_grads.hpp"

namespace mrl {

// grid = (row tiles, nets): blockIdx.y picks the net, so that an actor and a critic that read the
// same inputs go through the chip side by side
template <int H, int ACT>
__global__ __launch_bounds__(2 * H) void mlp3_fwd_kernel(int B, int IN, Mlp3Nets nets, FwdLoss fl) {
    constexpr int T = 2 * H;   // one 32-column accumulator tile per wavefront
    __shared__ float xs[PR * XS_LD];
    __shared__ float hT[H * HT_LD];
    __shared__ float h2[PR * (H + 1)];
    __shared__ float ys[PR * (PA_MAX + 1)];
    __shared__ __align__(16) float w2s[HEAD_LDS(H)];
    const Mlp3Net &nn = nets.n[blockIdx.y];
    const float *__restrict__ x = nn.x;
    const float *__restrict__ params = nn.params;
    float *__restrict__ out = nn.out;
    float *__restrict__ cache = nn.cache;
    const int A = nn.A;
    const bool GAUSS = nn.gauss != 0;
    const int t = threadIdx.x;
    const long row0 = (long)blockIdx.x * PR;
    const int nrow = (int)min((long)PR, B - row0);
    TileCache tc{nullptr, nullptr, nullptr, row0, nrow};
    if (cache != nullptr) {
        tc.c0 = cache;
        tc.c1 = cache + (size_t)B * (IN + H);
        tc.c2 = tc.c1 + (size_t)B * 2 * H;
    }
    // every load that does not depend on an earlier phase goes out first
    HiddenOperands<H, 1, 32> ops;
    ops.load(params, IN);
    constexpr int NX = (PR * PIN_MAX + T - 1) / T;
    float xv[NX];
#pragma unroll
    for (int q = 0; q < NX; ++q) {
        const int i = t + q * T;
        xv[q] = 0.0f;
        if (i < PR * IN && i / IN < nrow) {
            const int r = i / IN;
            xv[q] = fl.enabled ? fl.r_obs[(size_t)fl.idx[row0 + r] * IN + (i - r * IN)] : x[row0 * IN + i];
        }
    }
    stage_head(params + IN * H + H + H * H + H, H, A, GAUSS, w2s, t, T);
#pragma unroll
    for (int q = 0; q < NX; ++q) {
        const int i = t + q * T;
        if (i < PR * IN) {
            const int r = i / IN, k = i - r * IN;
            xs[r * XS_LD + k] = xv[q];
            if (r < nrow && cache != nullptr) tc.c0[(row0 + r) * (IN + H) + k] = xv[q];
        }
    }
    __syncthreads();
    hidden_stack<H, ACT, 1>(params, IN, xs, hT, h2, tc, ops);
    head<H>(w2s, A, h2, ys, PA_MAX + 1, t, 2 * H);
    __syncthreads();
    const int ld = GAUSS ? 2 * A : A;
    for (int i = t; i < nrow * ld; i += T) {
        const int r = i / ld, a = i - r * ld;
        float v;
        if (a < A) {
            v = ys[r * (PA_MAX + 1) + a];
        } else {   // state-independent log_std, clamped (deep_rl/model/stochastic_actor.mojo:260-275)
            v = w2s[HEAD_LOG_STD(H) + (a - A)];
            if (v < -5.0f) v = -5.0f;
            else if (v > 2.0f) v = 2.0f;
        }
        out[(row0 + r) * ld + a] = v;
    }
    if (!fl.enabled) return;
    // ---- loss gradients of the tile's rows, one lane per row (wavefront 0)
    if (t >= 64) return;
    const int b = (int)row0 + t;
    const bool mine = t < nrow;
    const long src = mine ? fl.idx[b] : 0;
    if (blockIdx.y == 1) {   // critic
        if (mine)
            fl.g_values[b] = critic_grad_value(ys[t * (PA_MAX + 1)], fl.clip_value ? fl.r_val[src] : 0.0f, fl.r_ret[src],
                                               fl.mb, fl.continuous, fl.clip_value, fl.value_coef, fl.clip_eps);
        return;
    }
    float kl = 0.0f;
    if (mine) {
        float adv = fl.r_adv[src];
        if (fl.adv_stats != nullptr) adv = (adv - fl.adv_stats[0]) / (fl.adv_stats[1] + 1e-8f);
        const float old_logp = fl.r_logp[src];
        float o[2 * PA_MAX], g[2 * PA_MAX];
#pragma unroll
        for (int a = 0; a < PA_MAX; ++a) {
            o[a] = ys[t * (PA_MAX + 1) + a];
            float ls = w2s[HEAD_LOG_STD(H) + a];
            o[PA_MAX + a] = ls;
        }
        if (fl.continuous) {
            float oo[2 * PA_MAX], act[PA_MAX];
            for (int j = 0; j < A; ++j) {
                oo[j] = o[j];
                oo[A + j] = o[PA_MAX + j];   // clamped inside the gradient, as in the stored output
                act[j] = fl.r_act[src * A + j];
            }
            kl = actor_grad_gaussian_row(oo, act, adv, old_logp, fl.mb, A, fl.clip_eps, fl.ent_coef, g);
            for (int j = 0; j < 2 * A; ++j) fl.g_actor_out[(size_t)b * 2 * A + j] = g[j];
        } else {
            kl = actor_grad_discrete_row(o, (int)fl.r_act[src], adv, old_logp, fl.mb, A, fl.clip_eps, fl.ent_coef, g);
            for (int a = 0; a < A; ++a) fl.g_actor_out[(size_t)b * A + a] = g[a];
        }
        fl.kl[b] = kl;
    }
    if (fl.kl_flag == nullptr) return;
    // KL test: every actor tile leaves the sum of its rows' estimates; the kernel that applies the
    // update adds the tiles up and compares the mean with target_kl
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) kl += __shfl_xor(kl, off, 64);
    if (t == 0) fl.kl_part[blockIdx.x] = kl;
}

template <int ACT>
MRL_DEV float act_deriv(float cached) {
    if (ACT == 1) return cached > 0.0f ? 1.0f : 0.0f;
    if (ACT == 2) return 1.0f - cached * cached;
    return 1.0f;
}

// grad_out [B, ld] (ld = A, or 2A for the Gaussian head: mean gradients first); g1, g0 [B, H];
// ls_part [tiles, A]: per-tile sums of the log_std gradient columns.  grid = (row tiles, nets).
template <int H, int ACT>
__global__ __launch_bounds__(2 * H) void mlp3_bwd_dx_kernel(int B, int IN, Mlp3Nets nets) {
    constexpr int T = 2 * H;   // one 32-column accumulator tile per wavefront
    const Mlp3Net &nn = nets.n[blockIdx.y];
    const float *__restrict__ grad_out = nn.grad_out;
    const float *__restrict__ params = nn.params;
    const float *__restrict__ cache = nn.cache;
    float *__restrict__ g1 = nn.g1;
    float *__restrict__ g0 = nn.g0;
    float *__restrict__ ls_part = nn.ls_part;
    float *__restrict__ db_part = nn.db_part + (size_t)blockIdx.x * (2 * H + PA_MAX);   // this tile's slice
    const int A = nn.A;
    // this tile's share of the two thin weight gradients: [dW0 (IN x H) | dW2 (H x A)]
    float *__restrict__ thin_part = nn.thin_part + (size_t)blockIdx.x * (size_t)nn.thin_stride;
    const bool GAUSS = nn.gauss != 0;
    constexpr int KCH = 64;                       // k-chunk of W1 staged per round
    __shared__ float g2s[PR * (2 * PA_MAX + 1)];
    __shared__ float xs[PR * XS_LD];              // the tile's inputs, for dW0
    __shared__ float gT[H * HT_LD];               // g1 of the tile, k-major
    __shared__ float wT[KCH * (H + 1)];           // W1[i][o0 + k] stored as [k][i]
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, half = lane >> 5, l31 = lane & 31;
    const long row0 = (long)blockIdx.x * PR;
    const int nrow = (int)min((long)PR, B - row0);
    const int ld = GAUSS ? 2 * A : A;
    const float *c0 = cache, *c1 = cache + (size_t)B * (IN + H), *c2 = c1 + (size_t)B * 2 * H;
    const float *W1 = params + IN * H + H;
    const float *W2 = W1 + H * H + H;
    // what the later phases need from global memory is requested now, in few wide loads (a
    // wavefront can keep 64 vector-memory instructions in flight), so that the block waits for
    // memory once: the cached activations behind act' of both hidden layers as row tiles, the head
    // weights, the first chunk of W1
    static_assert(PR * H == 4 * 4 * T && 2 * PR * H <= KCH * (H + 1), "tile staging layout");
    float4 t1[4], t2[4];   // 32 x H tiles of the layer-1 cache entries and of h2, 16 bytes per thread and load
    float w2row[PA_MAX];   // thread t < H: W2[t][:]
    float d0[16];          // layer-0 cache entries at this lane's accumulator positions
    const int wrow = t % H, wseg = (t / H) * (KCH / 2);   // thread copies W1[wrow][o0 + wseg .. + KCH / 2)
    float4 nxt[KCH / 8];
    auto fetch = [&](int o0) {
        const float4 *src = reinterpret_cast<const float4 *>(W1 + (size_t)wrow * H + o0 + wseg);
#pragma unroll
        for (int q = 0; q < KCH / 8; ++q) nxt[q] = src[q];
    };
    {
        const bool vec = ((reinterpret_cast<uintptr_t>(c1) | reinterpret_cast<uintptr_t>(c2)) & 15) == 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int e = 4 * (t + q * T), r = e / H, ci = e % H;
            const float *s1 = c1 + (row0 + r) * (2 * H) + H + ci;
            const float *s2 = c2 + (row0 + r) * H + ci;
            t1[q] = t2[q] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (r < nrow) {
                if (vec) {
                    t1[q] = *reinterpret_cast<const float4 *>(s1);
                    t2[q] = *reinterpret_cast<const float4 *>(s2);
                } else {
                    t1[q] = make_float4(s1[0], s1[1], s1[2], s1[3]);
                    t2[q] = make_float4(s2[0], s2[1], s2[2], s2[3]);
                }
            }
        }
#pragma unroll
        for (int a = 0; a < PA_MAX; ++a) w2row[a] = a < A ? W2[wrow * A + a] : 0.0f;
        const int colq = 32 * w + l31;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = 8 * (v >> 2) + 4 * half + (v & 3);
            d0[v] = row < nrow ? c0[(row0 + row) * (IN + H) + IN + colq] : 0.0f;
        }
        fetch(0);
    }
    for (int i = t; i < PR * ld; i += T) {
        const int r = i / ld, a = i - r * ld;
        g2s[r * (2 * PA_MAX + 1) + a] = r < nrow ? grad_out[row0 * ld + i] : 0.0f;
    }
    for (int i = t; i < PR * IN; i += T) {
        const int r = i / IN, k = i - r * IN;
        xs[r * XS_LD + k] = r < nrow ? c0[(row0 + r) * (IN + H) + k] : 0.0f;
    }
    // the two tiles rest in the W1 staging buffer until the chunk loop claims it
    float *tile1 = wT, *tile2 = wT + PR * H;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int e = 4 * (t + q * T);
        *reinterpret_cast<float4 *>(tile1 + e) = t1[q];
        *reinterpret_cast<float4 *>(tile2 + e) = t2[q];
    }
    __syncthreads();
    if (t < H) {   // g1[r][n] = (sum_a g2[r][a] W2[n][a]) * act'(layer 1); thread t owns column n = t
        float colsum = 0.0f;
#pragma unroll
        for (int r = 0; r < PR; ++r) {
            float s = 0.0f;
#pragma unroll
            for (int a = 0; a < PA_MAX; ++a)
                if (a < A) s = fmaf(g2s[r * (2 * PA_MAX + 1) + a], w2row[a], s);
            float g = 0.0f;
            if (r < nrow) {
                g = s * act_deriv<ACT>(tile1[r * H + t]);
                g1[(row0 + r) * H + t] = g;
            }
            gT[t * HT_LD + r] = g;
            colsum += g;
        }
        db_part[H + t] = colsum;   // bias gradient of layer 1, this tile's rows
    } else {       // meanwhile the other half of the block: dW2[n][a] of the tile = sum_r h2[r][n] g2[r][a]
        const int n = t - H;
        float s[PA_MAX];
#pragma unroll
        for (int a = 0; a < PA_MAX; ++a) s[a] = 0.0f;
#pragma unroll
        for (int r = 0; r < PR; ++r) {
            const float h = tile2[r * H + n];
#pragma unroll
            for (int a = 0; a < PA_MAX; ++a)
                if (a < A) s[a] = fmaf(h, g2s[r * (2 * PA_MAX + 1) + a], s[a]);
        }
        float *o2 = thin_part + (size_t)IN * H + (size_t)n * A;
#pragma unroll
        for (int a = 0; a < PA_MAX; ++a)
            if (a < A) o2[a] = s[a];
        if (n < ld) {   // column sums of the tile: bias gradient of the head, log_std gradient
            float cs2 = 0.0f;
            for (int r = 0; r < PR; ++r) cs2 += g2s[r * (2 * PA_MAX + 1) + n];
            if (n < A) db_part[2 * H + n] = cs2;
            else ls_part[(long)blockIdx.x * A + (n - A)] = cs2;
        }
    }
    // dh1 = g1 W1^T: wavefront w owns input columns [32w, 32w + 32).  The next chunk of W1 is
    // fetched into registers while the matrix cores work on the current one.
    floatx16 acc = {0};
    const int col = 32 * w + l31;
    for (int o0 = 0; o0 < H; o0 += KCH) {
        __syncthreads();   // gT complete (first round) / previous chunk consumed
#pragma unroll
        for (int q = 0; q < KCH / 8; ++q) {
            wT[(wseg + 4 * q + 0) * (H + 1) + wrow] = nxt[q].x;
            wT[(wseg + 4 * q + 1) * (H + 1) + wrow] = nxt[q].y;
            wT[(wseg + 4 * q + 2) * (H + 1) + wrow] = nxt[q].z;
            wT[(wseg + 4 * q + 3) * (H + 1) + wrow] = nxt[q].w;
        }
        __syncthreads();
        if (o0 + KCH < H) fetch(o0 + KCH);
        __builtin_amdgcn_sched_barrier(0);   // keep the loads ahead of the MFMAs that hide them
#pragma unroll
        for (int kk = 0; kk < KCH / 2; ++kk) {
            const int k = 2 * kk + half;
            const float a = gT[(o0 + k) * HT_LD + l31];
            const float b = wT[k * (H + 1) + col];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
        }
    }
    float cs = 0.0f;
    float gv[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int row = 8 * (v >> 2) + 4 * half + (v & 3);
        gv[v] = 0.0f;
        if (row >= nrow) continue;
        const float val = acc[v] * act_deriv<ACT>(d0[v]);
        g0[(row0 + row) * H + col] = val;
        gv[v] = val;
        cs += val;
    }
    // the two halves of the wavefront hold the other 16 rows of the same column
    cs += __shfl_xor(cs, 32, 64);
    if (half == 0) db_part[col] = cs;   // bias gradient of layer 0, this tile's rows
    // dW0[i][col] of the tile = sum_r x[r][i] g0[r][col]
    for (int i = 0; i < IN; ++i) {
        float s = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; ++v) s = fmaf(xs[(8 * (v >> 2) + 4 * half + (v & 3)) * XS_LD + i], gv[v], s);
        s += __shfl_xor(s, 32, 64);
        if (half == 0) thin_part[(size_t)i * H + col] = s;
    }
}

// ---------------------------------------------------------------- forward + loss + backward of a tile
// The PPO minibatch never needs the activations outside the workgroup that made them: a row tile
// goes forward (as mlp3_fwd_kernel with its loss tail), and while h1 and h2 are still in LDS the
// same workgroup takes the loss gradient back through the three layers (as mlp3_bwd_dx_kernel).
// Only what the H x H weight gradient needs leaves the chip -- h1 (into the cache's c1 rows) and
// g1 -- next to the per-tile bias / thin-layer partials.  act' comes from the activation's output
// (y > 0 for ReLU, 1 - y^2 for tanh), which is what the cached entries decide as well.
template <int ACT>
MRL_DEV float act_deriv_out(float y) {
    if (ACT == 1) return y > 0.0f ? 1.0f : 0.0f;
    if (ACT == 2) return 1.0f - y * y;
    return 1.0f;
}

template <int H, int ACT>
__global__ __launch_bounds__(2 * H) void mlp3_fb_kernel(int B, int IN, Mlp3Nets nets, FwdLoss fl) {
    constexpr int T = 2 * H, KCH = 64;
    static_assert(KCH * (H + 1) <= H * HT_LD + PR * (H + 1), "the W1 staging buffer fits over the two activation tiles");
    __shared__ float xs[PR * XS_LD];
    __shared__ float big[H * HT_LD + PR * (H + 1)];   // hT | h2 going forward, W1 chunks going back
    __shared__ float ys[PR * (PA_MAX + 1)];
    __shared__ __align__(16) float w2s[HEAD_LDS(H)];
    __shared__ float g2s[PR * (2 * PA_MAX + 1)];
    __shared__ float gT[H * HT_LD];                   // g1 of the tile, k-major
    float *hT = big, *h2 = big + H * HT_LD, *wT = big;
    const Mlp3Net &nn = nets.n[blockIdx.y];
    const float *__restrict__ params = nn.params;
    float *__restrict__ out = nn.out;
    float *__restrict__ g1 = nn.g1;
    float *__restrict__ ls_part = nn.ls_part;
    float *__restrict__ db_part = nn.db_part + (size_t)blockIdx.x * (2 * H + PA_MAX);
    const int A = nn.A;
    float *__restrict__ thin_part = nn.thin_part + (size_t)blockIdx.x * (size_t)nn.thin_stride;
    const bool GAUSS = nn.gauss != 0;
    const int ld = GAUSS ? 2 * A : A;
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, half = lane >> 5, l31 = lane & 31;
    const long row0 = (long)blockIdx.x * PR;
    const int nrow = (int)min((long)PR, B - row0);
    const float *W1 = params + IN * H + H;
    TileCache tc{nullptr, nn.cache + (size_t)B * (IN + H), nullptr, row0, nrow};   // h1 only

    // ---- forward
    HiddenOperands<H, 1, 32> ops;
    ops.load(params, IN);
    constexpr int NX = (PR * PIN_MAX + T - 1) / T;
    float xv[NX];
#pragma unroll
    for (int q = 0; q < NX; ++q) {
        const int i = t + q * T;
        xv[q] = 0.0f;
        if (i < PR * IN && i / IN < nrow) {
            const int r = i / IN;
            xv[q] = fl.r_obs[(size_t)fl.idx[row0 + r] * IN + (i - r * IN)];
        }
    }
    stage_head(params + IN * H + H + H * H + H, H, A, GAUSS, w2s, t, T);
    for (int i = t; i < PR * (2 * PA_MAX + 1); i += T) g2s[i] = 0.0f;
    // The loss lanes ask for their rows' rollout entries now.  Critic: the lane of row t (wavefront 0).
    // Actor: eight lanes per row, lane lj on logit / action component lj (rows lr, lr + T / 8, ...), so
    // that a row's exponentials and logarithms are taken side by side instead of one after the other.
    static_assert(PA_MAX == 8 && T % 8 == 0, "eight lanes per row");
    constexpr int LR = (PR + T / 8 - 1) / (T / 8);   // rows per actor loss lane (lanes past the tile's rows idle)
    const bool loss_lane = t < nrow;
    const int lr = t >> 3, lj = t & 7;
    float l_ret = 0.0f, l_val = 0.0f, l_mean = 0.0f, l_std = 1.0f;
    float l_adv[LR], l_logp[LR], l_act[LR];   // l_act: the action (discrete) or its component lj
    if (blockIdx.y == 1) {
        if (loss_lane) {
            const long src = fl.idx[row0 + t];
            l_ret = fl.r_ret[src];
            if (fl.clip_value) l_val = fl.r_val[src];
        }
    } else {
        if (fl.adv_stats != nullptr) { l_mean = fl.adv_stats[0]; l_std = fl.adv_stats[1]; }
#pragma unroll
        for (int q = 0; q < LR; ++q) {
            const int r = lr + q * (T / 8);
            l_adv[q] = 0.0f; l_logp[q] = 0.0f; l_act[q] = 0.0f;
            if (r < nrow) {
                const long src = fl.idx[row0 + r];
                l_adv[q] = fl.r_adv[src];
                l_logp[q] = fl.r_logp[src];
                if (!fl.continuous) l_act[q] = fl.r_act[src];
                else if (lj < A) l_act[q] = fl.r_act[src * A + lj];
            }
        }
    }
#pragma unroll
    for (int q = 0; q < NX; ++q) {
        const int i = t + q * T;
        if (i < PR * IN) xs[(i / IN) * XS_LD + (i % IN)] = xv[q];
    }
    __syncthreads();
    hidden_stack<H, ACT, 1>(params, IN, xs, hT, h2, tc, ops);
    head<H>(w2s, A, h2, ys, PA_MAX + 1, t, 2 * H);
    __syncthreads();
    for (int i = t; i < nrow * ld; i += T) {
        const int r = i / ld, a = i - r * ld;
        float v;
        if (a < A) {
            v = ys[r * (PA_MAX + 1) + a];
        } else {   // state-independent log_std, clamped (deep_rl/model/stochastic_actor.mojo:260-275)
            v = w2s[HEAD_LOG_STD(H) + (a - A)];
            if (v < -5.0f) v = -5.0f;
            else if (v > 2.0f) v = 2.0f;
        }
        out[(row0 + r) * ld + a] = v;
    }
    // what the way back needs from the forward tiles before their memory is reused: act'(h1) at
    // this lane's accumulator positions; and the first chunk of W1
    const int col = 32 * w + l31;
    float d0[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) d0[v] = act_deriv_out<ACT>(hT[col * HT_LD + 8 * (v >> 2) + 4 * half + (v & 3)]);
    const int wrow = t % H, wseg = (t / H) * (KCH / 2);   // thread copies W1[wrow][o0 + wseg .. + KCH / 2)
    float4 nxt[KCH / 8];
    auto fetch = [&](int o0) {
        const float4 *src = reinterpret_cast<const float4 *>(W1 + (size_t)wrow * H + o0 + wseg);
#pragma unroll
        for (int q = 0; q < KCH / 8; ++q) nxt[q] = src[q];
    };
    fetch(0);

    // ---- loss gradients of the tile's rows into g2s and out
    if (blockIdx.y == 1) {   // critic: one lane per row
        if (loss_lane) {
            const float g = critic_grad_value(ys[t * (PA_MAX + 1)], l_val, l_ret, fl.mb, fl.continuous, fl.clip_value,
                                              fl.value_coef, fl.clip_eps);
            g2s[t * (2 * PA_MAX + 1)] = g;
            fl.g_values[(int)row0 + t] = g;
        }
    } else {
        // (rows past nrow are worked on like the others -- their lanes take part in the exchanges -- and not stored)
#pragma unroll
        for (int q = 0; q < LR; ++q) {
            const int r = lr + q * (T / 8), b = (int)row0 + r;
            float *g2row = g2s + r * (2 * PA_MAX + 1);
            float adv = l_adv[q];
            if (fl.adv_stats != nullptr) adv = (adv - l_mean) / (l_std + 1e-8f);
            const float mine = ys[(r < PR ? r : 0) * (PA_MAX + 1) + lj];
            float kl;
            if (fl.continuous) {
                float gm, gs;   // (log_std is clamped inside the gradient, as in the stored output)
                kl = actor_grad_gaussian_lanes(mine, w2s[HEAD_LOG_STD(H) + lj], l_act[q], lj, lane & ~7, adv, l_logp[q], fl.mb,
                                               A, fl.clip_eps, fl.ent_coef, gm, gs);
                if (r < nrow && lj < A) {
                    g2row[lj] = gm;
                    g2row[A + lj] = gs;
                    fl.g_actor_out[(size_t)b * ld + lj] = gm;
                    fl.g_actor_out[(size_t)b * ld + A + lj] = gs;
                }
            } else {
                float g;
                kl = actor_grad_discrete_lanes(mine, lj, lane & ~7, (int)l_act[q], adv, l_logp[q], fl.mb, A, fl.clip_eps,
                                               fl.ent_coef, g);
                if (r < nrow && lj < A) {
                    g2row[lj] = g;
                    fl.g_actor_out[(size_t)b * ld + lj] = g;
                }
            }
            if (r < nrow && lj == 0) {
                fl.kl[b] = kl;
                g2row[2 * PA_MAX] = kl;   // (the spare float of the row, for the tile's sum below)
            }
        }
    }
    __syncthreads();   // g2s complete
    if (fl.kl_flag != nullptr && blockIdx.y == 0 && t < 64) {
        // KL test: every actor tile leaves the sum of its rows' estimates; the kernel that applies the
        // update (clip + Adam) adds the tiles up and compares the mean with target_kl, so that nothing
        // here waits for other workgroups
        float kl = t < nrow ? g2s[t * (2 * PA_MAX + 1) + 2 * PA_MAX] : 0.0f;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) kl += __shfl_xor(kl, off, 64);
        if (t == 0) fl.kl_part[blockIdx.x] = kl;
    }

    // ---- back through the head and layer 1's activation, on the matrix cores; wavefront w owns
    // columns [32w, 32w + 32) of the hidden layers throughout
    {   // g1[r][n] = (sum_a g2[r][a] W2[n][a]) * act'(layer 1): K = PA_MAX (W2 rows are zero beyond A)
        floatx16 c = {0};
#pragma unroll
        for (int kk = 0; kk < PA_MAX / 2; ++kk) {
            const int k = 2 * kk + half;
            c = __builtin_amdgcn_mfma_f32_32x32x2f32(g2s[l31 * (2 * PA_MAX + 1) + k], w2s[col * PA_MAX + k], c, 0, 0, 0);
        }
        float colsum = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = 8 * (v >> 2) + 4 * half + (v & 3);
            float g = 0.0f;
            if (row < nrow) {
                g = c[v] * act_deriv_out<ACT>(h2[row * (H + 1) + col]);
                g1[(row0 + row) * H + col] = g;
            }
            gT[col * HT_LD + row] = g;
            colsum += g;
        }
        colsum += __shfl_xor(colsum, 32, 64);
        if (half == 0) db_part[H + col] = colsum;   // bias gradient of layer 1, this tile's rows
    }
    {   // dW2[n][a] of the tile = sum_r h2[r][n] g2[r][a]: K = the tile's 32 rows (g2 rows beyond nrow are zero)
        floatx16 c = {0};
#pragma unroll
        for (int kk = 0; kk < PR / 2; ++kk) {
            const int r = 2 * kk + half;
            const float gb = l31 < 2 * PA_MAX ? g2s[r * (2 * PA_MAX + 1) + l31] : 0.0f;
            c = __builtin_amdgcn_mfma_f32_32x32x2f32(h2[r * (H + 1) + col], gb, c, 0, 0, 0);
        }
        if (l31 < A) {
            float *o2 = thin_part + (size_t)IN * H + l31;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int n = 32 * w + 8 * (v >> 2) + 4 * half + (v & 3);
                o2[(size_t)n * A] = c[v];
            }
        }
    }
    if (t < ld) {   // column sums of the tile: bias gradient of the head, log_std gradient
        float cs2 = 0.0f;
        for (int r = 0; r < PR; ++r) cs2 += g2s[r * (2 * PA_MAX + 1) + t];
        if (t < A) db_part[2 * H + t] = cs2;
        else ls_part[(long)blockIdx.x * A + (t - A)] = cs2;
    }
    if constexpr (H == 64) {
        // Hidden width 64: the hidden layer's weight gradient of the tile, dW1[k][n] = sum_r h1[r][k] g1[r][n],
        // is four 32 x 32 tiles of 16 k-steps.  It is taken here, from h1 and g1 while both lie in LDS, as one
        // more per-tile piece for the sum kernel (wavefront w: columns [32w, 32w + 32)), instead of in a launch
        // of its own that reads h1 and g1 back from global memory: that launch was 10 us of a 37 us minibatch.
        __syncthreads();   // gT complete
        float *o1 = thin_part + (size_t)IN * H + (size_t)H * A;
#pragma unroll
        for (int kt = 0; kt < H / 32; ++kt) {
            floatx16 c = {0};
#pragma unroll
            for (int kk = 0; kk < PR / 2; ++kk) {
                const int r = 2 * kk + half;
                c = __builtin_amdgcn_mfma_f32_32x32x2f32(hT[(32 * kt + l31) * HT_LD + r], gT[col * HT_LD + r], c, 0, 0, 0);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int k = 32 * kt + 8 * (v >> 2) + 4 * half + (v & 3);
                o1[(size_t)k * H + col] = c[v];
            }
        }
    }
    // ---- dh1 = g1 W1^T: wavefront w owns input columns [32w, 32w + 32); the next chunk of W1 is
    // fetched into registers while the matrix cores work on the current one
    floatx16 acc = {0};
    for (int o0 = 0; o0 < H; o0 += KCH) {
        __syncthreads();   // gT complete and the activation tiles read (first round) / previous chunk consumed
#pragma unroll
        for (int q = 0; q < KCH / 8; ++q) {
            wT[(wseg + 4 * q + 0) * (H + 1) + wrow] = nxt[q].x;
            wT[(wseg + 4 * q + 1) * (H + 1) + wrow] = nxt[q].y;
            wT[(wseg + 4 * q + 2) * (H + 1) + wrow] = nxt[q].z;
            wT[(wseg + 4 * q + 3) * (H + 1) + wrow] = nxt[q].w;
        }
        __syncthreads();
        if (o0 + KCH < H) fetch(o0 + KCH);
        __builtin_amdgcn_sched_barrier(0);   // keep the loads ahead of the MFMAs that hide them
        // operands of eight k-steps are read from LDS while the previous eight are multiplied
        constexpr int G = 8;
        float a[G], b[G], na[G], nb[G];
#pragma unroll
        for (int j = 0; j < G; ++j) {
            a[j] = gT[(o0 + 2 * j + half) * HT_LD + l31];
            b[j] = wT[(2 * j + half) * (H + 1) + col];
        }
#pragma unroll
        for (int g = 0; g < KCH / 2 / G; ++g) {
            if (g + 1 < KCH / 2 / G) {
#pragma unroll
                for (int j = 0; j < G; ++j) {
                    const int k = 2 * ((g + 1) * G + j) + half;
                    na[j] = gT[(o0 + k) * HT_LD + l31];
                    nb[j] = wT[k * (H + 1) + col];
                }
            }
#pragma unroll
            for (int j = 0; j < G; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], b[j], acc, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < G; ++j) { a[j] = na[j]; b[j] = nb[j]; }
        }
    }
    float cs = 0.0f;
    float gv[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int row = 8 * (v >> 2) + 4 * half + (v & 3);
        gv[v] = row < nrow ? acc[v] * d0[v] : 0.0f;
        cs += gv[v];
    }
    // the two halves of the wavefront hold the other 16 rows of the same column
    cs += __shfl_xor(cs, 32, 64);
    if (half == 0) db_part[col] = cs;   // bias gradient of layer 0, this tile's rows
    // dW0[i][col] of the tile = sum_r x[r][i] g0[r][col]
    for (int i = 0; i < IN; ++i) {
        float s = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; ++v) s = fmaf(xs[(8 * (v >> 2) + 4 * half + (v & 3)) * XS_LD + i], gv[v], s);
        s += __shfl_xor(s, 32, 64);
        if (half == 0) thin_part[(size_t)i * H + col] = s;
    }
}

// ---------------------------------------------------------------- [dW | db] of the three layers
constexpr int DBM = 64, DBN = 64, DKC = 32, DLD = 65;

struct DwProblem {
    const float *X;   // layer input per batch row (row stride xs)
    const float *G;   // gradient at the layer's pre-activation (row stride gs)
    int xs, gs, K, N; // K inputs, N outputs: the block written is dW [K, N]
    int poff;         // offset of the layer's W in the flat parameter vector
    int tiles_n, tiles;   // tiles_n = ceil(N / 64); tiles = tiles_n * ceil(K / 64)
    int vec;              // rows of X and G can be read with 16-byte loads, K and N are multiples of 64
};
struct DwSet { DwProblem p[6]; int n; };

// dW = X^T G of every problem, split over the batch: grid.x = sum of the problems' tiles,
// grid.y = batch splits; partial[z][P].  The next 32-row chunk is fetched into registers while
// the matrix cores work on the current one.
// Workgroups go to the chip's eight XCDs in turn (workgroup n to XCD n % 8), and each XCD has an L2 of its
// own.  The tiles of one (problem, batch split) read the same rows of X and G -- every 64-column block of X
// is wanted by all tiles of its tile row, every block of G by all tiles of its tile column --, so the
// launch is a flat list of workgroups ordered so that those tiles sit on ONE XCD: the group is fetched
// from memory once and its re-reads are L2 hits (measured: 50 MB -> 17 MB fetched per launch at a
// minibatch of 4096, which is what X and G hold).  groups = problems x splits, `tiles` workgroups each
// (every problem of a launch has the same number of tiles); group g runs on XCD g % 8.
constexpr int XCDS = 8;

__global__ __launch_bounds__(256) void dw3_kernel(DwSet d, int M, int rows_per_split, int P,
                                                  float *__restrict__ partial, int splits) {
    __shared__ float As[DKC * DLD];
    __shared__ float Bs[DKC * DLD];
    const int tiles = d.p[0].tiles, groups = d.n * splits;
    // workgroup n = (round r, XCD x): the r-th workgroup that XCD x receives.  An XCD walks its groups
    // g = x, x + 8, ... one after the other, `tiles` workgroups each; with a group count that is not a
    // multiple of 8 the last round is short and its workgroups keep the plain order.
    int g, tile;
    {
        const int n = blockIdx.x, full = (groups / XCDS) * XCDS * tiles;   // workgroups of whole rounds of 8 groups
        if (n < full) {
            const int x = n % XCDS, q = n / XCDS;
            tile = q % tiles;
            g = (q / tiles) * XCDS + x;
        } else {
            const int m = n - full;
            tile = m % tiles;
            g = (groups / XCDS) * XCDS + m / tiles;
        }
    }
    const int li = g / splits, z = g % splits;
    const DwProblem &pr = d.p[li];
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wr = w >> 1, wc = w & 1;
    const int half = lane >> 5, l31 = lane & 31;
    const int j0 = (tile % pr.tiles_n) * DBN, i0 = (tile / pr.tiles_n) * DBM;
    const long b_begin = (long)z * rows_per_split;
    long b_end = b_begin + rows_per_split;
    if (b_end > M) b_end = M;
    floatx16 acc = {0};
    const int bb = t >> 3, seg = (t & 7) * 8;
    float xa[8], gb[8];
    // each thread moves 8 consecutive floats of X and of G per chunk: two 16-byte loads each when
    // the problem allows (whole tiles inside K and N, 16-byte aligned rows), scalar loads otherwise
    const bool vec = pr.vec != 0;
    auto fetch = [&](long b0) {
        const long b = b0 + bb;
        const bool inb = b < b_end;
        if (vec) {
            float4 x0 = {0, 0, 0, 0}, x1 = x0, g0 = x0, g1 = x0;
            if (inb) {
                const float4 *px = reinterpret_cast<const float4 *>(pr.X + b * pr.xs + i0 + seg);
                const float4 *pg = reinterpret_cast<const float4 *>(pr.G + b * pr.gs + j0 + seg);
                x0 = px[0]; x1 = px[1]; g0 = pg[0]; g1 = pg[1];
            }
            xa[0] = x0.x; xa[1] = x0.y; xa[2] = x0.z; xa[3] = x0.w; xa[4] = x1.x; xa[5] = x1.y; xa[6] = x1.z; xa[7] = x1.w;
            gb[0] = g0.x; gb[1] = g0.y; gb[2] = g0.z; gb[3] = g0.w; gb[4] = g1.x; gb[5] = g1.y; gb[6] = g1.z; gb[7] = g1.w;
            return;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int ii = i0 + seg + i, j = j0 + seg + i;
            xa[i] = (inb && ii < pr.K) ? pr.X[b * pr.xs + ii] : 0.0f;
            gb[i] = (inb && j < pr.N) ? pr.G[b * pr.gs + j] : 0.0f;
        }
    };
    fetch(b_begin);
    for (long b0 = b_begin; b0 < b_end; b0 += DKC) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            As[bb * DLD + seg + i] = xa[i];
            Bs[bb * DLD + seg + i] = gb[i];
        }
        __syncthreads();
        if (b0 + DKC < b_end) fetch(b0 + DKC);
        __builtin_amdgcn_sched_barrier(0);   // keep the loads ahead of the MFMAs that hide them
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
            if (row < pr.K) out[(size_t)row * pr.N + col] = acc[v];
        }
    }
}

// Flat gradient vector of each net from the pieces: weight blocks = sum over the batch splits of
// `partial`, bias rows and the log_std tail (Gaussian head) = sum over the row tiles of the column
// sums the backward-dx kernel left.  The nets' vectors lie back to back in `partial`.
struct SumNets {
    float *grads[2];
    const float *ls_part[2], *db_part[2], *thin_part[2];
    int P[2], A[2], gauss[2];
    int n, IN, H;
    int thin_stride[2];   // floats per row tile in thin_part, per net
    int hh_in_tiles;   // the H x H block is summed from the row tiles' pieces (behind dW0 and dW2) instead of `partial`
};

__global__ __launch_bounds__(256) void sum3_kernel(const float *__restrict__ partial, int splits, int Ptot,
                                                   int tiles, SumNets sn, float *__restrict__ sq_part) {
    __shared__ float red[2][4];
    const int gi = blockIdx.x * blockDim.x + threadIdx.x;
    int net = 0;
    float s = 0.0f;
    if (gi < Ptot) {
        int i = gi;
        if (sn.n > 1 && i >= sn.P[0]) { net = 1; i -= sn.P[0]; }
        const int IN = sn.IN, H = sn.H, A = sn.A[net];
        const int o1 = (IN + 1) * H, o2 = o1 + (H + 1) * H, o3 = o2 + (H + 1) * A;
        // which bias row (or the log_std tail) does i fall in?  -1: a weight
        int bias_layer = -1, j = 0;
        if (i >= IN * H && i < o1) { bias_layer = 0; j = i - IN * H; }
        else if (i >= o1 + H * H && i < o2) { bias_layer = 1; j = i - (o1 + H * H); }
        else if (i >= o2 + H * A && i < o3) { bias_layer = 2; j = i - (o2 + H * A); }
        else if (i >= o3) { bias_layer = 3; j = i - o3; }
        // n terms, `stride` floats apart, added in order; loads are issued 64 (then 16) at a time so that
        // the chain of memory round trips is that many times shorter than one dependent load per term
        // (the per-tile pieces are 128 terms at a minibatch of 4096: two round trips instead of eight)
        const float *p;
        size_t stride;
        int n;
        if (bias_layer < 0 && i >= o1 && i < o1 + H * H && sn.hh_in_tiles) {
            p = sn.thin_part[net] + (size_t)IN * H + (size_t)H * A + (i - o1);
            stride = (size_t)sn.thin_stride[net];
            n = tiles;
        }
        else if (bias_layer < 0 && i >= o1 && i < o1 + H * H) { p = partial + gi; stride = (size_t)Ptot; n = splits; }
        else if (bias_layer < 0) {   // a weight of layer 0 or of the head: per-tile pieces of the dx kernel
            p = sn.thin_part[net] + (i < o1 ? i : (size_t)IN * H + (i - o2));
            stride = (size_t)sn.thin_stride[net];
            n = tiles;
        }
        else if (bias_layer == 3) { p = sn.ls_part[net] + j; stride = (size_t)A; n = tiles; }
        else {
            p = sn.db_part[net] + (bias_layer == 0 ? 0 : (bias_layer == 1 ? H : 2 * H)) + j;
            stride = (size_t)(2 * H + PA_MAX);
            n = tiles;
        }
        int q = 0;
        for (; q + 64 <= n; q += 64) {
            float v[64];
#pragma unroll
            for (int k = 0; k < 64; ++k) v[k] = p[(size_t)(q + k) * stride];
#pragma unroll
            for (int k = 0; k < 64; ++k) s += v[k];
        }
        for (; q + 16 <= n; q += 16) {
            float v[16];
#pragma unroll
            for (int k = 0; k < 16; ++k) v[k] = p[(size_t)(q + k) * stride];
#pragma unroll
            for (int k = 0; k < 16; ++k) s += v[k];
        }
        for (; q < n; ++q) s += p[(size_t)q * stride];
        sn.grads[net][i] = s;
    }
    if (sq_part == nullptr) return;
    // per-block sums of squares, one per net (a block may straddle the two vectors): the partials
    // of the global-norm clip, sq_part[net * 1024 + block]
    float v0 = net == 0 ? s * s : 0.0f, v1 = net == 1 ? s * s : 0.0f;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v0 += __shfl_xor(v0, off, 64);
        v1 += __shfl_xor(v1, off, 64);
    }
    if ((threadIdx.x & 63) == 0) { red[0][threadIdx.x >> 6] = v0; red[1][threadIdx.x >> 6] = v1; }
    __syncthreads();
    if (threadIdx.x < 2) {
        const float *r = red[threadIdx.x];
        sq_part[threadIdx.x * 1024 + blockIdx.x] = r[0] + r[1] + r[2] + r[3];
    }
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

static int net_P(const mrl_mlp_desc &d) {
    const int IN = d.layers[0].in_dim, H = d.layers[0].out_dim, A = d.layers[2].out_dim;
    return (IN + 1) * H + (H + 1) * H + (H + 1) * A + (d.layers[2].kind == MRL_STOCHASTIC_ACTOR ? A : 0);
}

// true when the two nets can share launches: both fusable, same input width, width and activation
bool mlp3_pair_fusable(const mrl_mlp_desc &a, const mrl_mlp_desc &b) {
    int ha, hb, aa, ab;
    bool ga, gb;
    return mlp3_fusable(a, &ha, &aa, &ga) && mlp3_fusable(b, &hb, &ab, &gb) && ha == hb && aa == ab &&
           a.layers[0].in_dim == b.layers[0].in_dim;
}

template <int H, int ACT>
static void launch_fwd_t(mrl_ctx *ctx, int batch, int IN, const Mlp3Nets &nets, int n_nets, const FwdLoss &fl) {
    dim3 grid((batch + PR - 1) / PR, n_nets);
    hipLaunchKernelGGL((mlp3_fwd_kernel<H, ACT>), grid, dim3(2 * H), 0, ctx->stream, batch, IN, nets, fl);
}
template <int H, int ACT>
static void launch_bwd_t(mrl_ctx *ctx, int batch, int IN, const Mlp3Nets &nets, int n_nets, const FwdLoss *fused) {
    dim3 grid((batch + PR - 1) / PR, n_nets);
    if (fused != nullptr)
        hipLaunchKernelGGL((mlp3_fb_kernel<H, ACT>), grid, dim3(2 * H), 0, ctx->stream, batch, IN, nets, *fused);
    else
        hipLaunchKernelGGL((mlp3_bwd_dx_kernel<H, ACT>), grid, dim3(2 * H), 0, ctx->stream, batch, IN, nets);
}

// forward of one or two nets (descs[i], io.n[i]) in one launch
int mlp3_forward_n(mrl_ctx *ctx, const mrl_mlp_desc *const *descs, int n_nets, int batch, Mlp3Nets io,
                   const FwdLoss *loss) {
    int H = 0, act = 0;
    bool gauss = false;
    for (int i = 0; i < n_nets; ++i) {
        if (!mlp3_fusable(*descs[i], &H, &act, &gauss)) return MRL_E_UNSUPPORTED;
        io.n[i].A = descs[i]->layers[2].out_dim;
        io.n[i].gauss = gauss ? 1 : 0;
    }
    if (n_nets == 2 && !mlp3_pair_fusable(*descs[0], *descs[1])) return MRL_E_UNSUPPORTED;
    const int IN = descs[0]->layers[0].in_dim;
    FwdLoss fl{};
    if (loss != nullptr) {
        if (n_nets != 2 || (batch + PR - 1) / PR > 1024) return MRL_E_UNSUPPORTED;   // one KL partial per row tile
        fl = *loss;
        fl.enabled = 1;
    }
    if (H == 256 && act == 1) launch_fwd_t<256, 1>(ctx, batch, IN, io, n_nets, fl);
    else if (H == 256) launch_fwd_t<256, 2>(ctx, batch, IN, io, n_nets, fl);
    else if (act == 1) launch_fwd_t<64, 1>(ctx, batch, IN, io, n_nets, fl);
    else launch_fwd_t<64, 2>(ctx, batch, IN, io, n_nets, fl);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mlp3_forward(mrl_ctx *ctx, const mrl_mlp_desc &d, int batch, const float *in, const float *params,
                 float *out, float *cache) {
    Mlp3Nets io{};
    io.n[0].x = in; io.n[0].params = params; io.n[0].out = out; io.n[0].cache = cache;
    const mrl_mlp_desc *ds[1] = {&d};
    return mlp3_forward_n(ctx, ds, 1, batch, io);
}

// floats of workspace mlp3_backward_n needs for these nets
size_t mlp3_backward_ws(const mrl_mlp_desc *const *descs, int n_nets, int batch) {
    size_t total = 0, P = 0;
    for (int i = 0; i < n_nets; ++i) {
        const int H = descs[i]->layers[0].out_dim;
        const int IN = descs[i]->layers[0].in_dim, A = descs[i]->layers[2].out_dim;
        total += (size_t)2 * batch * H +
                 (size_t)((batch + PR - 1) / PR) * (2 * PA_MAX + 2 * H + (size_t)IN * H + (size_t)H * A +
                                                    (H == 64 ? (size_t)H * H : 0));
        P += net_P(*descs[i]);
    }
    return total + (size_t)32 * P;
}

// backward (parameter gradients only) of one or two nets: io.n[i].grad_out / params / cache in,
// grads[i] out; ws as sized by mlp3_backward_ws
int mlp3_backward_n(mrl_ctx *ctx, const mrl_mlp_desc *const *descs, int n_nets, int batch, Mlp3Nets io,
                    float *const *grads, float *ws, float *sq_part, int *sq_blocks, const FwdLoss *fused) {
    if (fused != nullptr && (n_nets != 2 || (batch + PR - 1) / PR > 1024)) return MRL_E_UNSUPPORTED;
    int H = 0, act = 0;
    bool gauss = false;
    for (int i = 0; i < n_nets; ++i) {
        if (!mlp3_fusable(*descs[i], &H, &act, &gauss)) return MRL_E_UNSUPPORTED;
        io.n[i].A = descs[i]->layers[2].out_dim;
        io.n[i].gauss = gauss ? 1 : 0;
        // the W1 rows are staged with 16-byte loads
        const int IN = descs[i]->layers[0].in_dim;
        if (reinterpret_cast<uintptr_t>(io.n[i].params + IN * H + H) % 16 != 0) return MRL_E_UNSUPPORTED;
    }
    if (n_nets == 2 && !mlp3_pair_fusable(*descs[0], *descs[1])) return MRL_E_UNSUPPORTED;
    const int IN = descs[0]->layers[0].in_dim;
    const int tiles = (batch + PR - 1) / PR;
    int splits = std::max(1, std::min(32, batch / 256));
    int rows_per = ((batch + splits - 1) / splits + DKC - 1) / DKC * DKC;
    splits = (batch + rows_per - 1) / rows_per;
    const bool hh_in_tiles = fused != nullptr && H == 64;
    // workspace: per net g1 [B, H] | g0 [B, H] | ls_part [tiles, PA_MAX] | db_part [tiles, 2H + PA_MAX] |
    // thin_part [tiles, IN H + H A]; then partial [splits, Ptot]
    float *w = ws;
    for (int i = 0; i < n_nets; ++i) {
        io.n[i].g1 = w; w += (size_t)batch * H;
        io.n[i].g0 = w; w += (size_t)batch * H;
        io.n[i].ls_part = w; w += (size_t)tiles * PA_MAX;
        io.n[i].db_part = w; w += (size_t)tiles * (2 * H + PA_MAX);
        // (the fused forward + backward kernel of the 64-wide nets leaves the tile's dW1 there as well)
        io.n[i].thin_stride = IN * H + H * descs[i]->layers[2].out_dim + (hh_in_tiles ? H * H : 0);
        io.n[i].thin_part = w; w += (size_t)tiles * (size_t)io.n[i].thin_stride;
    }
    float *partial = w;
    FwdLoss fl{};
    if (fused != nullptr) {
        fl = *fused;
        fl.enabled = 1;
        fused = &fl;
    }
    if (H == 256 && act == 1) launch_bwd_t<256, 1>(ctx, batch, IN, io, n_nets, fused);
    else if (H == 256) launch_bwd_t<256, 2>(ctx, batch, IN, io, n_nets, fused);
    else if (act == 1) launch_bwd_t<64, 1>(ctx, batch, IN, io, n_nets, fused);
    else launch_bwd_t<64, 2>(ctx, batch, IN, io, n_nets, fused);
    MRL_CHECK_LAUNCH();
    DwSet dw;
    dw.n = n_nets;   // the H x H layer of each net; the thin layers come out of the dx kernel
    SumNets sn{};
    sn.n = n_nets;
    sn.IN = IN;
    sn.H = H;
    sn.hh_in_tiles = hh_in_tiles ? 1 : 0;
    int base = 0, total_tiles = 0;
    for (int i = 0; i < n_nets; ++i) {
        const Mlp3Net &nn = io.n[i];
        const int A = nn.A;
        const float *c1 = nn.cache + (size_t)batch * (IN + H);
        DwProblem &p = dw.p[i];
        p.X = c1; p.xs = 2 * H; p.G = nn.g1; p.gs = H; p.K = H; p.N = H; p.poff = base + (IN + 1) * H;
        p.tiles_n = (H + DBN - 1) / DBN;
        p.tiles = p.tiles_n * ((H + DBM - 1) / DBM);
        p.vec = (H % 64 == 0 && reinterpret_cast<uintptr_t>(c1) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(nn.g1) % 16 == 0) ? 1 : 0;
        total_tiles += p.tiles;
        sn.grads[i] = grads[i];
        sn.ls_part[i] = nn.ls_part;
        sn.db_part[i] = nn.db_part;
        sn.thin_part[i] = nn.thin_part;
        sn.thin_stride[i] = nn.thin_stride;
        sn.P[i] = net_P(*descs[i]);
        sn.A[i] = A;
        sn.gauss[i] = nn.gauss;
        base += sn.P[i];
    }
    const int Ptot = base;
    // (both nets have the same width: every problem has the same number of tiles, see dw3_kernel)
    if (!hh_in_tiles)
        hipLaunchKernelGGL(dw3_kernel, dim3(total_tiles * splits), dim3(256), 0, ctx->stream, dw, batch, rows_per,
                           Ptot, partial, splits);
    const int sum_blocks = grid_for(Ptot, 256);
    if (sum_blocks > 1024) sq_part = nullptr;   // more partials than the caller's buffer holds
    if (sq_blocks) *sq_blocks = sq_part ? sum_blocks : 0;
    hipLaunchKernelGGL(sum3_kernel, dim3(sum_blocks), dim3(256), 0, ctx->stream, partial, splits, Ptot, tiles,
                       sn, sq_part);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

int mlp3_backward(mrl_ctx *ctx, const mrl_mlp_desc &d, int batch, const float *grad_out, const float *params,
                  const float *cache, float *grads, float *ws) {
    Mlp3Nets io{};
    io.n[0].grad_out = grad_out; io.n[0].params = params; io.n[0].cache = const_cast<float *>(cache);
    const mrl_mlp_desc *ds[1] = {&d};
    float *gs[1] = {grads};
    return mlp3_backward_n(ctx, ds, 1, batch, io, gs, ws, nullptr, nullptr);
}

}  // namespace mrl
