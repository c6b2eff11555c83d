// One 32-row tile of a three-layer MLP  IN -> H -> H -> out  on the fp32 matrix cores, shared by
// the fused rollout policy kernel and the fused forward / backward kernels of the update.
//   layers 0 and 1: v_mfma_f32_32x32x2_f32, each wavefront owns 64 output columns (two accumulator
//                   tiles), A operand from LDS, B operand (the weights) streamed from L2 a block
//                   of k-steps ahead of the MFMAs that use it;
//   layer 2 (N <= 8): H/32 lanes per row, shuffle reduction.
#pragma once
#include "mrl_device.hpp"

namespace mrl {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int PR = 32;        // rows (envs) per workgroup
constexpr int PIN_MAX = 32;   // max observation width
constexpr int PA_MAX = 8;     // max number of discrete actions
constexpr int XS_LD = PIN_MAX + 1;
constexpr int HT_LD = PR + 1;

template <int ACT>
MRL_DEV float activate(float x) {
    if (ACT == 1) return x > 0.0f ? x : 0.0f;
    if (ACT == 2) return tanhf(x);
    return x;
}

// Where a tile's forward leaves the reference's per-layer cache (deep_rl/model/sequential.mojo:
// 104-133, blocked per layer): c0 rows [x (IN) | layer-0 pre-activation or tanh output (H)],
// c1 rows [h1 (H) | layer-1 pre-activation or tanh output (H)], c2 rows [h2 (H)].  c0 == nullptr:
// nothing is cached.
struct TileCache {
    float *c0, *c1, *c2;
    long row0;   // first batch row of the tile
    int nrow;    // rows of the tile inside the batch
};

// hidden stack of one net for the block's 32 rows; leaves act(layer1) in h2[32][H+1]
template <int H, int ACT>
MRL_DEV void hidden_stack(const float *__restrict__ p, int IN, const float *xs, float *hT, float *h2,
                          const TileCache tc) {
    const int t = threadIdx.x % H, lane = t & 63, w = t >> 6, half = lane >> 5, l31 = lane & 31;
    const float *W0 = p, *b0 = p + IN * H;
    const float *W1 = b0 + H, *b1 = W1 + H * H;
    const int col0 = 64 * w + l31, col1 = col0 + 32;
    {   // layer 0 (K = IN <= 32, padded to even with zeros): wavefront w owns columns [64w, 64w + 64)
        floatx16 c0 = {0}, c1 = {0};
        for (int kk = 0; kk < (IN + 1) / 2; ++kk) {
            const int k = 2 * kk + half;
            const bool in = k < IN;
            const float a = in ? xs[l31 * XS_LD + k] : 0.0f;
            const float bv0 = in ? W0[k * H + col0] : 0.0f;
            const float bv1 = in ? W0[k * H + col1] : 0.0f;
            c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bv0, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bv1, c1, 0, 0, 0);
        }
        const float bb0 = b0[col0], bb1 = b0[col1];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = 8 * (v >> 2) + 4 * half + (v & 3);
            const float p0 = c0[v] + bb0, p1 = c1[v] + bb1;
            const float y0 = activate<ACT>(p0), y1 = activate<ACT>(p1);
            hT[col0 * HT_LD + row] = y0;
            hT[col1 * HT_LD + row] = y1;
            if (tc.c0 != nullptr && row < tc.nrow) {
                float *q0 = tc.c0 + (tc.row0 + row) * (IN + H) + IN, *q1 = tc.c1 + (tc.row0 + row) * (2 * H);
                q0[col0] = ACT == 1 ? p0 : y0; q0[col1] = ACT == 1 ? p1 : y1;
                q1[col0] = y0; q1[col1] = y1;
            }
        }
    }
    __syncthreads();
    {   // layer 1 (H x H): weights streamed from L2 one block of KB k-steps ahead of the MFMAs
        constexpr int KB = 8;
        floatx16 c0 = {0}, c1 = {0};
        const float *Wc = W1 + col0;
        float a[KB], bv0[KB], bv1[KB], na[KB], nb0[KB], nb1[KB];
#pragma unroll
        for (int j = 0; j < KB; ++j) {
            const int k = 2 * j + half;
            a[j] = hT[k * HT_LD + l31];
            bv0[j] = Wc[k * H];
            bv1[j] = Wc[k * H + 32];
        }
        for (int blk = 0; blk < H / (2 * KB); ++blk) {
            const bool more = blk + 1 < H / (2 * KB);
            if (more) {
#pragma unroll
                for (int j = 0; j < KB; ++j) {
                    const int k = 2 * ((blk + 1) * KB + j) + half;
                    na[j] = hT[k * HT_LD + l31];
                    nb0[j] = Wc[k * H];
                    nb1[j] = Wc[k * H + 32];
                }
            }
#pragma unroll
            for (int j = 0; j < KB; ++j) {
                c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], bv0[j], c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], bv1[j], c1, 0, 0, 0);
            }
            if (more) {
#pragma unroll
                for (int j = 0; j < KB; ++j) { a[j] = na[j]; bv0[j] = nb0[j]; bv1[j] = nb1[j]; }
            }
        }
        const float bb0 = b1[col0], bb1 = b1[col1];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = 8 * (v >> 2) + 4 * half + (v & 3);
            const float p0 = c0[v] + bb0, p1 = c1[v] + bb1;
            const float y0 = activate<ACT>(p0), y1 = activate<ACT>(p1);
            h2[row * (H + 1) + col0] = y0;
            h2[row * (H + 1) + col1] = y1;
            if (tc.c0 != nullptr && row < tc.nrow) {
                float *q1 = tc.c1 + (tc.row0 + row) * (2 * H) + H, *q2 = tc.c2 + (tc.row0 + row) * H;
                q1[col0] = ACT == 1 ? p0 : y0; q1[col1] = ACT == 1 ? p1 : y1;
                q2[col0] = y0; q2[col1] = y1;
            }
        }
    }
    __syncthreads();
}

// out[r][a] = h2[r] . W2[:, a] + b2[a] for the block's rows; TPR = H/32 lanes cooperate per row
template <int H>
MRL_DEV void head(const float *__restrict__ W2, int A, const float *h2, float *out, int out_ld) {
    constexpr int TPR = H / PR;
    const int t = threadIdx.x % H, r = t / TPR, part = t % TPR;
    const float *b2 = W2 + H * A;
    float acc[PA_MAX];
#pragma unroll
    for (int a = 0; a < PA_MAX; ++a) acc[a] = 0.0f;
    for (int i = 0; i < PR; ++i) {
        const int n = i * TPR + part;
        const float hv = h2[r * (H + 1) + n];
#pragma unroll
        for (int a = 0; a < PA_MAX; ++a)
            if (a < A) acc[a] = fmaf(hv, W2[n * A + a], acc[a]);
    }
#pragma unroll
    for (int a = 0; a < PA_MAX; ++a) {
        float v = acc[a];
#pragma unroll
        for (int off = TPR / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
        if (part == 0 && a < A) out[r * out_ld + a] = v + b2[a];
    }
}

}  // namespace mrl
