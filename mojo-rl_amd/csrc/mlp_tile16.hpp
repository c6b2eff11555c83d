// The hidden stack and head of mlp_tile.hpp for a tile of 16 rows instead of 32:
// v_mfma_f32_16x16x4_f32, each wavefront owning NT tiles of 16 output columns.
//
// The fp32 matrix instructions accumulate their k products as one serial chain of fused
// multiply-adds in ascending k, whatever the tile shape, so with the k-steps taken in ascending
// order this tile gives the same bits as the 32-row tile (and as a serial fmaf loop): a kernel may
// pick the tile height that suits its launch without changing results.
//
// Operand layout of v_mfma_f32_16x16x4_f32, lane = 16 g + n:
//   A[row n][k g], B[k g][column n]  ->  D[row 4 g + v][column n], v = 0 .. 3.
// The columns of a wavefront start at c0; its first four tiles interleave (tile q holds columns
// c0 + 4 n + q), so that one 16-byte load per k-step fetches the B operands of all four from one
// contiguous 256-byte run of the weight row; a fifth tile holds c0 + 64 + n, a fifth and sixth
// together c0 + 64 + 2 n + (q - 4), one 8-byte load.
#pragma once
#include "mlp_tile.hpp"

namespace mrl {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int PR16 = 16;            // rows per tile
constexpr int HT16_LD = PR16 + 1;   // k-major activations hT[k][row]

template <int NT>
MRL_DEV int tile16_col(int c0, int q, int n) {
    static_assert(NT >= 1 && NT <= 6, "one to six column tiles per wavefront");
    if (NT <= 4 || q < 4) return c0 + (NT >= 4 ? 4 * n + q : NT * n + q);
    return NT == 5 ? c0 + 64 + n : c0 + 64 + 2 * n + (q - 4);
}

// B operands of one k-step: weight row `wk` (points at column c0 of row k), lane column index n
template <int NT>
MRL_DEV void tile16_load_b(const float *__restrict__ wk, int n, float (&b)[NT]) {
    if constexpr (NT >= 4) {
        const float4 v = *reinterpret_cast<const float4 *>(wk + 4 * n);
        b[0] = v.x; b[1] = v.y; b[2] = v.z; b[3] = v.w;
        if constexpr (NT == 5) b[4] = wk[64 + n];
        if constexpr (NT == 6) {
            const float2 x = *reinterpret_cast<const float2 *>(wk + 64 + 2 * n);
            b[4] = x.x; b[5] = x.y;
        }
    } else {
#pragma unroll
        for (int q = 0; q < NT; ++q) b[q] = wk[NT * n + q];
    }
}

// Row-independent operands of the hidden stack (biases, layer-0 weights, first block of layer-1
// weights), requested before the tile's rows are staged.  IN = input width (compile time here).
template <int H, int IN, int NT, int KB>
struct Hidden16Operands {
    static constexpr int K0 = (IN + 3) / 4;
    float bias0[NT], bias1[NT];
    float w0[K0][NT];
    float bv[KB][NT];
    MRL_DEV void load(const float *__restrict__ p, int c0, int lane) {
        const int g = lane >> 4, n = lane & 15;
        const float *W0 = p, *b0 = p + IN * H;
        const float *W1 = b0 + H, *b1 = W1 + H * H;
#pragma unroll
        for (int q = 0; q < NT; ++q) {
            const int col = tile16_col<NT>(c0, q, n);
            bias0[q] = b0[col];
            bias1[q] = b1[col];
        }
#pragma unroll
        for (int kk = 0; kk < K0; ++kk) {
            const int k = 4 * kk + g;
            if (k < IN) {
                tile16_load_b<NT>(W0 + k * H + c0, n, w0[kk]);
            } else {
#pragma unroll
                for (int q = 0; q < NT; ++q) w0[kk][q] = 0.0f;
            }
        }
#pragma unroll
        for (int j = 0; j < KB; ++j) tile16_load_b<NT>(W1 + (4 * j + g) * H + c0, n, bv[j]);
    }
};

// Hidden stack of one net for the block's 16 rows on the wavefronts that share it (each with its
// own c0 / NT; `lane` = lane of the calling wavefront).  xs[16][XS_LD] holds the inputs, hT
// [H][HT16_LD] receives act(layer 0) k-major, h2 [16][H + 1] act(layer 1) row-major; h2 may share
// its memory with hT (H2_ON_HT: everyone has finished reading hT before h2 is written).  sync() is
// the barrier of the wavefronts that work on this net.
template <int H, int IN, int ACT, int NT, int KB, bool H2_ON_HT, class Sync>
MRL_DEV void hidden_stack16(const float *__restrict__ p, const float *xs, float *hT, float *h2,
                            Hidden16Operands<H, IN, NT, KB> &ops, int c0, int lane, Sync &sync) {
    static_assert(PR16 * (H + 1) <= H * HT16_LD, "h2 fits into hT");
    static_assert((H / 4) % KB == 0, "whole blocks of k-steps");
    constexpr int K0 = (IN + 3) / 4;
    const int g = lane >> 4, n = lane & 15;
    const float *W1 = p + IN * H + H;
    {   // layer 0
        float a0[K0];
#pragma unroll
        for (int kk = 0; kk < K0; ++kk) {
            const int k = 4 * kk + g;
            a0[kk] = k < IN ? xs[n * XS_LD + k] : 0.0f;
        }
        floatx4 c[NT];
#pragma unroll
        for (int q = 0; q < NT; ++q) c[q] = floatx4{0};
#pragma unroll
        for (int kk = 0; kk < K0; ++kk) {
#pragma unroll
            for (int q = 0; q < NT; ++q)
                c[q] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[kk], ops.w0[kk][q], c[q], 0, 0, 0);
        }
#pragma unroll
        for (int q = 0; q < NT; ++q) {
            const int col = tile16_col<NT>(c0, q, n);
#pragma unroll
            for (int v = 0; v < 4; ++v) hT[col * HT16_LD + 4 * g + v] = activate<ACT>(c[q][v] + ops.bias0[q]);
        }
    }
    sync();
    {   // layer 1: weights streamed from L2 one block of KB k-steps ahead of the MFMAs
        floatx4 c[NT];
#pragma unroll
        for (int q = 0; q < NT; ++q) c[q] = floatx4{0};
        float a[KB], na[KB], nb[KB][NT];
#pragma unroll
        for (int j = 0; j < KB; ++j) a[j] = hT[(4 * j + g) * HT16_LD + n];
        constexpr int NBLK = H / (4 * KB);
        for (int blk = 0; blk < NBLK; ++blk) {
            const bool more = blk + 1 < NBLK;
            if (more) {
#pragma unroll
                for (int j = 0; j < KB; ++j) {
                    const int k = 4 * ((blk + 1) * KB + j) + g;
                    na[j] = hT[k * HT16_LD + n];
                    tile16_load_b<NT>(W1 + k * H + c0, n, nb[j]);
                }
            }
            // keep the next block's loads ahead of this block's MFMAs
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < KB; ++j) {
#pragma unroll
                for (int q = 0; q < NT; ++q)
                    c[q] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], ops.bv[j][q], c[q], 0, 0, 0);
            }
            if (more) {
#pragma unroll
                for (int j = 0; j < KB; ++j) {
                    a[j] = na[j];
#pragma unroll
                    for (int q = 0; q < NT; ++q) ops.bv[j][q] = nb[j][q];
                }
            }
        }
        if (H2_ON_HT) sync();
#pragma unroll
        for (int q = 0; q < NT; ++q) {
            const int col = tile16_col<NT>(c0, q, n);
#pragma unroll
            for (int v = 0; v < 4; ++v) h2[(4 * g + v) * (H + 1) + col] = activate<ACT>(c[q][v] + ops.bias1[q]);
        }
    }
    sync();
}

// head_rows of mlp_tile.hpp for 16 rows; PITCH = floats per padded weight row in w2s (PA_MAX for a
// head staged with stage_head, 1 for a single-output head stored as a plain column followed by its
// bias).  Same lane split per row and same butterfly, hence the same bits as head_rows.
template <int H, int NA, int PITCH>
MRL_DEV void head_rows16(const float *w2s, int A, const float *h2, float *out, int out_ld, int t, int nthreads) {
    constexpr int CP = 16, TPR = H / CP;
    static_assert(64 % TPR == 0, "the lanes of a row sit in one wavefront");
    static_assert(NA == 1 || (PITCH == PA_MAX && (NA == 4 || NA == 8)), "one float, one float4 or two per padded row");
    const float *b2 = w2s + H * PITCH;
    for (int pair = t; pair < PR16 * TPR; pair += nthreads) {
        const int r = pair / TPR, part = pair % TPR;
        float acc[NA];
#pragma unroll
        for (int a = 0; a < NA; ++a) acc[a] = 0.0f;
#pragma unroll 8
        for (int i = 0; i < CP; ++i) {
            const int nn = part * CP + ((i + part) & (CP - 1));
            const float hv = h2[r * (H + 1) + nn];
            if (NA == 1) {
                acc[0] = fmaf(hv, w2s[nn * PITCH], acc[0]);
            } else {
                const float4 wa = *reinterpret_cast<const float4 *>(w2s + nn * PITCH);
                acc[0] = fmaf(hv, wa.x, acc[0]); acc[1] = fmaf(hv, wa.y, acc[1]);
                acc[2] = fmaf(hv, wa.z, acc[2]); acc[3] = fmaf(hv, wa.w, acc[3]);
                if (NA == 8) {
                    const float4 wb = *reinterpret_cast<const float4 *>(w2s + nn * PITCH + 4);
                    acc[4] = fmaf(hv, wb.x, acc[4]); acc[5] = fmaf(hv, wb.y, acc[5]);
                    acc[6] = fmaf(hv, wb.z, acc[6]); acc[7] = fmaf(hv, wb.w, acc[7]);
                }
            }
        }
#pragma unroll
        for (int a = 0; a < NA; ++a) {
            float v = acc[a];
#pragma unroll
            for (int off = TPR / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
            if (part == 0 && a < A) out[r * out_ld + a] = v + b2[a];
        }
    }
}

template <int H>
MRL_DEV void head16(const float *w2s, int A, const float *h2, float *out, int out_ld, int t, int nthreads) {
    if (A == 1) head_rows16<H, 1, PA_MAX>(w2s, A, h2, out, out_ld, t, nthreads);
    else if (A <= 4) head_rows16<H, 4, PA_MAX>(w2s, A, h2, out, out_ld, t, nthreads);
    else head_rows16<H, 8, PA_MAX>(w2s, A, h2, out, out_ld, t, nthreads);
}

}  // namespace mrl
