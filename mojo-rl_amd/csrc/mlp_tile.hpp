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
    if (ACT == 2) return tanh_mlp(x);
    return x;
}

// Where a tile's forward leaves the reference's per-layer cache (deep_rl/model/sequential.mojo:
// 104-133, blocked per layer): c0 rows [x (IN) | layer-0 pre-activation or tanh output (H)],
// c1 rows [h1 (H) | layer-1 pre-activation or tanh output (H)], c2 rows [h2 (H)].  All null:
// nothing is cached; c1 alone: only h1 is stored (what the H x H weight gradient reads).
struct TileCache {
    float *c0, *c1, *c2;
    long row0;   // first batch row of the tile
    int nrow;    // rows of the tile inside the batch
};

// Everything the hidden stack of one net needs from global memory that does not depend on the
// tile's rows: biases, the layer-0 weights, the first block of layer-1 weights.  A kernel issues
// these loads first thing (before it stages its inputs), so that a block pays the memory latency
// once rather than once per phase.
// threads that work on one net: one wavefront per TPW column tiles of 32 (the last wavefront's
// tiles beyond H are computed on repeated columns and dropped)
constexpr int hidden_threads(int H, int TPW) { return 64 * ((H / 32 + TPW - 1) / TPW); }

template <int H, int TPW, int KB>
struct HiddenOperands {
    static constexpr int K0 = PIN_MAX / 2;   // k-steps of layer 0 at the widest input
    int col[TPW];
    int ntile;   // column tiles of this wavefront that exist (TPW, or fewer on the last wavefront)
    float bias0[TPW], bias1[TPW];
    float w0[TPW][K0];
    float bv[TPW][KB];

    // tid: the caller's thread index (a caller that loops over many tiles may pass a copy the
    // optimiser cannot see through, so that nothing derived from it is kept across iterations).
    // tile0 / tiles: the column tiles of this wavefront when the caller deals them out itself
    // (tiles <= TPW of them from tile0 on); by default wavefront w takes tiles TPW w .. TPW w + TPW - 1.
    MRL_DEV void load(const float *__restrict__ p, int IN, int tid = threadIdx.x, int tile0 = -1, int tiles = 0) {
        constexpr int T = hidden_threads(H, TPW);
        const int t = tid % T, lane = tid & 63, w = t >> 6, half = lane >> 5, l31 = lane & 31;
        const float *W0 = p, *b0 = p + IN * H;
        const float *W1 = b0 + H, *b1 = W1 + H * H;
        ntile = (H / 32) % TPW == 0 ? TPW : min(TPW, H / 32 - TPW * w);
        if (tile0 < 0) tile0 = TPW * w;
        else ntile = tiles;
#pragma unroll
        for (int q = 0; q < TPW; ++q) {
            col[q] = (q < ntile && tile0 + q < H / 32 ? 32 * (tile0 + q) : 0) + l31;
            bias0[q] = b0[col[q]];
            bias1[q] = b1[col[q]];
        }
#pragma unroll
        for (int kk = 0; kk < K0; ++kk) {
            const int k = 2 * kk + half;
#pragma unroll
            for (int q = 0; q < TPW; ++q) w0[q][kk] = k < IN ? W0[k * H + col[q]] : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < KB; ++j) {
#pragma unroll
            for (int q = 0; q < TPW; ++q) bv[q][j] = W1[(2 * j + half) * H + col[q]];
        }
    }
};

// Hidden stack of one net for the block's 32 rows; leaves act(layer1) in h2[32][H+1].
// TPW = accumulator tiles (32 columns each) per wavefront: the net is worked on by 2H / TPW
// threads (threadIdx.x modulo that count picks the role), so TPW = 1 spreads the same MFMA chain
// over twice the wavefronts.  `ops` = the operands loaded ahead by the same thread.
// H2_ON_HT: h2 may share its memory with hT (the block waits until every wavefront has finished
// reading hT before the first h2 element is written).
// `sync` is what the threads working on this net wait at between the phases: the whole block by
// default; a caller that runs the net on some of its wavefronts only passes their own barrier.
struct BlockSync {
    MRL_DEV void operator()() const { __syncthreads(); }
};

// A barrier among `nwaves` wavefronts of a workgroup (all of them resident, as wavefronts of one
// workgroup always are), for phases in which the rest of the block does something else: a counter
// in LDS that only grows; every arrival adds one, and everyone waits until all arrivals of the
// current round are in.  Every wavefront of the group must call it the same number of times,
// outside divergent code.  The counter must be zero before the first use.
//
// The wait is bounded: after `spin_limit` polls without the round completing, the waiting
// wavefront raises the workgroup's `failed` word (LDS) and goes on, and so does every later wait of
// the workgroup as soon as it sees the word raised -- a wavefront that missed a round therefore costs
// the launch its results, never its end.  The kernel reports the word to the host when it exits.
struct WaveGroupSync {
    unsigned *counter;
    unsigned target;   // arrivals expected by the end of the round in progress
    unsigned nwaves;
    unsigned *failed;      // LDS word shared by the workgroup, zero before the first use
    unsigned spin_limit;   // polls of the counter before a wait gives up
    MRL_DEV void arrive() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");   // this wavefront's LDS writes are out
        if ((threadIdx.x & 63) == 0)
            __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    MRL_DEV void wait_for(unsigned arrivals) const {
        unsigned polls = 0;
        while ((int)(__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) - arrivals) < 0) {
            if (++polls > spin_limit ||
                ((polls & 255u) == 0u && __hip_atomic_load(failed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0u)) {
                __hip_atomic_store(failed, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }
    MRL_DEV void operator()() {
        target += nwaves;
        arrive();
        wait_for(target);
    }
};

// NT = the column tiles this wavefront really has (ops.ntile, known at compile time here): the
// MFMAs, weight loads and epilogues of the other TPW - NT slots are left out.
template <int H, int ACT, int TPW, int KB, bool H2_ON_HT, int NT, class Sync>
MRL_DEV void hidden_stack_tiles(const float *__restrict__ p, int IN, const float *xs, float *hT, float *h2,
                                const TileCache tc, HiddenOperands<H, TPW, KB> &ops, int tid, Sync &sync) {
    static_assert(PR * (H + 1) <= H * HT_LD, "h2 fits into hT");
    constexpr int T = hidden_threads(H, TPW);
    constexpr int K0 = PIN_MAX / 2;
    const int t = tid % T, lane = t & 63, half = lane >> 5, l31 = lane & 31;
    const float *W1 = p + IN * H + H;
    int (&col)[TPW] = ops.col;
    float (&bias0)[TPW] = ops.bias0, (&bias1)[TPW] = ops.bias1;
    float (&w0)[TPW][K0] = ops.w0;
    float (&bv)[TPW][KB] = ops.bv;
    {   // layer 0 (K = IN <= 32, padded to even with zeros): all operands first, then the MFMAs
        float a0[K0];
#pragma unroll
        for (int kk = 0; kk < K0; ++kk) {
            const int k = 2 * kk + half;
            a0[kk] = k < IN ? xs[l31 * XS_LD + k] : 0.0f;
        }
        floatx16 c[TPW];
#pragma unroll
        for (int q = 0; q < NT; ++q) c[q] = floatx16{0};
#pragma unroll
        for (int kk = 0; kk < K0; ++kk) {
            if (2 * kk < IN) {
#pragma unroll
                for (int q = 0; q < NT; ++q)
                    c[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[kk], w0[q][kk], c[q], 0, 0, 0);
            }
        }
#pragma unroll
        for (int q = 0; q < NT; ++q) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = 8 * (v >> 2) + 4 * half + (v & 3);
                const float pre = c[q][v] + bias0[q];
                const float y = activate<ACT>(pre);
                hT[col[q] * HT_LD + row] = y;
                if (tc.c1 != nullptr && row < tc.nrow) {
                    if (tc.c0 != nullptr) tc.c0[(tc.row0 + row) * (IN + H) + IN + col[q]] = ACT == 1 ? pre : y;
                    tc.c1[(tc.row0 + row) * (2 * H) + col[q]] = y;
                }
            }
        }
    }
    sync();
    {   // layer 1 (H x H): weights streamed from L2 one block of KB k-steps ahead of the MFMAs
        floatx16 c[TPW];
#pragma unroll
        for (int q = 0; q < NT; ++q) c[q] = floatx16{0};
        float a[KB], na[KB], nb[TPW][KB];
#pragma unroll
        for (int j = 0; j < KB; ++j) a[j] = hT[(2 * j + half) * HT_LD + l31];
        for (int blk = 0; blk < H / (2 * KB); ++blk) {
            const bool more = blk + 1 < H / (2 * KB);
            if (more) {
#pragma unroll
                for (int j = 0; j < KB; ++j) {
                    const int k = 2 * ((blk + 1) * KB + j) + half;
                    na[j] = hT[k * HT_LD + l31];
#pragma unroll
                    for (int q = 0; q < NT; ++q) nb[q][j] = W1[k * H + col[q]];
                }
            }
            // the next block's loads stay ahead of this block's MFMAs (left alone, the scheduler moves
            // them behind the MFMAs, next to their first use, and their latency is no longer hidden)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < KB; ++j) {
#pragma unroll
                for (int q = 0; q < NT; ++q)
                    c[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], bv[q][j], c[q], 0, 0, 0);
            }
            if (more) {
#pragma unroll
                for (int j = 0; j < KB; ++j) {
                    a[j] = na[j];
#pragma unroll
                    for (int q = 0; q < NT; ++q) bv[q][j] = nb[q][j];
                }
            }
        }
        if (H2_ON_HT) sync();
#pragma unroll
        for (int q = 0; q < NT; ++q) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = 8 * (v >> 2) + 4 * half + (v & 3);
                const float pre = c[q][v] + bias1[q];
                const float y = activate<ACT>(pre);
                h2[row * (H + 1) + col[q]] = y;
                if (tc.c2 != nullptr && row < tc.nrow) {
                    tc.c1[(tc.row0 + row) * (2 * H) + H + col[q]] = ACT == 1 ? pre : y;
                    tc.c2[(tc.row0 + row) * H + col[q]] = y;
                }
            }
        }
    }
    sync();
}

template <int H, int ACT, int TPW = 2, int KB = (TPW == 2 ? 8 : 32), bool H2_ON_HT = false, class Sync = BlockSync>
MRL_DEV void hidden_stack(const float *__restrict__ p, int IN, const float *xs, float *hT, float *h2,
                          const TileCache tc, HiddenOperands<H, TPW, KB> &ops, int tid = threadIdx.x,
                          Sync &&sync = Sync()) {
    // ops.ntile is the same for all lanes of a wavefront; a wavefront with fewer tiles than slots
    // runs the variant without the spare slots' work (every variant meets the same barriers)
    if (ops.ntile >= TPW) return hidden_stack_tiles<H, ACT, TPW, KB, H2_ON_HT, TPW>(p, IN, xs, hT, h2, tc, ops, tid, sync);
    if constexpr (TPW >= 3) {
        if (ops.ntile == 2) return hidden_stack_tiles<H, ACT, TPW, KB, H2_ON_HT, 2>(p, IN, xs, hT, h2, tc, ops, tid, sync);
    }
    if constexpr (TPW >= 2) {
        if (ops.ntile == 1) return hidden_stack_tiles<H, ACT, TPW, KB, H2_ON_HT, 1>(p, IN, xs, hT, h2, tc, ops, tid, sync);
    }
    hidden_stack_tiles<H, ACT, TPW, KB, H2_ON_HT, 0>(p, IN, xs, hT, h2, tc, ops, tid, sync);
}

// floats of LDS that hold one net's head parameters, every row padded to PA_MAX columns with
// zeros: [W2 (H x PA_MAX) | b2 (PA_MAX) | log_std (PA_MAX)]; the array must be 16-byte aligned
constexpr int HEAD_LDS(int H) { return (H + 2) * PA_MAX; }
constexpr int HEAD_B2(int H) { return H * PA_MAX; }
constexpr int HEAD_LOG_STD(int H) { return (H + 1) * PA_MAX; }

// copies the head parameters of a net into LDS (call by `nthreads` threads with 0 <= t < nthreads,
// early in the kernel: the head then never waits on global memory).  The padding lets head() read
// whole rows with two 16-byte loads and no test on A.
MRL_DEV void stage_head(const float *__restrict__ W2, int H, int A, bool with_log_std, float *w2s, int t,
                        int nthreads) {
    const int rows = H + 1 + (with_log_std ? 1 : 0);   // the parameters are [H + 1 (+ 1)][A], row-major
    const int total = rows * PA_MAX;
    for (int i0 = t; i0 < total; i0 += 4 * nthreads) {   // four independent loads in flight per thread
        float v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int i = i0 + k * nthreads, n = i / PA_MAX, a = i % PA_MAX;
            v[k] = (i < total && a < A) ? W2[n * A + a] : 0.0f;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (i0 + k * nthreads < total) w2s[i0 + k * nthreads] = v[k];
    }
}

// out[r][a] = h2[r] . W2[:, a] + b2[a] for the block's rows; TPR = H/16 lanes cooperate per row,
// each over 16 consecutive columns that it walks from a different starting point (the lanes of a
// wavefront then spread over the LDS banks, for the activations and for the padded weight rows
// alike), and add their sums up in a butterfly.  The result does not depend on how many threads
// share the work: the 2 H (row, part) pairs are dealt out nthreads at a time.
// w2s: the head parameters in LDS (stage_head).
// NA = outputs carried per lane (1, 4 or 8 >= A): narrower heads read less of each padded row.
template <int H, int NA>
MRL_DEV void head_rows(const float *w2s, int A, const float *h2, float *out, int out_ld, int t, int nthreads) {
    constexpr int CP = 16, TPR = H / CP;
    static_assert(64 % TPR == 0, "the lanes of a row sit in one wavefront");
    static_assert(PA_MAX == 8 && (NA == 1 || NA == 4 || NA == 8), "one float, one float4 or two per padded row");
    const float *b2 = w2s + HEAD_B2(H);
    // nthreads must be a multiple of TPR
    for (int pair = t; pair < PR * TPR; pair += nthreads) {
        const int r = pair / TPR, part = pair % TPR;
        float acc[NA];
#pragma unroll
        for (int a = 0; a < NA; ++a) acc[a] = 0.0f;
#pragma unroll 8
        for (int i = 0; i < CP; ++i) {
            const int n = part * CP + ((i + part) & (CP - 1));
            const float hv = h2[r * (H + 1) + n];
            if (NA == 1) {
                acc[0] = fmaf(hv, w2s[n * PA_MAX], acc[0]);
            } else {
                const float4 wa = *reinterpret_cast<const float4 *>(w2s + n * PA_MAX);
                acc[0] = fmaf(hv, wa.x, acc[0]); acc[1] = fmaf(hv, wa.y, acc[1]);
                acc[2] = fmaf(hv, wa.z, acc[2]); acc[3] = fmaf(hv, wa.w, acc[3]);
                if (NA == 8) {
                    const float4 wb = *reinterpret_cast<const float4 *>(w2s + n * PA_MAX + 4);
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

// t = index of the calling thread among the `nthreads` (a multiple of H / 16) that share the work;
// by default the first H threads of the net call it, two (row, part) pairs each
template <int H>
MRL_DEV void head(const float *w2s, int A, const float *h2, float *out, int out_ld, int t = threadIdx.x % H,
                  int nthreads = H) {
    if (A == 1) head_rows<H, 1>(w2s, A, h2, out, out_ld, t, nthreads);
    else if (A <= 4) head_rows<H, 4>(w2s, A, h2, out, out_ld, t, nthreads);
    else head_rows<H, 8>(w2s, A, h2, out, out_ld, t, nthreads);
}

}  // namespace mrl
