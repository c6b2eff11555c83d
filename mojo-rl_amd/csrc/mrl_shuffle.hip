// The reference's host shuffle -- Fisher-Yates over the indices 0 .. n-1, driven by draws of
// random_float64() (core/utils/shuffle.mojo:21-48, inline in deep_agents/ppo/ppo.mojo:2425-2434) --
// on uniforms that the caller supplies, with the same result index for index, computed in parallel.
//
// The serial loop is  for i = n-1 .. 1:  j_i = min(Int(u_i * Float64(i + 1)), i);  a[i] <-> a[j_i].
// Position i is final once iteration i has run (later iterations only touch positions below i), and it
// receives whatever position j_i holds at that moment.  A position p holds its initial value p until an
// iteration i' > p with j_i' = p drops the old content of position i' there.  So the value that ends at
// position i is found by walking "who wrote this position last before now" links:
//     p = j_i, t = i;  while there is an i' > t with j_i' = p:  take the smallest such i', p = t = i';
//     result[i] = p.
// (Iterations run downwards, so the smallest i' above t is the most recent writer.)  The set
// {i' : j_i' = p} is bucket p of a counting sort of the iterations by target; a bucket holds ln(n / p)
// entries on average, so a walk step scans a handful of entries and a walk is O(log n) steps long.
// Off the hot path: the update draws its permutations with mrl_permutation; this entry point exists so
// that a caller holding the reference's random stream gets the reference's minibatches.
#include "mrl_host.hpp"
#include "mrl_device.hpp"

namespace mrl {

constexpr int STPB = 256;

// target of iteration i (1 <= i < n); the draws are consumed in loop order, u[0] by i = n - 1
MRL_DEV int fy_target(const double *__restrict__ u, int n, int i) {
    int j = (int)(u[n - 1 - i] * (double)(i + 1));   // the conversion saturates; NaN gives 0
    if (j > i) j = i;                                // shuffle.mojo:42-43
    if (j < 0) j = 0;                                // a draw below 0 is not a uniform: stay inside the array
    return j;
}

__global__ __launch_bounds__(STPB) void fy_zero_kernel(int32_t *__restrict__ cnt, int n1) {
    const int i = blockIdx.x * STPB + threadIdx.x;
    if (i < n1) cnt[i] = 0;
}

__global__ __launch_bounds__(STPB) void fy_count_kernel(const double *__restrict__ u, int n,
                                                        int32_t *__restrict__ cnt) {
    const int i = blockIdx.x * STPB + threadIdx.x + 1;
    if (i < n) atomicAdd(&cnt[fy_target(u, n, i)], 1);
}

// inclusive prefix sum of cnt[0 .. n) in place (cnt[p] = end of bucket p), cnt[n] = the total;
// one workgroup walks the array in chunks of 4 elements per thread
constexpr int SCAN_T = 1024, SCAN_PER = 4;
__global__ __launch_bounds__(SCAN_T) void fy_scan_kernel(int32_t *__restrict__ cnt, int n) {
    __shared__ int32_t wsum[SCAN_T / 64];
    __shared__ int32_t carry_s;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (threadIdx.x == 0) carry_s = 0;
    __syncthreads();
    for (int base = 0; base < n; base += SCAN_T * SCAN_PER) {
        const int at = base + threadIdx.x * SCAN_PER;
        int32_t v[SCAN_PER];
#pragma unroll
        for (int k = 0; k < SCAN_PER; ++k) v[k] = at + k < n ? cnt[at + k] : 0;
#pragma unroll
        for (int k = 1; k < SCAN_PER; ++k) v[k] += v[k - 1];
        int32_t incl = v[SCAN_PER - 1];
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int32_t o = __shfl_up(incl, off, 64);
            if (lane >= off) incl += o;
        }
        if (lane == 63) wsum[w] = incl;
        __syncthreads();
        int32_t before = carry_s;
        for (int k = 0; k < w; ++k) before += wsum[k];
        before += incl - v[SCAN_PER - 1];
#pragma unroll
        for (int k = 0; k < SCAN_PER; ++k)
            if (at + k < n) cnt[at + k] = v[k] + before;
        __syncthreads();
        if (threadIdx.x == SCAN_T - 1) carry_s = before + v[SCAN_PER - 1];
        __syncthreads();
    }
    if (threadIdx.x == 0) cnt[n] = carry_s;
}

// bucket[--cnt[j_i]] = i: afterwards cnt[p] is the start of bucket p and cnt[p + 1] its end
__global__ __launch_bounds__(STPB) void fy_fill_kernel(const double *__restrict__ u, int n,
                                                       int32_t *__restrict__ cnt, int32_t *__restrict__ bucket) {
    const int i = blockIdx.x * STPB + threadIdx.x + 1;
    if (i < n) bucket[atomicSub(&cnt[fy_target(u, n, i)], 1) - 1] = i;
}

// the smallest iteration above t that targets position p, or -1
MRL_DEV int fy_writer_after(const int32_t *__restrict__ cnt, const int32_t *__restrict__ bucket, int p, int t) {
    int best = 0x7fffffff;
    for (int k = cnt[p], e = cnt[p + 1]; k < e; ++k) {
        const int x = bucket[k];
        if (x > t && x < best) best = x;
    }
    return best == 0x7fffffff ? -1 : best;
}

__global__ __launch_bounds__(STPB) void fy_walk_kernel(const double *__restrict__ u, int n,
                                                       const int32_t *__restrict__ cnt,
                                                       const int32_t *__restrict__ bucket,
                                                       int32_t *__restrict__ indices) {
    const int i = blockIdx.x * STPB + threadIdx.x;
    if (i >= n) return;
    int p = i == 0 ? 0 : fy_target(u, n, i);
    int q = fy_writer_after(cnt, bucket, p, i);
    // every step moves to a strictly larger position, so the walk ends after fewer than n steps
    while (q >= 0) {
        p = q;
        q = fy_writer_after(cnt, bucket, p, p);
    }
    indices[i] = p;
}

}  // namespace mrl

using namespace mrl;

extern "C" {

int mrl_permutation_from_uniforms(mrl_ctx *ctx, int32_t *indices, int n, const double *uniforms,
                                  int32_t *workspace) {
    MRL_CHECK_ARG(ctx, "mrl_permutation_from_uniforms: ctx is NULL");
    MRL_CHECK_ARG(n >= 0 && n <= (1 << 30), "mrl_permutation_from_uniforms: n = %d out of range", n);
    if (n == 0) return MRL_OK;
    MRL_CHECK_ARG(indices && workspace, "mrl_permutation_from_uniforms: NULL buffer");
    MRL_CHECK_ARG(n == 1 || uniforms, "mrl_permutation_from_uniforms: NULL uniforms");
    int32_t *cnt = workspace, *bucket = workspace + n + 1;
    hipLaunchKernelGGL(fy_zero_kernel, dim3(grid_for(n + 1, STPB)), dim3(STPB), 0, ctx->stream, cnt, n + 1);
    if (n > 1) {
        hipLaunchKernelGGL(fy_count_kernel, dim3(grid_for(n - 1, STPB)), dim3(STPB), 0, ctx->stream, uniforms, n, cnt);
        hipLaunchKernelGGL(fy_scan_kernel, dim3(1), dim3(SCAN_T), 0, ctx->stream, cnt, n);
        hipLaunchKernelGGL(fy_fill_kernel, dim3(grid_for(n - 1, STPB)), dim3(STPB), 0, ctx->stream, uniforms, n, cnt,
                           bucket);
    }
    hipLaunchKernelGGL(fy_walk_kernel, dim3(grid_for(n, STPB)), dim3(STPB), 0, ctx->stream, uniforms, n, cnt, bucket,
                       indices);
    MRL_CHECK_LAUNCH();
    return MRL_OK;
}

}  // extern "C"
