// Probe: how do a vector-bound wavefront and a matrix-bound wavefront share a SIMD on gfx950?
// One workgroup of eight wavefronts; masks pick which wavefronts run a chain of dependent v_fma_f32
// and which run v_mfma_f32 back to back; every wavefront reports its SIMD and its elapsed clock.
// Not part of the library: it backs the choice between one and two collection workgroups per CU.
//   hipcc --offload-arch=gfx950 -O2 -ffp-contract=off simd_sharing.hip -o simd_sharing && ./simd_sharing
#include <hip/hip_runtime.h>
#include <stdio.h>
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
__global__ __launch_bounds__(512) void k(int mfma_mask, int valu_mask, int iters, long long *out, unsigned *simd, float *sink, int big) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) simd[wave] = (__builtin_amdgcn_s_getreg(63492) >> 4) & 3;
    __syncthreads();
    long long t0 = clock64();
    float r = 0.0f;
    if ((valu_mask >> wave) & 1) {
        float x = (float)lane * 0.001f, a = 1.0001f, b = 0.5f;
        for (int i = 0; i < iters; ++i) {
#pragma unroll
            for (int j = 0; j < 64; ++j) x = fmaf(x, a, b);
        }
        r = x;
    } else if ((mfma_mask >> wave) & 1) {
        if (big) {
            floatx16 c0 = {0}, c1 = {0};
            float a = (float)lane, b = 1.0f;
            for (int i = 0; i < iters; ++i) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c0, 0, 0, 0);
                    c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c1, 0, 0, 0);
                }
            }
            r = c0[0] + c1[3];
        } else {
            floatx4 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
            float a = (float)lane, b = 1.0f;
            for (int i = 0; i < iters; ++i) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    c0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c0, 0, 0, 0);
                    c1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c1, 0, 0, 0);
                    c2 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c2, 0, 0, 0);
                    c3 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c3, 0, 0, 0);
                }
            }
            r = c0[0] + c1[1] + c2[2] + c3[3];
        }
    }
    long long t1 = clock64();
    if (lane == 0) out[wave] = t1 - t0;
    sink[threadIdx.x] = r;
}
int main() {
    long long *out; unsigned *simd; float *sink;
    hipMallocManaged(&out, 64); hipMallocManaged(&simd, 32); hipMallocManaged(&sink, 2048);
    struct { const char *name; int mfma, valu, big; } cases[] = {
        {"valu wave0 alone", 0, 1, 0}, {"mfma16 wave4 alone", 1 << 4, 0, 0}, {"mfma32 wave4 alone", 1 << 4, 0, 1},
        {"valu w0 + mfma16 w4", 1 << 4, 1, 0}, {"valu w0 + mfma32 w4", 1 << 4, 1, 1},
        {"valu w0 + mfma16 w1,2,3", 0xE, 1, 0}, {"valu w0 + valu w4", 0, 0x11, 0}, {"mfma16 w0 + mfma16 w4", 0x11, 0, 0},
        {"valu w0 + mfma16 w1..7", 0xFE, 1, 0}};
    for (auto &c : cases) {
        for (int rep = 0; rep < 2; ++rep) {
            hipLaunchKernelGGL(k, dim3(1), dim3(512), 0, 0, c.mfma, c.valu, 2000, out, simd, sink, c.big);
            hipDeviceSynchronize();
        }
        printf("%-26s simd:", c.name);
        for (int w = 0; w < 8; ++w) printf(" %u", simd[w]);
        printf("  ticks:");
        for (int w = 0; w < 8; ++w) printf(" %lld", out[w]);
        printf("\n");
    }
    return 0;
}
