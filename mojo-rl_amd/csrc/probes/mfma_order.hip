// Probe: do v_mfma_f32_32x32x2_f32 and v_mfma_f32_16x16x4_f32 accumulate over k in the same order?
// Compares both tile shapes, a permuted k order, a serial multiply-add loop and a serial fmaf loop,
// bit for bit.  Not part of the library: it backs the 16-row tiles of mlp_tile16.hpp.
//   hipcc --offload-arch=gfx950 -O2 -ffp-contract=off mfma_order.hip -o mfma_order && ./mfma_order
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <math.h>
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
constexpr int K = 256;
// A [32][K] row-major, B [K][32] row-major
__global__ void k32(const float *A, const float *B, float *D) {
    const int lane = threadIdx.x, half = lane >> 5, l31 = lane & 31;
    floatx16 c = {0};
    for (int kk = 0; kk < K / 2; ++kk) {
        const int k = 2 * kk + half;
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(A[l31 * K + k], B[k * 32 + l31], c, 0, 0, 0);
    }
    for (int v = 0; v < 16; ++v) {
        const int row = 8 * (v >> 2) + 4 * half + (v & 3);
        D[row * 32 + l31] = c[v];
    }
}
// rows 0..15, cols 0..31 as two 16x16 tiles
__global__ void k16(const float *A, const float *B, float *D, int perm) {
    const int lane = threadIdx.x, g = lane >> 4, n = lane & 15;
    floatx4 c0 = {0}, c1 = {0};
    for (int kk = 0; kk < K / 4; ++kk) {
        int k = 4 * kk + g;
        if (perm) { const int j = kk / 4, cc = kk % 4; k = 16 * j + 4 * g + cc; }
        const float a = A[n * K + k];
        c0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, B[k * 32 + n], c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, B[k * 32 + 16 + n], c1, 0, 0, 0);
    }
    for (int v = 0; v < 4; ++v) {
        const int row = 4 * g + v;
        D[row * 32 + n] = c0[v];
        D[row * 32 + 16 + n] = c1[v];
    }
}
int main() {
    float *A, *B, *D1, *D2, *D3;
    hipMallocManaged(&A, 32 * K * 4); hipMallocManaged(&B, K * 32 * 4);
    hipMallocManaged(&D1, 32 * 32 * 4); hipMallocManaged(&D2, 32 * 32 * 4); hipMallocManaged(&D3, 32 * 32 * 4);
    srand(1);
    for (int i = 0; i < 32 * K; ++i) { A[i] = (float)rand() / RAND_MAX - 0.5f; B[i] = (float)rand() / RAND_MAX - 0.5f; }
    hipLaunchKernelGGL(k32, dim3(1), dim3(64), 0, 0, A, B, D1);
    hipLaunchKernelGGL(k16, dim3(1), dim3(64), 0, 0, A, B, D2, 0);
    hipLaunchKernelGGL(k16, dim3(1), dim3(64), 0, 0, A, B, D3, 1);
    hipDeviceSynchronize();
    int diff_nat = 0, diff_perm = 0, diff_serial = 0, diff_fma = 0;
    for (int r = 0; r < 16; ++r) for (int c = 0; c < 32; ++c) {
        float s = 0.0f, f = 0.0f;
        for (int k = 0; k < K; ++k) { s = s + A[r * K + k] * B[k * 32 + c]; f = fmaf(A[r * K + k], B[k * 32 + c], f); }
        diff_nat += D1[r * 32 + c] != D2[r * 32 + c];
        diff_perm += D1[r * 32 + c] != D3[r * 32 + c];
        diff_serial += D1[r * 32 + c] != s;
        diff_fma += D1[r * 32 + c] != f;
    }
    printf("of 512: 32x32x2 vs 16x16x4 natural k: %d differ; vs permuted k: %d; 32x32x2 vs serial mul-add: %d; vs serial fma: %d\n",
           diff_nat, diff_perm, diff_serial, diff_fma);
    return 0;
}
