// Peak of the bf16 MFMA instructions on this GPU: a loop of independent v_mfma_f32_32x32x16_bf16 /
// v_mfma_f32_16x16x32_bf16 with no memory traffic (2489 TFLOP/s measured on MI355X with one wavefront per SIMD).
#include <hip/hip_runtime.h>
#include <stdio.h>
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int NACC>
__global__ __launch_bounds__(256) void k32(float* out, int iters) {
    f32x16 acc[NACC];
    for (int i = 0; i < NACC; ++i) for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    bf16x8 a, b;
    for (int j = 0; j < 8; ++j) { a[j] = (__bf16)(float)(threadIdx.x & 3); b[j] = (__bf16)1.0f; }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < NACC; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i], 0, 0, 0);
    }
    float s = 0; for (int i = 0; i < NACC; ++i) for (int r = 0; r < 16; ++r) s += acc[i][r];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}
template <int NACC>
__global__ __launch_bounds__(256) void k16(float* out, int iters) {
    f32x4 acc[NACC];
    for (int i = 0; i < NACC; ++i) for (int r = 0; r < 4; ++r) acc[i][r] = 0.f;
    bf16x8 a, b;
    for (int j = 0; j < 8; ++j) { a[j] = (__bf16)(float)(threadIdx.x & 3); b[j] = (__bf16)1.0f; }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < NACC; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[i], 0, 0, 0);
    }
    float s = 0; for (int i = 0; i < NACC; ++i) for (int r = 0; r < 4; ++r) s += acc[i][r];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}
int main() {
    float* d; hipMalloc(&d, 4096 * 256 * 4);
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    const int iters = 20000;
    for (int wgs : {256, 512, 1024}) {
        for (int variant = 0; variant < 3; ++variant) {
            for (int rep = 0; rep < 2; ++rep) {
                hipEventRecord(e0);
                if (variant == 0) hipLaunchKernelGGL(k32<16>, dim3(wgs), dim3(256), 0, 0, d, iters);
                if (variant == 1) hipLaunchKernelGGL(k32<4>, dim3(wgs), dim3(256), 0, 0, d, iters);
                if (variant == 2) hipLaunchKernelGGL(k16<16>, dim3(wgs), dim3(256), 0, 0, d, iters);
                hipEventRecord(e1); hipEventSynchronize(e1);
                float ms; hipEventElapsedTime(&ms, e0, e1);
                int nacc = variant == 1 ? 4 : 16;
                double flop = (variant == 2 ? 2.0 * 16 * 16 * 32 : 2.0 * 32 * 32 * 16) * nacc * (double)iters * 4 * wgs;
                if (rep) printf("wgs=%d variant=%d ms=%.3f TFLOP/s=%.1f\n", wgs, variant, ms, flop / ms / 1e9);
            }
        }
    }
    return 0;
}
