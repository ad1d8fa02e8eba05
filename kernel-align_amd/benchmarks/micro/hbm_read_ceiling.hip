// Ceiling of a pure HBM read stream on this GPU: 32 GiB read once with 16-byte loads (non-temporal and
// cached), nothing computed.  The logprob kernel is priced against the published 8 TB/s; this shows what a
// read-only kernel can reach at all (7.19 TB/s measured on MI355X).
#include <hip/hip_runtime.h>
#include <stdio.h>
typedef unsigned u4 __attribute__((ext_vector_type(4)));
template <int U, bool NT>
__global__ __launch_bounds__(256) void rd(const u4* __restrict__ p, size_t n_per_block, unsigned* out) {
    const u4* base = p + blockIdx.x * n_per_block;
    u4 acc = {0, 0, 0, 0};
    for (size_t i = threadIdx.x; i + (U - 1) * 256 < n_per_block; i += U * 256) {
        u4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = NT ? __builtin_nontemporal_load(base + i + u * 256) : base[i + u * 256];
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= v[u];
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) out[0] = 1;
}
int main() {
    const size_t bytes = size_t(32) << 30;  // 32 GiB
    u4* d; hipMalloc(&d, bytes); hipMemset(d, 1, bytes);
    unsigned* o; hipMalloc(&o, 4);
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    for (size_t per_block_kb : {256, 1024, 4096}) {
        size_t n_per_block = per_block_kb * 1024 / 16;
        unsigned blocks = unsigned(bytes / 16 / n_per_block);
        for (int variant = 0; variant < 3; ++variant) {
            float best = 1e9;
            for (int rep = 0; rep < 4; ++rep) {
                hipEventRecord(e0);
                if (variant == 0) hipLaunchKernelGGL((rd<4, true>), dim3(blocks), dim3(256), 0, 0, d, n_per_block, o);
                if (variant == 1) hipLaunchKernelGGL((rd<8, true>), dim3(blocks), dim3(256), 0, 0, d, n_per_block, o);
                if (variant == 2) hipLaunchKernelGGL((rd<4, false>), dim3(blocks), dim3(256), 0, 0, d, n_per_block, o);
                hipEventRecord(e1); hipEventSynchronize(e1);
                float ms; hipEventElapsedTime(&ms, e0, e1); if (ms < best) best = ms;
            }
            printf("per-block %zu KB, variant %d (U=%d,%s): %.3f ms -> %.0f GB/s\n", per_block_kb, variant, variant == 1 ? 8 : 4, variant == 2 ? "cached" : "nt", best, bytes / best / 1e6);
        }
    }
    return 0;
}
