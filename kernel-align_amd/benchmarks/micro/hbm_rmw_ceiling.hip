// Ceiling of a read + write HBM stream on this GPU: 16 GiB read and written back (in place, and into a second
// buffer) with 16-byte accesses, one integer add per element in between.  The logprob backward kernel reads every
// logit once and writes its gradient once, so this, not the read-only stream, is what it can reach.
#include <hip/hip_runtime.h>
#include <stdio.h>
typedef unsigned u4 __attribute__((ext_vector_type(4)));
template <int U, bool NT>
__global__ __launch_bounds__(256) void rmw(const u4 *src, u4 *dst, size_t n_per_block) {
    const u4 *s = src + blockIdx.x * n_per_block;
    u4 *d = dst + blockIdx.x * n_per_block;
    for (size_t i = threadIdx.x; i + (U - 1) * 256 < n_per_block; i += U * 256) {
        u4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = NT ? __builtin_nontemporal_load(s + i + u * 256) : s[i + u * 256];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            v[u] += 1u;
            if (NT) __builtin_nontemporal_store(v[u], d + i + u * 256);
            else d[i + u * 256] = v[u];
        }
    }
}
int main() {
    const size_t bytes = size_t(16) << 30;
    u4 *a, *b;
    hipMalloc(&a, bytes);
    hipMalloc(&b, bytes);
    hipMemset(a, 1, bytes);
    hipMemset(b, 1, bytes);
    hipEvent_t e0, e1;
    hipEventCreate(&e0);
    hipEventCreate(&e1);
    for (size_t per_block_kb : {256, 1024}) {
        const size_t n_per_block = per_block_kb * 1024 / 16;
        const unsigned blocks = unsigned(bytes / 16 / n_per_block);
        for (int variant = 0; variant < 6; ++variant) {
            const bool in_place = variant < 3;
            const int kind = variant % 3;
            float best = 1e9;
            for (int rep = 0; rep < 4; ++rep) {
                u4 *dst = in_place ? a : b;
                hipEventRecord(e0);
                if (kind == 0) hipLaunchKernelGGL((rmw<4, true>), dim3(blocks), dim3(256), 0, 0, a, dst, n_per_block);
                if (kind == 1) hipLaunchKernelGGL((rmw<8, true>), dim3(blocks), dim3(256), 0, 0, a, dst, n_per_block);
                if (kind == 2) hipLaunchKernelGGL((rmw<4, false>), dim3(blocks), dim3(256), 0, 0, a, dst, n_per_block);
                hipEventRecord(e1);
                hipEventSynchronize(e1);
                float ms;
                hipEventElapsedTime(&ms, e0, e1);
                if (ms < best) best = ms;
            }
            printf("per-block %4zu KB, %s, U=%d %s: %.3f ms -> %.0f GB/s read + written\n", per_block_kb,
                   in_place ? "in place    " : "second buffer", kind == 1 ? 8 : 4, kind == 2 ? "cached" : "nt    ", best,
                   2.0 * bytes / best / 1e6);
        }
    }
    return 0;
}
