// Throughput of ds_read_b128 for the lane -> address patterns an MFMA fragment read can use (row = lane % 32,
// 16-byte chunk = lane / 32 XOR a swizzle of the row).  Used to choose the LDS swizzle of the lm_head kernel:
// with 128-byte rows, chunk ^ ((row >> 1) & 7) reads as fast as a contiguous pattern, chunk ^ (row & 7) is 1.5x
// slower and no swizzle 4.5x slower (16 wavefronts per CU, MI355X).
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <vector>
// Each lane reads 16 B at a fixed LDS byte offset given by a table; time per ds_read_b128.
__global__ __launch_bounds__(1024) void k(const int* offs, int npat, long long* cycles, unsigned* sink, int iters) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    for (int i = threadIdx.x; i < 65536 / 4; i += blockDim.x) ((unsigned*)lds)[i] = i;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    for (int p = 0; p < npat; ++p) {
        const int off = offs[p * 64 + lane];
        uint4 acc = make_uint4(0, 0, 0, 0);
        __syncthreads();
        long long t0 = __builtin_readcyclecounter();
        for (int it = 0; it < iters; ++it) {
            typedef unsigned u4 __attribute__((ext_vector_type(4)));
            u4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = *(const u4*)(lds + ((off + u * 8192) & 65535));
#pragma unroll
            for (int u = 0; u < 8; ++u) { asm volatile("" : "+v"(v[u])); acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w; }
        }
        long long t1 = __builtin_readcyclecounter();
        __syncthreads();
        if (threadIdx.x == 0 && blockIdx.x == 0) cycles[p] = t1 - t0;
        sink[threadIdx.x] = acc.x ^ acc.y ^ acc.z ^ acc.w;
    }
}
int main() {
    std::vector<int> offs; std::vector<const char*> names;
    auto add = [&](const char* name, auto f) { names.push_back(name); for (int l = 0; l < 64; ++l) offs.push_back(f(l)); };
    add("contiguous l*16", [](int l) { return l * 16; });
    add("pitch64 no swizzle", [](int l) { int r = l % 32, c = l / 32; return r * 64 + c * 16; });
    add("pitch64 f=(r>>1)&3", [](int l) { int r = l % 32, c = l / 32; return r * 64 + ((c ^ ((r >> 1) & 3)) * 16); });
    add("pitch64 f=(r&2)|((r>>2)&1)", [](int l) { int r = l % 32, c = l / 32; return r * 64 + ((c ^ ((r & 2) | ((r >> 2) & 1))) * 16); });
    add("pitch64 f=r&3", [](int l) { int r = l % 32, c = l / 32; return r * 64 + ((c ^ (r & 3)) * 16); });
    add("pitch128 no swizzle", [](int l) { int r = l % 32, c = l / 32; return r * 128 + c * 16; });
    add("pitch128 f=r&7", [](int l) { int r = l % 32, c = l / 32; return r * 128 + ((c ^ (r & 7)) * 16); });
    add("pitch128 f=((r&3)<<1)|((r>>2)&1)", [](int l) { int r = l % 32, c = l / 32; return r * 128 + ((c ^ (((r & 3) << 1) | ((r >> 2) & 1))) * 16); });
    add("pitch128 f=(r>>1)&7", [](int l) { int r = l % 32, c = l / 32; return r * 128 + ((c ^ ((r >> 1) & 7)) * 16); });
    add("pitch80 (64+16 pad)", [](int l) { int r = l % 32, c = l / 32; return r * 80 + c * 16; });
    add("pitch144 (128+16 pad)", [](int l) { int r = l % 32, c = l / 32; return r * 144 + c * 16; });
    add("pitch32: row=l%32 two chunks (r*32 + c*16)", [](int l) { int r = l % 32, c = l / 32; return r * 32 + c * 16; });
    add("halves split: c*512 + r*16", [](int l) { int r = l % 32, c = l / 32; return c * 512 + r * 16; });
    add("all same address", [](int l) { return 0; });
    add("stride 128 (worst)", [](int l) { return l * 128; });
    add("stride 32", [](int l) { return l * 32; });
    add("stride 64", [](int l) { return l * 64; });
    int npat = names.size();
    int* d_offs; long long* d_cyc; unsigned* d_sink;
    hipMalloc(&d_offs, offs.size() * 4); hipMalloc(&d_cyc, npat * 8); hipMalloc(&d_sink, 1024 * 4);
    hipMemcpy(d_offs, offs.data(), offs.size() * 4, hipMemcpyHostToDevice);
    hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    const int iters = 2000;
    for (int threads : {256, 1024}) {
        hipLaunchKernelGGL(k, dim3(1), dim3(threads), 65536, 0, d_offs, npat, d_cyc, d_sink, iters);
        hipDeviceSynchronize();
        std::vector<long long> cyc(npat); hipMemcpy(cyc.data(), d_cyc, npat * 8, hipMemcpyDeviceToHost);
        printf("threads per block = %d (waves %d)\n", threads, threads / 64);
        for (int p = 0; p < npat; ++p) printf("  %-45s %.1f cycles per ds_read_b128 (per wave)\n", names[p], double(cyc[p]) / (iters * 8.0));
    }
    return 0;
}
