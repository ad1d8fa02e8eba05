// Shared host/device helpers of libkernel_align_hip (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernel_align_hip.h"

#define KA_EXPORT extern "C" __attribute__((visibility("default")))

namespace ka {

// Records a thread-local error message and returns `status`.
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// Maps a HIP error to KA_ERR_HIP (recording its string) or KA_OK.
int check_hip(hipError_t err, const char *what);

constexpr int kWave = 64;

// ---------------------------------------------------------------------------
// Element traits: a 16-byte vector of logits and its widening to fp32.
// ---------------------------------------------------------------------------
struct Bf16 {
    static constexpr int kBytes = 2;
    static constexpr int kPerVec = 8;
    static constexpr int kDtype = KA_DTYPE_BF16;
    using raw_t = uint16_t;
    static __device__ __forceinline__ float widen(raw_t b) { return __uint_as_float(uint32_t(b) << 16); }
    static __device__ __forceinline__ void unpack(const uint4 &v, float (&x)[8]) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            x[2 * j] = __uint_as_float(w[j] << 16);
            x[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        }
    }
};

struct F16 {
    static constexpr int kBytes = 2;
    static constexpr int kPerVec = 8;
    static constexpr int kDtype = KA_DTYPE_F16;
    using raw_t = uint16_t;
    static __device__ __forceinline__ float widen(raw_t b) {
        union { uint16_t u; _Float16 h; } c;
        c.u = b;
        return float(c.h);
    }
    static __device__ __forceinline__ void unpack(const uint4 &v, float (&x)[8]) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            x[2 * j] = widen(uint16_t(w[j] & 0xffffu));
            x[2 * j + 1] = widen(uint16_t(w[j] >> 16));
        }
    }
};

struct F32 {
    static constexpr int kBytes = 4;
    static constexpr int kPerVec = 4;
    static constexpr int kDtype = KA_DTYPE_F32;
    using raw_t = uint32_t;
    static __device__ __forceinline__ float widen(raw_t b) { return __uint_as_float(b); }
    static __device__ __forceinline__ void unpack(const uint4 &v, float (&x)[4]) {
        x[0] = __uint_as_float(v.x);
        x[1] = __uint_as_float(v.y);
        x[2] = __uint_as_float(v.z);
        x[3] = __uint_as_float(v.w);
    }
};

// Streaming 16-byte load: the logits are read once, so they bypass cache
// retention.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
static __device__ __forceinline__ uint4 load_stream(const uint4 *p) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

// Raw v_exp_f32 / v_log_f32 (base 2, no denormal fix-up).
static __device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Butterfly reductions over a 64-lane wavefront; the exchange pattern is fixed,
// so every lane ends with the same bits on every run.
static __device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}
static __device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

}  // namespace ka
