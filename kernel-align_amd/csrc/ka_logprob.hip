// Per-token logprob: out[r] = logits[r, ids[r]] - logsumexp(logits[r, :]).
//
// One workgroup owns one row.  Every lane streams 16-byte vectors of the row
// (lane t takes vectors t, t + THREADS, ...) and keeps an online
// (max, sum of 2^(x*log2e - max*log2e)) pair in fp32; the row is read exactly
// once and nothing of the size of the logits is written.  The max is refreshed
// once per group of UNROLL vectors, so the rescale costs one extra exp2 per
// 8*UNROLL elements.  Lanes are combined by a fixed butterfly inside each
// wavefront and then in wavefront order through LDS: a row's bits depend on
// that row alone, never on the batch size, the chunking or the grid.
#include "ka_common.h"

namespace ka {
namespace {

constexpr float kLog2e = 1.44269504088896340736f;
constexpr double kLn2 = 0.693147180559945309417232;
// Running maxima start here instead of -inf so that (old max - new max) is
// never inf - inf; logits below this are treated as -inf.
constexpr float kFloor = -1.0e30f;

struct RowState {
    float m;    // running max of the lane's logits (>= kFloor)
    float ml2;  // m * log2(e)
    float s;    // sum of 2^(x*log2e - ml2)
    float a;    // sum of x * 2^(x*log2e - ml2)   (entropy variant only)
};

template <int N, bool ENTROPY>
__device__ __forceinline__ void fold(RowState &st, const float (&x)[N]) {
    // No implicit contraction here: fused into an FMA against the fresh product, (st.ml2 - mn * log2e) would return the
    // rounding residue of a 1e30-sized product instead of 0 while the maximum still sits at the floor (a row that starts
    // with -inf entries), and 2^residue overflows.  The FMAs below are written out.
#pragma clang fp contract(off)
    float mn = st.m;
#pragma unroll
    for (int j = 0; j < N; ++j) mn = fmaxf(mn, x[j]);
    const float ml2n = mn * kLog2e;
    const float rescale = fast_exp2(st.ml2 - ml2n);
    float e[N];
#pragma unroll
    for (int j = 0; j < N; ++j) e[j] = fast_exp2(fmaf(x[j], kLog2e, -ml2n));
    if (ENTROPY) {
        // sum of x * e in four chains of FMAs (element j goes to chain j % 4); x is clamped to a finite value first, so
        // that a masked entry (-inf, e = 0) adds 0 and not 0 * inf
        constexpr int CHAINS = N < 4 ? N : 4;
        float w[CHAINS];
#pragma unroll
        for (int c = 0; c < CHAINS; ++c) w[c] = 0.0f;
#pragma unroll
        for (int j = 0; j < N; ++j) w[j % CHAINS] = fmaf(fmaxf(x[j], -3.0e38f), e[j], w[j % CHAINS]);
        float sum = w[0];
        if (CHAINS == 4) sum = (w[0] + w[1]) + (w[2] + w[3]);
        else if (CHAINS == 2) sum = w[0] + w[1];
        st.a = fmaf(st.a, rescale, sum);
    }
    // Pairwise tree in a fixed order.
#pragma unroll
    for (int step = 1; step < N; step <<= 1)
#pragma unroll
        for (int j = 0; j + step < N; j += 2 * step) e[j] += e[j + step];
    st.s = fmaf(st.s, rescale, e[0]);
    st.m = mn;
    st.ml2 = ml2n;
}

template <typename T, int THREADS, int UNROLL, bool VEC, bool ENTROPY>
__global__ __launch_bounds__(THREADS) void logprob_rows(const typename T::raw_t *__restrict__ logits,
                                                        int64_t n_rows, int vocab, int64_t row_stride,
                                                        const int64_t *__restrict__ ids,
                                                        float *__restrict__ out,
                                                        float *__restrict__ entropy) {
    constexpr int EPV = T::kPerVec;
    constexpr int NWAVES = THREADS / kWave;
    __shared__ float red_a[NWAVES];
    __shared__ float red_b[NWAVES];
    __shared__ float red_c[NWAVES];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;

    for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
        const typename T::raw_t *rp = logits + row * row_stride;

        // Lane 0 fetches the target logit up front; its latency hides behind the stream.
        float xt = __builtin_nanf("");
        if (tid == 0) {
            const int64_t id = ids[row];
            if (id >= 0 && id < vocab) xt = T::widen(rp[id]);
        }

        RowState st{kFloor, kFloor * kLog2e, 0.0f, 0.0f};

        if (VEC) {
            const uint4 *vp = reinterpret_cast<const uint4 *>(rp);
            const int nvec = vocab / EPV;
            int i = tid;
            for (; i + (UNROLL - 1) * THREADS < nvec; i += UNROLL * THREADS) {
                uint4 v[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) v[u] = load_stream(vp + i + u * THREADS);
                float x[UNROLL * EPV];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    float xv[EPV];
                    T::unpack(v[u], xv);
#pragma unroll
                    for (int j = 0; j < EPV; ++j) x[u * EPV + j] = xv[j];
                }
                fold<UNROLL * EPV, ENTROPY>(st, x);
            }
            for (; i < nvec; i += THREADS) {
                float xv[EPV];
                T::unpack(load_stream(vp + i), xv);
                fold<EPV, ENTROPY>(st, xv);
            }
            const int tail = vocab - nvec * EPV;
            if (tid < tail) {
                const float xs[1] = {T::widen(rp[nvec * EPV + tid])};
                fold<1, ENTROPY>(st, xs);
            }
        } else {
            for (int i = tid; i < vocab; i += THREADS) {
                const float xs[1] = {T::widen(rp[i])};
                fold<1, ENTROPY>(st, xs);
            }
        }

        // Row max (exact, order-free), then every lane's sum rebased to it.
        const float wm = wave_max(st.ml2);
        if (lane == 0) red_a[wave] = wm;
        __syncthreads();
        float big = red_a[0];
#pragma unroll
        for (int w = 1; w < NWAVES; ++w) big = fmaxf(big, red_a[w]);
        const float rebase = fast_exp2(st.ml2 - big);
        const float ws = wave_sum(st.s * rebase);
        float wa = 0.0f;
        if (ENTROPY) wa = wave_sum(st.a * rebase);
        if (lane == 0) {
            red_b[wave] = ws;
            if (ENTROPY) red_c[wave] = wa;
        }
        __syncthreads();
        if (tid == 0) {
            float total = red_b[0];
#pragma unroll
            for (int w = 1; w < NWAVES; ++w) total += red_b[w];
            const double lse = (double(big) + log2(double(total))) * kLn2;
            out[row] = float(double(xt) - lse);
            if (ENTROPY && entropy != nullptr) {
                float ta = red_c[0];
#pragma unroll
                for (int w = 1; w < NWAVES; ++w) ta += red_c[w];
                entropy[row] = float(lse - double(ta) / double(total));
            }
        }
        // red_a / red_b are rewritten only after the next row's first barrier pair.
        __syncthreads();
    }
}

template <typename T, bool ENTROPY>
int launch(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride, const int64_t *ids,
           float *out, float *entropy, void *hip_stream) {
    if (n_rows < 0) return fail(KA_ERR_BAD_ARG, "logprob: n_rows %lld < 0", (long long)n_rows);
    if (n_rows == 0) return KA_OK;
    if (logits == nullptr || ids == nullptr || out == nullptr)
        return fail(KA_ERR_BAD_ARG, "logprob: null logits / ids / out pointer");
    if (vocab < 1) return fail(KA_ERR_BAD_ARG, "logprob: vocab %lld < 1", (long long)vocab);
    if (vocab >= (int64_t(1) << 31))
        return fail(KA_ERR_UNSUPPORTED, "logprob: vocab %lld does not fit 31 bits", (long long)vocab);
    if (row_stride < vocab)
        return fail(KA_ERR_BAD_ARG, "logprob: row_stride %lld < vocab %lld", (long long)row_stride,
                    (long long)vocab);

    constexpr int THREADS = 256;
    constexpr int UNROLL = 4;
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    const auto *lp = static_cast<const typename T::raw_t *>(logits);
    const bool aligned = (reinterpret_cast<uintptr_t>(logits) % 16 == 0) &&
                         ((row_stride * T::kBytes) % 16 == 0);
    const unsigned grid = unsigned(n_rows < (int64_t(1) << 30) ? n_rows : (int64_t(1) << 30));
    if (aligned) {
        hipLaunchKernelGGL((logprob_rows<T, THREADS, UNROLL, true, ENTROPY>), dim3(grid), dim3(THREADS), 0,
                           stream, lp, n_rows, int(vocab), row_stride, ids, out, entropy);
    } else {
        hipLaunchKernelGGL((logprob_rows<T, THREADS, 1, false, ENTROPY>), dim3(grid), dim3(THREADS), 0,
                           stream, lp, n_rows, int(vocab), row_stride, ids, out, entropy);
    }
    return check_hip(hipGetLastError(), "logprob launch");
}

}  // namespace
}  // namespace ka

KA_EXPORT int ka_logprob_bf16(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                              const int64_t *ids, float *out, void *hip_stream) {
    return ka::launch<ka::Bf16, false>(logits, n_rows, vocab, row_stride, ids, out, nullptr, hip_stream);
}

KA_EXPORT int ka_logprob_f16(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                             const int64_t *ids, float *out, void *hip_stream) {
    return ka::launch<ka::F16, false>(logits, n_rows, vocab, row_stride, ids, out, nullptr, hip_stream);
}

KA_EXPORT int ka_logprob_f32(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                             const int64_t *ids, float *out, void *hip_stream) {
    return ka::launch<ka::F32, false>(logits, n_rows, vocab, row_stride, ids, out, nullptr, hip_stream);
}

KA_EXPORT int ka_logprob_entropy_bf16(const void *logits, int64_t n_rows, int64_t vocab,
                                      int64_t row_stride, const int64_t *ids, float *out,
                                      float *entropy, void *hip_stream) {
    return ka::launch<ka::Bf16, true>(logits, n_rows, vocab, row_stride, ids, out, entropy, hip_stream);
}

KA_EXPORT int ka_logprob_entropy_f16(const void *logits, int64_t n_rows, int64_t vocab,
                                     int64_t row_stride, const int64_t *ids, float *out,
                                     float *entropy, void *hip_stream) {
    return ka::launch<ka::F16, true>(logits, n_rows, vocab, row_stride, ids, out, entropy, hip_stream);
}

KA_EXPORT int ka_logprob_entropy_f32(const void *logits, int64_t n_rows, int64_t vocab,
                                     int64_t row_stride, const int64_t *ids, float *out,
                                     float *entropy, void *hip_stream) {
    return ka::launch<ka::F32, true>(logits, n_rows, vocab, row_stride, ids, out, entropy, hip_stream);
}

// ---------------------------------------------------------------------------
// Backward of the per-token logprob:
//     dlogits[r, v] = grad[r] * ((v == ids[r]) - softmax(logits[r, :])[v])
// One pass: the row's log-sum-exp is recovered from the forward result
// (lse = logits[r, ids[r]] - logp[r]), every logit is read once and its
// gradient written once, in the logits' dtype.  dlogits may alias logits (each
// element is read and then written by the same lane), so the gradient of a
// [G, L, V] tensor needs no second tensor of that size.
// A target whose logit is -inf (a masked entry) has logp = -inf, from which the
// log-sum-exp cannot be recovered: such a row takes one more pass that
// recomputes it, and gets the finite gradient -g * softmax autograd gives.
// ---------------------------------------------------------------------------
namespace ka {
namespace {

template <typename T> struct Narrow;
template <> struct Narrow<Bf16> {
    static __device__ __forceinline__ uint16_t one(float v) {
        union { __bf16 b; uint16_t u; } c;
        c.b = (__bf16)v;  // round to nearest even
        return c.u;
    }
};
template <> struct Narrow<F16> {
    static __device__ __forceinline__ uint16_t one(float v) {
        union { _Float16 h; uint16_t u; } c;
        c.h = (_Float16)v;
        return c.u;
    }
};
template <> struct Narrow<F32> {
    static __device__ __forceinline__ uint32_t one(float v) { return __float_as_uint(v); }
};

template <typename T> __device__ __forceinline__ uint4 pack_vec(const float (&g)[8]);
template <typename T> __device__ __forceinline__ uint4 pack_vec(const float (&g)[4]);
template <> __device__ __forceinline__ uint4 pack_vec<Bf16>(const float (&g)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = uint32_t(Narrow<Bf16>::one(g[2 * j])) | (uint32_t(Narrow<Bf16>::one(g[2 * j + 1])) << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
}
template <> __device__ __forceinline__ uint4 pack_vec<F16>(const float (&g)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = uint32_t(Narrow<F16>::one(g[2 * j])) | (uint32_t(Narrow<F16>::one(g[2 * j + 1])) << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
}
template <> __device__ __forceinline__ uint4 pack_vec<F32>(const float (&g)[4]) {
    return make_uint4(__float_as_uint(g[0]), __float_as_uint(g[1]), __float_as_uint(g[2]), __float_as_uint(g[3]));
}

static __device__ __forceinline__ void store_stream(uint4 *p, const uint4 &v) {
    u32x4 q = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(q, reinterpret_cast<u32x4 *>(p));
}

template <typename T, int THREADS, int UNROLL, bool VEC>
__global__ __launch_bounds__(THREADS) void logprob_backward_rows(const typename T::raw_t *logits,
                                                                 int64_t n_rows, int vocab, int64_t row_stride,
                                                                 const int64_t *__restrict__ ids,
                                                                 const float *__restrict__ logp,
                                                                 const float *__restrict__ grad,
                                                                 typename T::raw_t *dlogits, int64_t d_stride) {
    constexpr int EPV = T::kPerVec;
    constexpr int NWAVES = THREADS / kWave;
    __shared__ float s_lse;
    __shared__ int s_masked;
    __shared__ float red_a[NWAVES];
    __shared__ float red_b[NWAVES];
    const int tid = threadIdx.x;
    for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
        const typename T::raw_t *rp = logits + row * row_stride;
        typename T::raw_t *dp = dlogits + row * d_stride;
        const int64_t id = ids[row];
        const bool id_ok = id >= 0 && id < vocab;
        const float g = grad[row];
        // lse = x_t - logp; an id outside the vocabulary has no defined forward value: its row gets NaN.
        // One lane reads x_t and the barrier comes before any store, because dlogits may be the logits.
        if (tid == 0) {
            const float x_t = id_ok ? T::widen(rp[id]) : __builtin_nanf("");
            s_lse = x_t - logp[row];
            s_masked = id_ok && x_t == -__builtin_inff();
        }
        __syncthreads();
        if (s_masked) {  // workgroup-uniform and rare: recompute the row's log-sum-exp (before any store)
            RowState st{kFloor, kFloor * kLog2e, 0.0f, 0.0f};
            for (int i = tid; i < vocab; i += THREADS) {
                const float xs[1] = {T::widen(rp[i])};
                fold<1, false>(st, xs);
            }
            const float wm = wave_max(st.ml2);
            if ((tid & (kWave - 1)) == 0) red_a[tid / kWave] = wm;
            __syncthreads();
            float big = red_a[0];
#pragma unroll
            for (int w = 1; w < NWAVES; ++w) big = fmaxf(big, red_a[w]);
            const float ws = wave_sum(st.s * fast_exp2(st.ml2 - big));
            if ((tid & (kWave - 1)) == 0) red_b[tid / kWave] = ws;
            __syncthreads();
            if (tid == 0) {
                float total = red_b[0];
#pragma unroll
                for (int w = 1; w < NWAVES; ++w) total += red_b[w];
                // a row of nothing but -inf keeps NaN, as softmax of such a row does
                s_lse = total > 0.0f ? float((double(big) + log2(double(total))) * kLn2) : __builtin_nanf("");
            }
            __syncthreads();
        }
        const float lse = s_lse;
        const float nl2 = -lse * kLog2e;
        const float ng = -g;
        // d = g * (onehot - p) = -g * p (+ g at the target)
        auto grad_of = [&](float x, int idx) {
            const float p = fast_exp2(fmaf(x, kLog2e, nl2));
            float d = ng * p;
            if (idx == int(id)) d += g;
            return d;
        };
        if (VEC) {
            const uint4 *vp = reinterpret_cast<const uint4 *>(rp);
            uint4 *op = reinterpret_cast<uint4 *>(dp);
            const int nvec = vocab / EPV;
            int i = tid;
            for (; i + (UNROLL - 1) * THREADS < nvec; i += UNROLL * THREADS) {
                uint4 v[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) v[u] = load_stream(vp + i + u * THREADS);
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    float x[EPV], d[EPV];
                    T::unpack(v[u], x);
#pragma unroll
                    for (int j = 0; j < EPV; ++j) d[j] = grad_of(x[j], (i + u * THREADS) * EPV + j);
                    store_stream(op + i + u * THREADS, pack_vec<T>(d));
                }
            }
            for (; i < nvec; i += THREADS) {
                float x[EPV], d[EPV];
                T::unpack(load_stream(vp + i), x);
#pragma unroll
                for (int j = 0; j < EPV; ++j) d[j] = grad_of(x[j], i * EPV + j);
                store_stream(op + i, pack_vec<T>(d));
            }
            const int t = nvec * EPV + tid;
            if (t < vocab) dp[t] = Narrow<T>::one(grad_of(T::widen(rp[t]), t));
        } else {
            for (int i = tid; i < vocab; i += THREADS) dp[i] = Narrow<T>::one(grad_of(T::widen(rp[i]), i));
        }
        __syncthreads();  // s_lse is rewritten for the next row
    }
}

template <typename T>
int launch_backward(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride, const int64_t *ids,
                    const float *logp, const float *grad, void *dlogits, int64_t d_stride, void *hip_stream) {
    if (n_rows < 0) return fail(KA_ERR_BAD_ARG, "logprob backward: n_rows %lld < 0", (long long)n_rows);
    if (n_rows == 0) return KA_OK;
    if (logits == nullptr || ids == nullptr || logp == nullptr || grad == nullptr || dlogits == nullptr)
        return fail(KA_ERR_BAD_ARG, "logprob backward: null pointer argument");
    if (vocab < 1) return fail(KA_ERR_BAD_ARG, "logprob backward: vocab %lld < 1", (long long)vocab);
    if (vocab >= (int64_t(1) << 31))
        return fail(KA_ERR_UNSUPPORTED, "logprob backward: vocab %lld does not fit 31 bits", (long long)vocab);
    if (row_stride < vocab || d_stride < vocab)
        return fail(KA_ERR_BAD_ARG, "logprob backward: a row stride is smaller than vocab %lld", (long long)vocab);
    if (dlogits == logits && d_stride != row_stride)
        return fail(KA_ERR_BAD_ARG, "logprob backward: in-place use needs equal strides");
    // Long rows take 1024-thread workgroups: a read + write stream runs faster in long bursts (a workgroup reads
    // 64 KB, then writes 64 KB).  Measured on bf16 [32768, 128256]: 256 threads 5.1 TB/s, 512 threads 5.4, 1024
    // threads 5.8 (unrolled by 4; by 2 or 8: 5.6), against 4.9 - 5.0 TB/s for the runtime's own device-to-device copy
    // of the same bytes.  Short rows keep 256 threads (a 1024-thread workgroup would not fill its unrolled tile).
    constexpr int UNROLL = 4;
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    const auto *lp = static_cast<const typename T::raw_t *>(logits);
    auto *dp = static_cast<typename T::raw_t *>(dlogits);
    const bool aligned = reinterpret_cast<uintptr_t>(logits) % 16 == 0 && reinterpret_cast<uintptr_t>(dlogits) % 16 == 0 &&
                         (row_stride * T::kBytes) % 16 == 0 && (d_stride * T::kBytes) % 16 == 0;
    const unsigned grid = unsigned(n_rows < (int64_t(1) << 30) ? n_rows : (int64_t(1) << 30));
    const bool long_rows = vocab >= int64_t(1024) * UNROLL * T::kPerVec * 2;  // two full tiles of the wide workgroup
    if (aligned && long_rows) {
        hipLaunchKernelGGL((logprob_backward_rows<T, 1024, UNROLL, true>), dim3(grid), dim3(1024), 0, stream, lp,
                           n_rows, int(vocab), row_stride, ids, logp, grad, dp, d_stride);
    } else if (aligned) {
        hipLaunchKernelGGL((logprob_backward_rows<T, 256, UNROLL, true>), dim3(grid), dim3(256), 0, stream, lp,
                           n_rows, int(vocab), row_stride, ids, logp, grad, dp, d_stride);
    } else {
        hipLaunchKernelGGL((logprob_backward_rows<T, 256, 1, false>), dim3(grid), dim3(256), 0, stream, lp,
                           n_rows, int(vocab), row_stride, ids, logp, grad, dp, d_stride);
    }
    return check_hip(hipGetLastError(), "logprob backward launch");
}

}  // namespace
}  // namespace ka

KA_EXPORT int ka_logprob_backward_bf16(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                                       const int64_t *ids, const float *logp, const float *grad, void *dlogits,
                                       int64_t dlogits_stride, void *hip_stream) {
    return ka::launch_backward<ka::Bf16>(logits, n_rows, vocab, row_stride, ids, logp, grad, dlogits, dlogits_stride,
                                         hip_stream);
}
KA_EXPORT int ka_logprob_backward_f16(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                                      const int64_t *ids, const float *logp, const float *grad, void *dlogits,
                                      int64_t dlogits_stride, void *hip_stream) {
    return ka::launch_backward<ka::F16>(logits, n_rows, vocab, row_stride, ids, logp, grad, dlogits, dlogits_stride,
                                        hip_stream);
}
KA_EXPORT int ka_logprob_backward_f32(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                                      const int64_t *ids, const float *logp, const float *grad, void *dlogits,
                                      int64_t dlogits_stride, void *hip_stream) {
    return ka::launch_backward<ka::F32>(logits, n_rows, vocab, row_stride, ids, logp, grad, dlogits, dlogits_stride,
                                        hip_stream);
}
