// Fused temperature -> top-k -> top-p -> draw, one workgroup per row.
//
// Every decision is taken on integers, so the sampled id does not depend on
// summation order, batch size or launch geometry:
//   * each scaled logit y maps to an order-preserving 32-bit key;
//   * the k-th largest key K* comes from an MSB-first radix descent over
//     2048-bin LDS count histograms (ties with K* survive, as in the reference);
//   * softmax masses are W(y - max) = trunc(2^40 * exp(y - max)), evaluated by a
//     fixed sequence of IEEE double operations, and summed as 64-bit integers;
//   * the top-p cut is a second radix descent over per-bin integer mass: it finds
//     the lowest key Kc whose first entry still has (mass before it) <= top_p * Z,
//     and how many entries r of the Kc tie group (ascending index) survive;
//   * the draw walks the row once more in index order with block-wide integer
//     prefix sums and stops at the first survivor whose inclusive mass exceeds
//     floor(u * Z_survivors).
// The row is re-read by every pass; after the first it comes from L2 / MALL.
// This radix path takes any row; shorter routes for common cases come first: the top-k candidate list
// (ka_sampling_topk.h: top_k <= 1024), and for 16-bit dtypes the no-filter and dense-histogram paths (ka_sampling_dense.h).
// For aligned fp32 rows outside the candidate list a variant of the kernel replaces the last pass by a draw
// over shares of the row (ka_sampling_draw.h).
#include <mutex>

#include "ka_sampling_kernel.h"

namespace ka {
namespace {

__global__ __launch_bounds__(256) void mass_fixed_kernel(const float *__restrict__ d, int64_t n, uint64_t *__restrict__ out) {
    const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) out[i] = weight_fix(d[i]);
}

// CUs of the current device (asked once per device).
inline int device_cu_count(int *out) {
    static std::mutex mutex;
    static int known[64] = {};
    int device = 0;
    hipError_t rc = hipGetDevice(&device);
    if (rc != hipSuccess) return check_hip(rc, "sample: hipGetDevice");
    if (device < 0 || device >= 64) return fail(KA_ERR_UNSUPPORTED, "sample: device index %d", device);
    std::lock_guard<std::mutex> lock(mutex);
    if (known[device] == 0) {
        int n = 0;
        rc = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device);
        if (rc != hipSuccess) return check_hip(rc, "sample: asking for the number of CUs");
        known[device] = n > 0 ? n : 1;
    }
    *out = known[device];
    return KA_OK;
}

template <typename T>
int launch(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride, const SampleParams &prm,
           void *workspace, size_t workspace_bytes, void *hip_stream, uint32_t flags = 0) {
    if (batch < 0) return fail(KA_ERR_BAD_ARG, "sample: batch %lld < 0", (long long)batch);
    if (batch == 0) return KA_OK;
    if (logits == nullptr || prm.uniforms == nullptr || prm.out_ids == nullptr)
        return fail(KA_ERR_BAD_ARG, "sample: null logits / uniforms / out_ids pointer");
    if (vocab < 1) return fail(KA_ERR_BAD_ARG, "sample: vocab %lld < 1", (long long)vocab);
    if (vocab >= (int64_t(1) << 22))
        return fail(KA_ERR_UNSUPPORTED, "sample: vocab %lld >= 2^22 (integer masses would overflow)",
                    (long long)vocab);
    if (row_stride < vocab) return fail(KA_ERR_BAD_ARG, "sample: row_stride < vocab");
    if (prm.temperature_rows == nullptr && !(prm.temperature > 0.0f))
        return fail(KA_ERR_BAD_ARG, "sample: temperature %g must be > 0", prm.temperature);
    if (prm.top_k_rows == nullptr && prm.top_k < 0) return fail(KA_ERR_BAD_ARG, "sample: top_k %d < 0", prm.top_k);
    if (prm.top_p_rows == nullptr && !(prm.top_p > 0.0f && prm.top_p <= 1.0f))
        return fail(KA_ERR_BAD_ARG, "sample: top_p %g outside (0, 1]", prm.top_p);
    if (batch >= (int64_t(1) << 31)) return fail(KA_ERR_UNSUPPORTED, "sample: batch too large");
    if (workspace_bytes < ka_sample_workspace_bytes(batch, vocab) || (workspace == nullptr && workspace_bytes > 0))
        return fail(KA_ERR_WORKSPACE, "sample: workspace of %zu B, need %zu B", workspace_bytes,
                    ka_sample_workspace_bytes(batch, vocab));
    const bool aligned = (reinterpret_cast<uintptr_t>(logits) % 16 == 0) && ((row_stride * T::kBytes) % 16 == 0);
    if (flags & ~uint32_t(KA_SAMPLE_FLAG_GENERAL_PATH | KA_SAMPLE_FLAG_BLOCK_WIDE_TOPK | KA_SAMPLE_FLAG_TWO_ROWS_PER_CU |
                          KA_SAMPLE_FLAG_ONE_ROW_PER_CU))
        return fail(KA_ERR_BAD_ARG, "sample: unknown flag bits 0x%x", flags);
    if ((flags & KA_SAMPLE_FLAG_TWO_ROWS_PER_CU) && (flags & KA_SAMPLE_FLAG_ONE_ROW_PER_CU))
        return fail(KA_ERR_BAD_ARG, "sample: both workgroup-size flags are set");
    const bool no_fast = (flags & KA_SAMPLE_FLAG_GENERAL_PATH) != 0;
    const int path_bits = int(flags & 3u);
    // The dense-histogram path needs 157 KB of LDS (one workgroup per CU).  It serves top-p without top-k,
    // top_k > 1024 and no filter at all on aligned 16-bit rows; with per-row parameters any row may need it.
    bool dense = false;
    if (T::kBytes == 2 && aligned && !no_fast) {
        const bool per_row = prm.top_k_rows != nullptr || prm.top_p_rows != nullptr;
        const bool k_on = prm.top_k > 0 && prm.top_k < vocab;
        // (no filter at all: the histogram path for bf16; an fp16 row has too many distinct values for its list and
        //  takes the register-resident no-filter path of the small-LDS kernel)
        const bool no_filter = !k_on && !(prm.top_p < 1.0f);
        const bool fits_registers = vocab / 8 <= RES_VECS * S_THREADS;  // what the other kernel's no-filter path takes
        dense = per_row || (k_on && prm.top_k > S_THREADS) || (!k_on && !no_filter) ||
                (no_filter && (T::kDtype == KA_DTYPE_BF16 || !fits_registers));
    }
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    const typename T::raw_t *lp = static_cast<const typename T::raw_t *>(logits);
    if constexpr (T::kBytes == 4) {
        // fp32 rows outside the top-k fast path (no filter, top-p alone, top_k > 1024): the radix path with the draw
        // done by shares of the row
        const bool per_row = prm.top_k_rows != nullptr || prm.top_p_rows != nullptr;
        const bool k_fast = prm.top_k > 0 && prm.top_k < vocab && prm.top_k <= S_THREADS;
        if (aligned && !per_row && !k_fast) {
            hipLaunchKernelGGL((sample_rows<T, true>), dim3(unsigned(batch)), dim3(S_THREADS), 0, stream, lp, int(vocab),
                               row_stride, prm, 1, path_bits);
            return check_hip(hipGetLastError(), "sample launch");
        }
    }
    if constexpr (T::kBytes == 2) {
      if (dense) {
        // the attribute belongs to the device: set once per device and dtype, not per call
        static std::mutex attr_mutex;
        static bool attr_set[64] = {};
        int device = 0;
        hipError_t rc = hipGetDevice(&device);
        if (rc != hipSuccess) return check_hip(rc, "sample: hipGetDevice");
        if (device < 0 || device >= 64) return fail(KA_ERR_UNSUPPORTED, "sample: device index %d", device);
        {
            std::lock_guard<std::mutex> lock(attr_mutex);
            if (!attr_set[device]) {
                rc = hipFuncSetAttribute(reinterpret_cast<const void *>(sample_rows<T, true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, int(DENSE_LDS_BYTES));
                if (rc != hipSuccess) return check_hip(rc, "sample: reserving LDS for the dense-histogram path");
                attr_set[device] = true;
            }
        }
        hipLaunchKernelGGL((sample_rows<T, true>), dim3(unsigned(batch)), dim3(S_THREADS), DENSE_LDS_BYTES, stream, lp,
                           int(vocab), row_stride, prm, aligned ? 1 : 0, path_bits & 2);
        return check_hip(hipGetLastError(), "sample launch");
      }
    }
    {
        // Short top-k route on a batch of more rows than CUs: 512 threads per row, two rows resident per CU (one
        // row's selection runs under the other row's read).  Up to one row per CU the 1024-thread workgroup reads its
        // row faster.  The flags force either build where the row qualifies.
        const bool k_short = prm.top_k_rows == nullptr && prm.top_k > 0 && prm.top_k < vocab && prm.top_k <= SHORT_TOPK;
        // a slot maximum per vector and lane (16-bit rows), or per group of up to four vectors (fp32 rows)
        const bool fits = aligned && vocab / T::kPerVec <= (T::kBytes == 4 ? 4 : 1) * 32 * 512;
        if (k_short && fits && path_bits == 0 && !(flags & KA_SAMPLE_FLAG_ONE_ROW_PER_CU)) {
            bool two_rows = (flags & KA_SAMPLE_FLAG_TWO_ROWS_PER_CU) != 0;
            if (!two_rows) {
                int n_cus = 0;
                const int rc = device_cu_count(&n_cus);
                if (rc != KA_OK) return rc;
                two_rows = batch > n_cus;
            }
            if (two_rows)
                return check_hip(launch_sample_rows_half(T::kDtype, logits, batch, int(vocab), row_stride, prm, 0, stream),
                                 "sample launch");
        }
    }
    hipLaunchKernelGGL((sample_rows<T, false>), dim3(unsigned(batch)), dim3(S_THREADS), 0, stream, lp, int(vocab),
                       row_stride, prm, aligned ? 1 : 0, path_bits);
    return check_hip(hipGetLastError(), "sample launch");
}

inline SampleParams scalar_params(float temperature, int32_t top_k, float top_p, const float *uniforms,
                                  int64_t *out_ids) {
    SampleParams p{};
    p.temperature = temperature;
    p.top_k = top_k;
    p.top_p = top_p;
    p.uniforms = uniforms;
    p.out_ids = out_ids;
    return p;
}

inline int launch_ex(int dtype, const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                     const SampleParams &prm, void *workspace, size_t workspace_bytes, void *hip_stream, uint32_t flags) {
    switch (dtype) {
        case KA_DTYPE_BF16: return launch<Bf16>(logits, batch, vocab, row_stride, prm, workspace, workspace_bytes, hip_stream, flags);
        case KA_DTYPE_F16: return launch<F16>(logits, batch, vocab, row_stride, prm, workspace, workspace_bytes, hip_stream, flags);
        case KA_DTYPE_F32: return launch<F32>(logits, batch, vocab, row_stride, prm, workspace, workspace_bytes, hip_stream, flags);
        default: return fail(KA_ERR_BAD_ARG, "sample: unknown dtype code %d", dtype);
    }
}

}  // namespace
}  // namespace ka

// The kernels keep all their state in LDS and registers; the workspace argument is reserved.
KA_EXPORT size_t ka_sample_workspace_bytes(int64_t batch, int64_t vocab) {
    (void)batch;
    (void)vocab;
    return 0;
}

KA_EXPORT int ka_sample_topk_topp_bf16(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                                       float temperature, int32_t top_k, float top_p, const float *uniforms,
                                       int64_t *out_ids, void *workspace, size_t workspace_bytes,
                                       void *hip_stream) {
    return ka::launch<ka::Bf16>(logits, batch, vocab, row_stride,
                              ka::scalar_params(temperature, top_k, top_p, uniforms, out_ids), workspace,
                              workspace_bytes, hip_stream);
}
KA_EXPORT int ka_sample_topk_topp_f16(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                                      float temperature, int32_t top_k, float top_p, const float *uniforms,
                                      int64_t *out_ids, void *workspace, size_t workspace_bytes,
                                      void *hip_stream) {
    return ka::launch<ka::F16>(logits, batch, vocab, row_stride,
                              ka::scalar_params(temperature, top_k, top_p, uniforms, out_ids), workspace,
                              workspace_bytes, hip_stream);
}
KA_EXPORT int ka_sample_topk_topp_f32(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                                      float temperature, int32_t top_k, float top_p, const float *uniforms,
                                      int64_t *out_ids, void *workspace, size_t workspace_bytes,
                                      void *hip_stream) {
    return ka::launch<ka::F32>(logits, batch, vocab, row_stride,
                              ka::scalar_params(temperature, top_k, top_p, uniforms, out_ids), workspace,
                              workspace_bytes, hip_stream);
}

#ifdef KA_SAMPLE_STAMPS
KA_EXPORT int ka_debug_read_stamps(unsigned long long *host, int n) {
    return int(hipMemcpyFromSymbol(host, HIP_SYMBOL(ka::ka_dbg_stamps), size_t(n) * 8, 0, hipMemcpyDeviceToHost));
}
#endif

KA_EXPORT int ka_sample_mass_fixed(const float *d, int64_t n, uint64_t *out, void *hip_stream) {
    using namespace ka;
    if (n < 0) return fail(KA_ERR_BAD_ARG, "mass: n %lld < 0", (long long)n);
    if (n == 0) return KA_OK;
    if (d == nullptr || out == nullptr) return fail(KA_ERR_BAD_ARG, "mass: null pointer argument");
    if ((n + 255) / 256 >= (int64_t(1) << 31)) return fail(KA_ERR_UNSUPPORTED, "mass: n too large");
    hipLaunchKernelGGL(mass_fixed_kernel, dim3(unsigned((n + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream), d, n, out);
    return check_hip(hipGetLastError(), "mass launch");
}

KA_EXPORT int ka_sample_ex(int dtype, const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                           float temperature, const float *temperature_rows, int32_t top_k,
                           const int32_t *top_k_rows, float top_p, const float *top_p_rows, const float *uniforms,
                           int64_t *out_ids, float *out_logprob, float *out_policy_logprob, uint32_t flags,
                           void *workspace, size_t workspace_bytes, void *hip_stream) {
    ka::SampleParams p = ka::scalar_params(temperature, top_k, top_p, uniforms, out_ids);
    p.temperature_rows = temperature_rows;
    p.top_k_rows = top_k_rows;
    p.top_p_rows = top_p_rows;
    p.out_logprob = out_logprob;
    p.out_policy = out_policy_logprob;
    return ka::launch_ex(dtype, logits, batch, vocab, row_stride, p, workspace, workspace_bytes, hip_stream, flags);
}
