// GRPO per-token objective on top of the logprob operator: the clipped policy-gradient surrogate, the k3
// estimator of the KL divergence to a reference policy, and the derivative of the per-token loss with
// respect to the new log-probability (the `grad` input of ka_logprob_backward_*).  Elementwise over the
// [G * L] tokens, fp32, one pass: every input is read once and every output written once.
//
//     ratio = exp(new - old)                                   (old == null: ratio = 1, the on-policy case)
//     surr  = min(ratio * A, clamp(ratio, 1 - clip_low, 1 + clip_high) * A)
//     kl    = exp(ref - new) - (ref - new) - 1                 (ref == null or beta == 0: kl = 0)
//     loss  = -(surr - beta * kl)
//     dloss/dnew = -[ratio * A if ratio * A <= clipped term else 0] + beta * (1 - exp(ref - new))
#include "ka_common.h"

namespace ka {
namespace {

__global__ __launch_bounds__(256) void grpo_token_terms(const float *__restrict__ logp_new,
                                                        const float *__restrict__ logp_old,
                                                        const float *__restrict__ logp_ref,
                                                        const float *__restrict__ adv, int64_t n, float lo, float hi,
                                                        float beta, float *__restrict__ out_loss,
                                                        float *__restrict__ out_kl, float *__restrict__ out_dlogp) {
    const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float lp = logp_new[i];
    const float a = adv[i];
    const float ratio = logp_old != nullptr ? expf(lp - logp_old[i]) : 1.0f;
    const float s1 = ratio * a;
    const float s2 = fminf(fmaxf(ratio, lo), hi) * a;
    const float surr = fminf(s1, s2);
    float kl = 0.0f, dkl = 0.0f;
    if (logp_ref != nullptr) {
        const float d = logp_ref[i] - lp;
        const float e = expf(d);
        kl = e - d - 1.0f;
        dkl = 1.0f - e;
    }
    if (out_loss != nullptr) out_loss[i] = -(surr - beta * kl);
    if (out_kl != nullptr) out_kl[i] = kl;
    if (out_dlogp != nullptr) out_dlogp[i] = -(s1 <= s2 ? s1 : 0.0f) + beta * dkl;
}

}  // namespace
}  // namespace ka

KA_EXPORT int ka_grpo_token_terms(const float *logp_new, const float *logp_old, const float *logp_ref,
                                  const float *advantages, int64_t n, float clip_low, float clip_high, float beta,
                                  float *out_loss, float *out_kl, float *out_dlogp, void *hip_stream) {
    using namespace ka;
    if (n < 0) return fail(KA_ERR_BAD_ARG, "grpo: n %lld < 0", (long long)n);
    if (n == 0) return KA_OK;
    if (logp_new == nullptr || advantages == nullptr)
        return fail(KA_ERR_BAD_ARG, "grpo: null logp_new / advantages pointer");
    if (!(clip_low >= 0.0f && clip_low < 1.0f) || !(clip_high >= 0.0f))
        return fail(KA_ERR_BAD_ARG, "grpo: clip range (%g, %g) must satisfy 0 <= low < 1, high >= 0", clip_low, clip_high);
    if (!(beta >= 0.0f)) return fail(KA_ERR_BAD_ARG, "grpo: beta %g < 0", beta);
    if ((n + 255) / 256 >= (int64_t(1) << 31)) return fail(KA_ERR_UNSUPPORTED, "grpo: n too large");
    hipLaunchKernelGGL(grpo_token_terms, dim3(unsigned((n + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream), logp_new, logp_old, logp_ref, advantages, n,
                       1.0f - clip_low, 1.0f + clip_high, beta, out_loss, out_kl, out_dlogp);
    return check_hip(hipGetLastError(), "grpo launch");
}
