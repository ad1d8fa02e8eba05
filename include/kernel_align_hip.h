/*
 * kernel_align_hip.h — C ABI of libkernel_align_hip.so (MI355X / gfx950).
 *
 * The library implements the data-parallel hot path of Kernel-Align as
 * hand-written HIP kernels: the per-token logprob operator, the fused
 * temperature / top-k / top-p sampling operator, and a fused
 * lm_head -> logprob operator.  Every entry point takes plain device pointers
 * and sizes, enqueues work on the caller's HIP stream and returns without
 * synchronising.  The library never allocates or frees device memory and never
 * keeps a pointer after the call returns; scratch space is passed in as a
 * workspace whose size the *_workspace_bytes queries report.
 *
 * Return value of every int-returning entry point: KA_OK (0) or a negative
 * KA_ERR_* code; ka_last_error() then holds a thread-local message.
 *
 * There is no CPU fallback in this library: without a HIP device every compute
 * entry point returns KA_ERR_HIP.
 */
#ifndef KERNEL_ALIGN_HIP_H
#define KERNEL_ALIGN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KA_OK 0
#define KA_ERR_BAD_ARG (-1)      /* null pointer, negative size, top_k < 0, top_p outside (0,1], T <= 0 */
#define KA_ERR_UNSUPPORTED (-2)  /* shape the kernels cannot take (e.g. vocab >= 2^31) */
#define KA_ERR_WORKSPACE (-3)    /* workspace missing or smaller than *_workspace_bytes() */
#define KA_ERR_HIP (-4)          /* a HIP runtime call or kernel launch failed */

/* Element types of a logits tensor. */
#define KA_DTYPE_BF16 0
#define KA_DTYPE_F16 1
#define KA_DTYPE_F32 2

/* Library version string, e.g. "kernel_align_hip 0.4 (gfx950)". */
const char *ka_version(void);
/*
 * Revision of this interface: raised whenever the signature or the meaning of an entry point changes.  A binding
 * compares ka_abi_revision() with the KA_ABI_REVISION it was written against and refuses a library that differs (a
 * caller bound to another prototype would pass its arguments in the wrong places without any error).
 * Result bits of the floating-point operators (fixed summation orders) are stable within one revision of the library,
 * not across revisions; token ids are defined exactly and never change.
 */
#define KA_ABI_REVISION 4
int ka_abi_revision(void);
/* Message of the last error on the calling thread ("" if none). */
const char *ka_last_error(void);
/* Name of a status code. */
const char *ka_status_string(int status);

/*
 * Per-token log-probability:
 *     out[r] = logits[r, ids[r]] - logsumexp_v(logits[r, :])          (fp32)
 * for r in [0, n_rows).  logits is row-major [n_rows, vocab] with
 * row_stride elements between rows; rows are the flattened G*L tokens.
 * Replaces the chunk loop of SamplerBackend.compute_logp
 * (rl_engine/kernels/sampling.py:92-112: log_softmax -> gather -> slice copy)
 * and the native comparator (benchmarks/benchmark_grpo_op.py:52-54).
 * One pass over the logits, fp32 accumulation, no temporary of the size of the
 * logits.  A row's result depends on that row only and is reduced in a fixed
 * order, so outputs are bit-identical across runs, batch sizes and chunkings.
 * An id outside [0, vocab) yields NaN for that row.
 */
int ka_logprob_bf16(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                    const int64_t *ids, float *out, void *hip_stream);
int ka_logprob_f16(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                   const int64_t *ids, float *out, void *hip_stream);
int ka_logprob_f32(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                   const int64_t *ids, float *out, void *hip_stream);

/*
 * Same pass as ka_logprob_*, which also returns the entropy of each row's
 * softmax, entropy[r] = -sum_v p_v log p_v (fp32).  entropy may be null.
 * No counterpart in the reference; GRPO-style losses consume both.
 */
int ka_logprob_entropy_bf16(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                            const int64_t *ids, float *out, float *entropy, void *hip_stream);
int ka_logprob_entropy_f16(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                           const int64_t *ids, float *out, float *entropy, void *hip_stream);
int ka_logprob_entropy_f32(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                           const int64_t *ids, float *out, float *entropy, void *hip_stream);

/*
 * Backward of ka_logprob_*:
 *     dlogits[r, v] = grad[r] * ((v == ids[r]) - softmax(logits[r, :])[v])
 * in the logits' dtype.  logp is the forward result for the same (logits, ids);
 * the row's log-sum-exp is recovered from it, so each logit is read once and
 * its gradient written once (a row whose target logit is -inf, where logp is
 * -inf too, is read twice: its log-sum-exp is recomputed).  dlogits may be the logits buffer itself (same
 * stride): the gradient then overwrites the logits and no second tensor of
 * their size exists.  No counterpart in the reference, whose operators run under
 * torch.inference_mode() (rl_engine/kernels/sampling.py:38,91); this is the
 * gradient autograd would build for sampling.py:108-110.
 */
int ka_logprob_backward_bf16(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                             const int64_t *ids, const float *logp, const float *grad, void *dlogits,
                             int64_t dlogits_stride, void *hip_stream);
int ka_logprob_backward_f16(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                            const int64_t *ids, const float *logp, const float *grad, void *dlogits,
                            int64_t dlogits_stride, void *hip_stream);
int ka_logprob_backward_f32(const void *logits, int64_t n_rows, int64_t vocab, int64_t row_stride,
                            const int64_t *ids, const float *logp, const float *grad, void *dlogits,
                            int64_t dlogits_stride, void *hip_stream);

/*
 * GRPO per-token objective from log-probabilities (all arrays fp32 [n], n = G * L tokens):
 *     ratio = exp(logp_new - logp_old)            (logp_old null: ratio = 1, the on-policy case)
 *     surr  = min(ratio * A, clamp(ratio, 1 - clip_low, 1 + clip_high) * A)
 *     kl    = exp(logp_ref - logp_new) - (logp_ref - logp_new) - 1      (logp_ref null: 0)
 *     out_loss  = -(surr - beta * kl)
 *     out_dlogp = d out_loss / d logp_new   (feeds ka_logprob_backward_* as `grad`)
 * Each output pointer may be null.  No counterpart in the reference, which stops at the log-probabilities
 * (rl_engine/kernels/sampling.py:92-112) and names the advantage step only in README.md:49; this is the
 * elementwise epilogue a GRPO trainer applies to them.
 */
int ka_grpo_token_terms(const float *logp_new, const float *logp_old, const float *logp_ref,
                        const float *advantages, int64_t n, float clip_low, float clip_high, float beta,
                        float *out_loss, float *out_kl, float *out_dlogp, void *hip_stream);

/*
 * Fused temperature -> top-k -> top-p -> draw, one token id per row.
 * Replaces SamplerBackend.sample (rl_engine/kernels/sampling.py:39-88) with the
 * filter semantics of native_sampling (benchmarks/benchmark_sampling.py:12-37):
 *   1. if temperature != 1: y = logits / temperature, rounded to the logits dtype;
 *   2. top_k > 0: keep {y >= k-th largest y}, ties included (top_k == 0: off);
 *   3. top_p < 1: order kept entries by (y descending, index ascending), take
 *      softmax over them, keep an entry iff the mass strictly before it is
 *      <= top_p (the first entry crossing top_p stays); top_p == 1: off;
 *   4. draw: over the survivors in ascending index order, pick the first index
 *      whose inclusive cumulative mass exceeds uniforms[r] * total mass.
 * Masses are exp(y - max y) evaluated by a fixed polynomial and truncated to
 * 2^-40 fixed point, then summed as integers, so the result does not depend on
 * summation order, batch size or launch geometry.
 * uniforms: one fp32 in [0,1) per row.  out_ids: int64 [batch].
 * A NaN logit counts as -inf; a row with nothing above -inf is sampled uniformly.
 */
size_t ka_sample_workspace_bytes(int64_t batch, int64_t vocab);
int ka_sample_topk_topp_bf16(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                             float temperature, int32_t top_k, float top_p, const float *uniforms,
                             int64_t *out_ids, void *workspace, size_t workspace_bytes,
                             void *hip_stream);
int ka_sample_topk_topp_f16(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                            float temperature, int32_t top_k, float top_p, const float *uniforms,
                            int64_t *out_ids, void *workspace, size_t workspace_bytes,
                            void *hip_stream);
int ka_sample_topk_topp_f32(const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                            float temperature, int32_t top_k, float top_p, const float *uniforms,
                            int64_t *out_ids, void *workspace, size_t workspace_bytes,
                            void *hip_stream);

/*
 * The same operator with per-row parameters and the sampled entry's log-probability.
 * dtype is a KA_DTYPE_* code.  Each of temperature_rows / top_k_rows / top_p_rows is either null (the
 * scalar next to it applies to every row) or a device array of `batch` values that replaces the scalar; a
 * row value that is not valid switches that filter off for the row (temperature <= 0 or NaN -> 1,
 * top_k < 0 -> off, top_p outside (0, 1] -> off).  out_logprob (optional, fp32 [batch]) receives
 * log(mass of the sampled entry / total surviving mass), the log-probability under the distribution the
 * entry was drawn from.  The reference takes scalars only (rl_engine/kernels/sampling.py:39); the
 * FlashInfer operators it forwards to accept per-row tensors (sampling.py:62-64).
 * out_policy_logprob (optional, fp32 [batch]) receives the sampled entry's log-probability under the unfiltered
 * softmax of the raw logits, logits[r, id] - logsumexp(logits[r, :]): what ka_logprob_* returns for it (to 1e-5:
 * the sum runs over the row in another fixed order) and what a GRPO ratio is built from.  With top_k <= 256 the
 * log-sum-exp is taken along while the row streams by (a decode step then needs no second kernel); the other
 * routes pass over the row once more at their end.
 * flags (0 in production) selects among routes that compute the same function, so that a caller can check one
 * against the other: KA_SAMPLE_FLAG_GENERAL_PATH runs the general radix-select path even where a shorter route
 * applies; KA_SAMPLE_FLAG_BLOCK_WIDE_TOPK keeps the top-k route on its block-wide selection and tail instead of the
 * short ones it takes for top_k <= 256 (bound from pooled maxima up to top_k = 64, from a radix descent above).  Ids
 * and log-probabilities do not depend on the flags.  KA_SAMPLE_FLAG_TWO_ROWS_PER_CU / KA_SAMPLE_FLAG_ONE_ROW_PER_CU: the
 * short top-k route (scalar top_k <= 256, 16-byte aligned rows of at most 131,072 16-bit or 262,144 fp32 entries) exists on 512 and on
 * 1024 threads per row; the library takes 512, with two rows resident per CU, for batches of more rows than the device has
 * CUs, and these flags force either where the row qualifies (both give the same ids and the same log-probability bits).
 */
#define KA_SAMPLE_FLAG_GENERAL_PATH 1u
#define KA_SAMPLE_FLAG_BLOCK_WIDE_TOPK 2u
#define KA_SAMPLE_FLAG_TWO_ROWS_PER_CU 4u
#define KA_SAMPLE_FLAG_ONE_ROW_PER_CU 8u
int ka_sample_ex(int dtype, const void *logits, int64_t batch, int64_t vocab, int64_t row_stride,
                 float temperature, const float *temperature_rows, int32_t top_k, const int32_t *top_k_rows,
                 float top_p, const float *top_p_rows, const float *uniforms, int64_t *out_ids,
                 float *out_logprob, float *out_policy_logprob, uint32_t flags, void *workspace,
                 size_t workspace_bytes, void *hip_stream);

/*
 * The integer mass function of the sampling operator, element-wise: out[i] = W(d[i]) =
 * trunc(2^40 * exp(d[i])) for d <= 0 (W(0) = 2^40, 0 once d * log2(e) < -41), evaluated by the fixed
 * operation sequence the sampling kernels use.  Exported so that the function every sampled id depends on
 * can be checked bit for bit against its CPU statement; no counterpart in the reference, whose masses are
 * torch.softmax values (benchmarks/benchmark_sampling.py:27,36).
 */
int ka_sample_mass_fixed(const float *d, int64_t n, uint64_t *out, void *hip_stream);

/*
 * Fused lm_head -> logprob without materialised logits:
 *     out[r] = h_r . W[ids[r]] - logsumexp_v(h_r . W[v])               (fp32)
 * hidden: bf16 [n_rows, hidden_dim] row-major; weight: bf16 [vocab, hidden_dim]
 * row-major (the nn.Linear.weight layout).  bf16 MFMA with fp32 accumulation;
 * logit tiles stay in registers and feed an online max / log-sum-exp.
 * hidden_dim must be a multiple of 64 and both matrices 16-byte aligned; the
 * workspace (as the query reports: 16 bytes per row and vocabulary split, four
 * times that for calls of so few rows - token blocks x splits < 256 - that every
 * split is spread over four workgroups to fill the part) must be 16-byte
 * aligned.  A row's result does not depend on n_rows, bit for bit.  An id outside
 * [0, vocab) gives NaN for its row.  The kernel is launched as one workgroup
 * per CU, each walking its share of the work.
 * No counterpart in the reference; the nearest behaviour is
 * compute_logp(lm_head(hidden)) (rl_engine/kernels/sampling.py:92-112).
 */
size_t ka_lmhead_workspace_bytes(int64_t n_rows, int64_t hidden_dim, int64_t vocab);
int ka_lmhead_logprob_bf16(const void *hidden, const void *weight, const int64_t *ids, float *out,
                           int64_t n_rows, int64_t hidden_dim, int64_t vocab, void *workspace,
                           size_t workspace_bytes, void *hip_stream);

/*
 * ka_lmhead_logprob_bf16 that also returns the entropy of every row's softmax over the vocabulary,
 * entropy[r] = -sum_v p_v log p_v (fp32), from the same pass: one more accumulator per token in the kernel
 * (about 1 % more time), same workspace.  No counterpart in the reference; GRPO-style losses consume both.
 */
int ka_lmhead_logprob_entropy_bf16(const void *hidden, const void *weight, const int64_t *ids, float *out,
                                   float *entropy, int64_t n_rows, int64_t hidden_dim, int64_t vocab,
                                   void *workspace, size_t workspace_bytes, void *hip_stream);

/*
 * ka_lmhead_logprob_bf16 that also returns every row's log-sum-exp over the vocabulary, lse[r] (fp32), which the
 * backward below takes; same kernels, same workspace, same log-probabilities bit for bit.
 *
 * ka_lmhead_dlogits_bf16: the first half of the backward of ka_lmhead_logprob_bf16.  The logits tiles are computed
 * again by the forward's MFMA kernel, and every logit x of row r goes out as
 * dlogits[r, v] = grad_logprob[r] * ([v == ids[r]] - exp(x - lse[r])), rounded to bf16, into a [n_rows, vocab] matrix
 * (row stride in elements, a multiple of 4, matrix 8-byte aligned); the logits themselves are never stored.  The
 * caller contracts the matrix with weight (gradient of hidden) and with hidden (gradient of weight).  An id outside
 * [0, vocab) contributes no one-hot term.  No workspace.  No counterpart in the reference, whose operators are
 * inference-only (rl_engine/kernels/sampling.py:38,91).
 */
int ka_lmhead_logprob_lse_bf16(const void *hidden, const void *weight, const int64_t *ids, float *out, float *lse,
                               int64_t n_rows, int64_t hidden_dim, int64_t vocab, void *workspace,
                               size_t workspace_bytes, void *hip_stream);
int ka_lmhead_dlogits_bf16(const void *hidden, const void *weight, const int64_t *ids, const float *lse,
                           const float *grad_logprob, void *dlogits, int64_t dlogits_row_stride, int64_t n_rows,
                           int64_t hidden_dim, int64_t vocab, void *hip_stream);

/*
 * ka_lmhead_logprob_bf16 for callers that cannot allocate device memory or bring a workspace: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same kernels, same results bit
 * for bit; the per-split partials go to a static array in device memory (KA_LMHEAD_STATIC_SCRATCH_BYTES,
 * one copy on every GPU the library runs on, held until the process ends) instead of a workspace, and the
 * call makes no hipMalloc / hipFree.  It has no counterpart in the reference.
 * Limit: ka_lmhead_workspace_bytes(n_rows, hidden_dim, vocab) <= KA_LMHEAD_STATIC_SCRATCH_BYTES (16,384
 * rows at a vocabulary of 128,256: 16 MiB; up to 768 rows the same vocabulary takes 64 KiB per row: 3 MiB); more returns KA_ERR_WORKSPACE and nothing is launched.  Every call on
 * a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race; calls on
 * one stream are ordered and safe.  The first call on a device looks the array's address up (one
 * hipGetSymbolAddress and the kernels' attribute set-up), so make one call per device before capturing.
 */
#define KA_LMHEAD_STATIC_SCRATCH_BYTES (16u << 20)
int ka_lmhead_logprob_bf16_noalloc(const void *hidden, const void *weight, const int64_t *ids, float *out,
                                   int64_t n_rows, int64_t hidden_dim, int64_t vocab, void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* KERNEL_ALIGN_HIP_H */
