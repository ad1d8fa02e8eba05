// Fused lm_head -> logprob (placeholder entry points while the kernel is being written).
#include "ka_common.h"

KA_EXPORT size_t ka_lmhead_workspace_bytes(int64_t n_rows, int64_t hidden_dim, int64_t vocab) { return 256; }

KA_EXPORT int ka_lmhead_logprob_bf16(const void *, const void *, const int64_t *, float *, int64_t, int64_t,
                                     int64_t, void *, size_t, void *) {
    return ka::fail(KA_ERR_UNSUPPORTED, "ka_lmhead_logprob_bf16: not implemented");
}
