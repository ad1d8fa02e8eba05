// Fused sampling (placeholder entry points while the kernels are being written).
#include "ka_common.h"

KA_EXPORT size_t ka_sample_workspace_bytes(int64_t batch, int64_t vocab) { return 256; }

#define KA_SAMPLE_STUB(name)                                                                          \
    KA_EXPORT int name(const void *, int64_t, int64_t, int64_t, float, int32_t, float, const float *, \
                       int64_t *, void *, size_t, void *) {                                           \
        return ka::fail(KA_ERR_UNSUPPORTED, #name ": not implemented");                               \
    }
KA_SAMPLE_STUB(ka_sample_topk_topp_bf16)
KA_SAMPLE_STUB(ka_sample_topk_topp_f16)
KA_SAMPLE_STUB(ka_sample_topk_topp_f32)
