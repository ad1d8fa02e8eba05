// The top-k route of the sampling kernel on 512 threads per row: two workgroups share a CU, so one row's selection runs
// while the other row streams in.  Launched for aligned rows of at most 131,072 16-bit or 262,144 fp32 entries when the
// batch holds more rows than the device has CUs; same ids, same log-probabilities as the 1024-thread build.
#define KA_SAMPLING_THREADS 512
#include "ka_sampling_kernel.h"

namespace ka {

hipError_t launch_sample_rows_half(int dtype, const void *logits, int64_t batch, int vocab, int64_t row_stride,
                                   const SampleParams &prm, int path_bits, hipStream_t stream) {
    if (dtype == KA_DTYPE_BF16)
        hipLaunchKernelGGL((sample_rows<Bf16, false>), dim3(unsigned(batch)), dim3(S_THREADS), 0, stream,
                           static_cast<const Bf16::raw_t *>(logits), vocab, row_stride, prm, 1, path_bits);
    else if (dtype == KA_DTYPE_F16)
        hipLaunchKernelGGL((sample_rows<F16, false>), dim3(unsigned(batch)), dim3(S_THREADS), 0, stream,
                           static_cast<const F16::raw_t *>(logits), vocab, row_stride, prm, 1, path_bits);
    else
        hipLaunchKernelGGL((sample_rows<F32, false>), dim3(unsigned(batch)), dim3(S_THREADS), 0, stream,
                           static_cast<const F32::raw_t *>(logits), vocab, row_stride, prm, 1, path_bits);
    return hipGetLastError();
}

}  // namespace ka
