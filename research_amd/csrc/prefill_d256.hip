// Instantiates the head_dim 256 matrix-core prefill kernels (bf16 / fp16).
#include "prefill_d256.h"

namespace pa_decode_detail {

// `checked`: block sizes that are not multiples of 16 (compiled loop); otherwise the instances whose subtile loop is
// scheduled assembly, one without and one with lower bounds (a sliding window or per-row first keys).
prefill_mfma_fn pa_prefill_d256_kernel(int dtype, bool checked, bool lower_bounds) {
    if (dtype == PA_BF16)
        return checked ? prefill_d256_kernel<pa_bf16, true, false, false>
                       : lower_bounds ? prefill_d256_kernel<pa_bf16, false, true, true> : prefill_d256_kernel<pa_bf16, false, true, false>;
    if (dtype == PA_F16)
        return checked ? prefill_d256_kernel<pa_f16, true, false, false>
                       : lower_bounds ? prefill_d256_kernel<pa_f16, false, true, true> : prefill_d256_kernel<pa_f16, false, true, false>;
    return nullptr;
}

}  // namespace pa_decode_detail
