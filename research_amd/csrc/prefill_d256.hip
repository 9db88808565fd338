// Instantiates the head_dim 256 matrix-core prefill kernels (bf16 / fp16) whose tables are filled once; those that
// fill them again on the way are in prefill_d256_long.hip.
#include "prefill_d256.h"

namespace pa_decode_detail {

prefill_mfma_fn pa_prefill_d256_kernel(int dtype, bool lower_bounds, bool long_table) {
    if (long_table) return pa_prefill_d256_kernel_long(dtype, lower_bounds);
    if (dtype == PA_BF16) return lower_bounds ? prefill_d256_kernel<pa_bf16, true, false> : prefill_d256_kernel<pa_bf16, false, false>;
    if (dtype == PA_F16) return lower_bounds ? prefill_d256_kernel<pa_f16, true, false> : prefill_d256_kernel<pa_f16, false, false>;
    return nullptr;
}

}  // namespace pa_decode_detail
