// Instantiates the head_dim 256 matrix-core prefill kernels (bf16 / fp16) for contexts longer than their slot tables.
#include "prefill_d256.h"

namespace pa_decode_detail {

prefill_mfma_fn pa_prefill_d256_kernel_long(int dtype, bool lower_bounds) {
    if (dtype == PA_BF16) return lower_bounds ? prefill_d256_kernel<pa_bf16, true, true> : prefill_d256_kernel<pa_bf16, false, true>;
    if (dtype == PA_F16) return lower_bounds ? prefill_d256_kernel<pa_f16, true, true> : prefill_d256_kernel<pa_f16, false, true>;
    return nullptr;
}

}  // namespace pa_decode_detail
