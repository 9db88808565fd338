// Instantiates the head_dim 32 prefill kernels whose tile loop is scheduled assembly (bf16 / fp16, without and with
// lower bounds).
#include "prefill_asm.h"

namespace pa_decode_detail {

prefill_mfma_fn pa_prefill_asm_kernel_d32(int dtype, bool lower_bounds) {
    if (dtype == PA_BF16) return lower_bounds ? prefill_asm_kernel<pa_bf16, true, 32> : prefill_asm_kernel<pa_bf16, false, 32>;
    if (dtype == PA_F16) return lower_bounds ? prefill_asm_kernel<pa_f16, true, 32> : prefill_asm_kernel<pa_f16, false, 32>;
    return nullptr;
}

}  // namespace pa_decode_detail
