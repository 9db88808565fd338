// Instantiates the head_dim 64 prefill kernels whose tile loop is scheduled assembly for contexts longer than their
// slot tables (bf16 / fp16, without and with lower bounds).
#include "prefill_asm.h"

namespace pa_decode_detail {

prefill_mfma_fn pa_prefill_asm_kernel_d64_long(int dtype, bool lower_bounds) {
    if (dtype == PA_BF16)
        return lower_bounds ? prefill_asm_kernel<pa_bf16, true, 64, true> : prefill_asm_kernel<pa_bf16, false, 64, true>;
    if (dtype == PA_F16)
        return lower_bounds ? prefill_asm_kernel<pa_f16, true, 64, true> : prefill_asm_kernel<pa_f16, false, 64, true>;
    return nullptr;
}

}  // namespace pa_decode_detail
