// Instantiates the head_dim 128 prefill kernels whose tile loop is scheduled assembly (bf16 / fp16).
#include "prefill_asm.h"

namespace pa_decode_detail {

prefill_mfma_fn pa_prefill_asm_kernel(int dtype) {
    if (dtype == PA_BF16) return prefill_asm_kernel<pa_bf16>;
    if (dtype == PA_F16) return prefill_asm_kernel<pa_f16>;
    return nullptr;
}

}  // namespace pa_decode_detail
