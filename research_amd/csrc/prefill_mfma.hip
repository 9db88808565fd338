// Instantiates the matrix-core prefill kernels (bf16 / fp16, head_dim 32, 64, 128).
#include "prefill_mfma.h"

namespace pa_decode_detail {

prefill_mfma_fn pa_prefill_mfma_kernel(int dtype, int d) {
    if (dtype == PA_BF16) {
        if (d == 32) return prefill_mfma_kernel<pa_bf16, 32>;
        if (d == 64) return prefill_mfma_kernel<pa_bf16, 64>;
        if (d == 128) return prefill_mfma_kernel<pa_bf16, 128>;
    } else if (dtype == PA_F16) {
        if (d == 32) return prefill_mfma_kernel<pa_f16, 32>;
        if (d == 64) return prefill_mfma_kernel<pa_f16, 64>;
        if (d == 128) return prefill_mfma_kernel<pa_f16, 128>;
    }
    return nullptr;
}

}  // namespace pa_decode_detail
