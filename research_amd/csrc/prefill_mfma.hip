// Instantiates the matrix-core prefill kernels (bf16 / fp16, head_dim 32, 64, 128).
#include "prefill_mfma.h"

namespace pa_decode_detail {

template <typename T> static prefill_mfma_fn by_shape(int d, bool bs16) {
    if (d == 32) return bs16 ? prefill_mfma_kernel<T, 32, true> : prefill_mfma_kernel<T, 32, false>;
    if (d == 64) return bs16 ? prefill_mfma_kernel<T, 64, true> : prefill_mfma_kernel<T, 64, false>;
    if (d == 128) return bs16 ? prefill_mfma_kernel<T, 128, true> : prefill_mfma_kernel<T, 128, false>;
    return nullptr;
}

prefill_mfma_fn pa_prefill_mfma_kernel(int dtype, int d, bool bs16) {
    if (dtype == PA_BF16) return by_shape<pa_bf16>(d, bs16);
    if (dtype == PA_F16) return by_shape<pa_f16>(d, bs16);
    return nullptr;
}

}  // namespace pa_decode_detail
