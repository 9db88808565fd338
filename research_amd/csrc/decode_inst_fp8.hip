// Instantiates the single-query-row attention kernels for a fp8 KV pool.
#include "decode_impl.h"

namespace pa_decode_detail {
KernelSet pa_kernels_fp8(int q_dtype, int d, int nrep_t) {
    if (q_dtype == PA_BF16) return kernels_for<pa_fp8, pa_bf16>(d, nrep_t);
    if (q_dtype == PA_F16) return kernels_for<pa_fp8, pa_f16>(d, nrep_t);
    return KernelSet{};
}
}  // namespace pa_decode_detail
