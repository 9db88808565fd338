// Selects among the prefill kernels whose tile loop is scheduled assembly; one translation unit per head size
// instantiates them (prefill_asm_d128.hip, prefill_asm_d64.hip, prefill_asm_d32.hip, and prefill_asm_d*_long.hip for the
// instances that fill their tables more than once: they compile side by side).
#include "prefill_mfma.h"

namespace pa_decode_detail {

prefill_mfma_fn pa_prefill_asm_kernel_d128(int dtype, bool lower_bounds);
prefill_mfma_fn pa_prefill_asm_kernel_d128_long(int dtype, bool lower_bounds);
prefill_mfma_fn pa_prefill_asm_kernel_d64_long(int dtype, bool lower_bounds);
prefill_mfma_fn pa_prefill_asm_kernel_d32_long(int dtype, bool lower_bounds);
prefill_mfma_fn pa_prefill_asm_kernel_d64(int dtype, bool lower_bounds);
prefill_mfma_fn pa_prefill_asm_kernel_d32(int dtype, bool lower_bounds);

prefill_mfma_fn pa_prefill_asm_kernel(int dtype, int head_dim, bool lower_bounds, bool long_table) {
    if (long_table) {
        if (head_dim == 128) return pa_prefill_asm_kernel_d128_long(dtype, lower_bounds);
        if (head_dim == 64) return pa_prefill_asm_kernel_d64_long(dtype, lower_bounds);
        if (head_dim == 32) return pa_prefill_asm_kernel_d32_long(dtype, lower_bounds);
        return nullptr;
    }
    if (head_dim == 128) return pa_prefill_asm_kernel_d128(dtype, lower_bounds);
    if (head_dim == 64) return pa_prefill_asm_kernel_d64(dtype, lower_bounds);
    if (head_dim == 32) return pa_prefill_asm_kernel_d32(dtype, lower_bounds);
    return nullptr;
}

}  // namespace pa_decode_detail
