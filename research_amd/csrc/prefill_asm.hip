// Instantiates the prefill kernels whose tile loop is scheduled assembly (head_dim 128, 64 and 32; bf16 / fp16).
#include "prefill_asm.h"

namespace pa_decode_detail {

namespace {
template <int D> prefill_mfma_fn pick(int dtype, bool lower_bounds) {
    if (dtype == PA_BF16) return lower_bounds ? prefill_asm_kernel<pa_bf16, true, D> : prefill_asm_kernel<pa_bf16, false, D>;
    if (dtype == PA_F16) return lower_bounds ? prefill_asm_kernel<pa_f16, true, D> : prefill_asm_kernel<pa_f16, false, D>;
    return nullptr;
}
}  // namespace

prefill_mfma_fn pa_prefill_asm_kernel(int dtype, int head_dim, bool lower_bounds) {
    if (head_dim == 128) return pick<128>(dtype, lower_bounds);
    if (head_dim == 64) return pick<64>(dtype, lower_bounds);
    if (head_dim == 32) return pick<32>(dtype, lower_bounds);
    return nullptr;
}

}  // namespace pa_decode_detail
