// The single-query-row attention kernels for a fp8 KV pool: one translation unit per query type instantiates them
// (decode_inst_fp8_bf16.hip, decode_inst_fp8_f16.hip: they compile side by side).
#include "decode_impl.h"

namespace pa_decode_detail {
KernelSet pa_kernels_fp8_bf16(int d, int nrep_t);
KernelSet pa_kernels_fp8_f16(int d, int nrep_t);

KernelSet pa_kernels_fp8(int q_dtype, int d, int nrep_t) {
    if (q_dtype == PA_BF16) return pa_kernels_fp8_bf16(d, nrep_t);
    if (q_dtype == PA_F16) return pa_kernels_fp8_f16(d, nrep_t);
    return KernelSet{};
}
}  // namespace pa_decode_detail
