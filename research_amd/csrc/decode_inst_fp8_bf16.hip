// Instantiates the single-query-row attention kernels for a fp8 KV pool with bf16 queries.
#include "decode_impl.h"

namespace pa_decode_detail {
KernelSet pa_kernels_fp8_bf16(int d, int nrep_t) { return kernels_for<pa_fp8, pa_bf16>(d, nrep_t); }
}  // namespace pa_decode_detail
