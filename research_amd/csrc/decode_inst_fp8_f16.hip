// Instantiates the single-query-row attention kernels for a fp8 KV pool with f16 queries.
#include "decode_impl.h"

namespace pa_decode_detail {
KernelSet pa_kernels_fp8_f16(int d, int nrep_t) { return kernels_for<pa_fp8, pa_f16>(d, nrep_t); }
}  // namespace pa_decode_detail
