// Instantiates the single-query-row attention kernels for a bf16 KV pool.
#include "decode_impl.h"

namespace pa_decode_detail {
KernelSet pa_kernels_bf16(int d, int nrep_t) { return kernels_for<pa_bf16, pa_bf16>(d, nrep_t); }
}  // namespace pa_decode_detail
