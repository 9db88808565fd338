// Instantiates the single-query-row attention kernels for a f16 KV pool.
#include "decode_impl.h"

namespace pa_decode_detail {
KernelSet pa_kernels_f16(int d, int nrep_t) { return kernels_for<pa_f16, pa_f16>(d, nrep_t); }
}  // namespace pa_decode_detail
