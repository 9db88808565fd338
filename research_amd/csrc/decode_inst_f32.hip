// Instantiates the single-query-row attention kernels for a f32 KV pool.
#include "decode_impl.h"

namespace pa_decode_detail {
KernelSet pa_kernels_f32(int d, int nrep_t) { return kernels_for<float, float>(d, nrep_t); }
}  // namespace pa_decode_detail
