// fp8-e4m3 pool construction: one workgroup per (block, kv head) finds the
// absolute maximum of the block_size x head_dim tile, stores scale = max/448
// and writes the tile as OCP e4m3fn bytes of x/scale (round to nearest even).
#include "pa_common.h"

namespace {

constexpr int kQThreads = 256;

template <typename T>
__global__ __launch_bounds__(kQThreads) void quantize_e4m3_kernel(const T *__restrict__ src,
                                                                   uint8_t *__restrict__ dst,
                                                                   float *__restrict__ scale, int block_size,
                                                                   int hkv, int d) {
    __shared__ float s_max[kQThreads / PA_WAVE];
    const int64_t blk = blockIdx.x / hkv;
    const int h = blockIdx.x - (int)(blk * hkv);
    const int n = block_size * d;  // elements of the tile
    const int64_t tile0 = (blk * block_size * hkv + h) * (int64_t)d;
    const int64_t tok_stride = (int64_t)hkv * d;

    float amax = 0.f;
    for (int i = threadIdx.x; i < n; i += kQThreads) {
        const int t = i / d, e = i - t * d;
        amax = fmaxf(amax, fabsf(pa_scalar<T>::load(src + tile0 + t * tok_stride + e)));
    }
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
    const float sc = amax > 0.f ? amax / 448.0f : 1.0f;
    if (threadIdx.x == 0) scale[blk * hkv + h] = sc;

    for (int i = threadIdx.x; i < n; i += kQThreads) {
        const int t = i / d, e = i - t * d;
        const float x = pa_scalar<T>::load(src + tile0 + t * tok_stride + e) / sc;
        // gfx950 encodes OCP e4m3fn here; the low byte of the packed pair is x
        const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(x, 0.f, 0, false);
        dst[tile0 + t * tok_stride + e] = (uint8_t)(packed & 0xff);
    }
}

}  // namespace

extern "C" int pa_quantize_kv_e4m3(const void *src, void *dst, float *scale, int64_t num_blocks,
                                   int block_size, int num_kv_heads, int head_dim, int src_dtype,
                                   void *stream) {
    pa_clear_error();
    PA_REQUIRE(num_blocks >= 0, "num_blocks=%lld is negative", (long long)num_blocks);
    PA_REQUIRE(block_size > 0 && num_kv_heads > 0 && head_dim > 0, "block_size / num_kv_heads / head_dim must be positive");
    PA_REQUIRE(src_dtype == PA_F32 || src_dtype == PA_BF16 || src_dtype == PA_F16, "src_dtype=%d is not F32, BF16 or F16",
               src_dtype);
    PA_REQUIRE(num_blocks * num_kv_heads <= 0x7fffffffll, "num_blocks*num_kv_heads above 2^31-1");
    PA_REQUIRE((int64_t)block_size * head_dim <= (1 << 24), "tile of %d x %d elements is too large", block_size, head_dim);
    if (num_blocks == 0) return PA_OK;
    PA_REQUIRE(src && dst && scale, "NULL src / dst / scale");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)(num_blocks * num_kv_heads)), block(kQThreads);
    if (src_dtype == PA_F32)
        quantize_e4m3_kernel<float><<<grid, block, 0, s>>>((const float *)src, (uint8_t *)dst, scale, block_size,
                                                           num_kv_heads, head_dim);
    else if (src_dtype == PA_BF16)
        quantize_e4m3_kernel<pa_bf16><<<grid, block, 0, s>>>((const pa_bf16 *)src, (uint8_t *)dst, scale, block_size,
                                                             num_kv_heads, head_dim);
    else
        quantize_e4m3_kernel<pa_f16><<<grid, block, 0, s>>>((const pa_f16 *)src, (uint8_t *)dst, scale, block_size,
                                                            num_kv_heads, head_dim);
    PA_CHECK_LAUNCH("pa_quantize_kv_e4m3");
    return PA_OK;
}
