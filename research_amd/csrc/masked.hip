// Attention under an arbitrary (row, key) mask given as bits: the general path behind ctx.block_mask objects that
// are not one of the structured masks the other kernels apply themselves.  Not a fast path: one workgroup per
// (query head, row), every visible key costs a wave-wide reduction.
#include "pa_common.h"

namespace {

constexpr int kMThreads = 256;
constexpr int kMWaves = kMThreads / PA_WAVE;
constexpr int kMaxEpl = 4;  // head_dim up to 256: element d of a row lives in lane d % 64, register d / 64
constexpr int kKeysAtOnce = 4;

struct MaskedArgs {
    const void *q, *k, *v;
    void *out;
    const int32_t *bt;
    int64_t bt_stride;
    const int32_t *ctx_lens, *q_lens, *q_starts;
    const float *k_scale, *v_scale;  // fp8 pools: float [num_blocks][hkv]
    const uint32_t *mask;  // [total rows][mask_heads][mask_words]
    int mask_heads, mask_words, n_keys;
    int hq, hkv, d, bs;
    int64_t num_blocks;
    float scale_log2;
};

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) x += __shfl_xor(x, o, PA_WAVE);
    return x;
}

// One element of a pool row as a float: the pool's own 16- or 32-bit type, or an OCP e4m3 byte (the caller
// multiplies by the tile's scale).
template <typename KV> struct PoolElem {
    static __device__ __forceinline__ float load(const KV *p) { return pa_scalar<KV>::load(p); }
};
template <> struct PoolElem<pa_fp8> {
    static __device__ __forceinline__ float load(const pa_fp8 *p) { return __builtin_amdgcn_cvt_f32_fp8((int)p->bits, 0); }
};

// T: type of q and out; KV: type of the pool (T itself, or fp8-e4m3 with per-(block, kv head) scales).
template <typename T, typename KV>
__global__ __launch_bounds__(kMThreads) void attend_masked_kernel(const MaskedArgs a) {
    constexpr bool kFp8 = sizeof(KV) == 1;
    __shared__ float s_acc[kMWaves][kMaxEpl * PA_WAVE];
    __shared__ float s_ml[kMWaves][2];
    const int h = blockIdx.x, row = blockIdx.y, b = blockIdx.z;
    if (row >= a.q_lens[b]) return;  // uniform
    const int lane = threadIdx.x & (PA_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PA_WAVE);
    const int64_t grow = (int64_t)a.q_starts[b] + row;
    const int ctx_len = a.ctx_lens[b];
    const int kvh = h / (a.hq / a.hkv);
    const int epl = (a.d + PA_WAVE - 1) / PA_WAVE;
    const T *qrow = reinterpret_cast<const T *>(a.q) + (grow * a.hq + h) * a.d;
    float q[kMaxEpl], acc[kMaxEpl];
#pragma unroll
    for (int i = 0; i < kMaxEpl; ++i) {
        const int e = lane + i * PA_WAVE;
        q[i] = i < epl && e < a.d ? pa_scalar<T>::load(qrow + e) * a.scale_log2 : 0.f;
        acc[i] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    const uint32_t *mrow = a.mask + (grow * a.mask_heads + (a.mask_heads == 1 ? 0 : h)) * (int64_t)a.mask_words;
    const int32_t *bt = a.bt + (int64_t)b * a.bt_stride;
    const int n_words = (a.n_keys + 31) / 32;

    // pool row of key j, or -1 for a zero row (past the context end, or in an absent block)
    auto slot_of = [&](int j) -> int64_t {
        if (j >= ctx_len) return -1;
        const int blk = j / a.bs;
        if (blk >= a.bt_stride) return -1;
        const int64_t bid = bt[blk];
        return bid >= 0 && bid < a.num_blocks ? bid * a.bs + j % a.bs : -1;
    };
    for (int w = wave; w < n_words; w += kMWaves) {
        uint32_t bits = __builtin_amdgcn_readfirstlane(mrow[w]);
        if (w == n_words - 1 && (a.n_keys & 31)) bits &= (1u << (a.n_keys & 31)) - 1u;
        while (bits) {
            int key[kKeysAtOnce];
            float kx[kKeysAtOnce][kMaxEpl], vx[kKeysAtOnce][kMaxEpl];
            int n = 0;
#pragma unroll
            for (int t = 0; t < kKeysAtOnce; ++t) {
                key[t] = -1;
                if (bits) {
                    key[t] = w * 32 + __builtin_ctz(bits);
                    bits &= bits - 1;
                    n = t + 1;
                }
            }
#pragma unroll
            for (int t = 0; t < kKeysAtOnce; ++t) {
                const int64_t slot = key[t] >= 0 ? slot_of(key[t]) : -1;
                const KV *kr = reinterpret_cast<const KV *>(a.k) + (slot * a.hkv + kvh) * a.d;
                const KV *vr = reinterpret_cast<const KV *>(a.v) + (slot * a.hkv + kvh) * a.d;
                float ks = 1.f, vs = 1.f;
                if (kFp8 && slot >= 0) {
                    ks = a.k_scale[slot / a.bs * a.hkv + kvh];
                    vs = a.v_scale[slot / a.bs * a.hkv + kvh];
                }
#pragma unroll
                for (int i = 0; i < kMaxEpl; ++i) {
                    const int e = lane + i * PA_WAVE;
                    const bool live = slot >= 0 && i < epl && e < a.d;
                    kx[t][i] = live ? PoolElem<KV>::load(kr + e) * ks : 0.f;
                    vx[t][i] = live ? PoolElem<KV>::load(vr + e) * vs : 0.f;
                }
            }
            float s[kKeysAtOnce];
#pragma unroll
            for (int t = 0; t < kKeysAtOnce; ++t) {
                float p = 0.f;
#pragma unroll
                for (int i = 0; i < kMaxEpl; ++i) p = fmaf(q[i], kx[t][i], p);
                s[t] = wave_sum(p);  // base-2 logit (the scale and log2(e) are folded into q)
            }
#pragma unroll
            for (int t = 0; t < kKeysAtOnce; ++t) {
                if (t >= n) break;  // uniform
                const float m_new = fmaxf(m, s[t]);
                const float alpha = exp2f(m - m_new);  // exp2(-inf) = 0 on the first key
                const float p = exp2f(s[t] - m_new);
                l = l * alpha + p;
#pragma unroll
                for (int i = 0; i < kMaxEpl; ++i) acc[i] = fmaf(p, vx[t][i], acc[i] * alpha);
                m = m_new;
            }
        }
    }
    // merge the four waves' partial rows
#pragma unroll
    for (int i = 0; i < kMaxEpl; ++i) s_acc[wave][lane + i * PA_WAVE] = acc[i];
    if (lane == 0) { s_ml[wave][0] = m; s_ml[wave][1] = l; }
    __syncthreads();
    if (wave != 0) return;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < kMWaves; ++w) M = fmaxf(M, s_ml[w][0]);
    float den = 0.f, num[kMaxEpl] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < kMWaves; ++w) {
        const float wgt = s_ml[w][1] > 0.f ? exp2f(s_ml[w][0] - M) : 0.f;
        den += wgt * s_ml[w][1];
#pragma unroll
        for (int i = 0; i < kMaxEpl; ++i) num[i] = fmaf(wgt, s_acc[w][lane + i * PA_WAVE], num[i]);
    }
    const float inv = den > 0.f ? 1.f / den : 0.f;  // a row that sees no key gives zeros
    T *orow = reinterpret_cast<T *>(a.out) + (grow * a.hq + h) * a.d;
#pragma unroll
    for (int i = 0; i < kMaxEpl; ++i) {
        const int e = lane + i * PA_WAVE;
        if (i < epl && e < a.d) pa_scalar<T>::store(orow + e, num[i] * inv);
    }
}

}  // namespace

extern "C" int pa_attend_masked(const void *q, const void *k_cache, const void *v_cache, void *out,
                                const int32_t *block_tables, int64_t bt_stride, const int32_t *ctx_lens,
                                const int32_t *q_lens, const int32_t *q_starts, const uint32_t *mask, int mask_heads,
                                int mask_words, int n_keys, int batch, int max_q_len, int num_q_heads,
                                int num_kv_heads, int head_dim, int block_size, int64_t num_blocks, float scale,
                                int dtype, int kv_dtype, const float *k_scale, const float *v_scale, void *stream) {
    pa_clear_error();
    PA_REQUIRE(batch >= 0 && max_q_len >= 0 && n_keys >= 0, "batch / max_q_len / n_keys must be non-negative");
    PA_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && num_q_heads % num_kv_heads == 0,
               "num_q_heads=%d must be a positive multiple of num_kv_heads=%d", num_q_heads, num_kv_heads);
    PA_REQUIRE(head_dim > 0 && head_dim <= kMaxEpl * PA_WAVE, "head_dim=%d must be in 1..%d", head_dim, kMaxEpl * PA_WAVE);
    PA_REQUIRE(block_size > 0 && num_blocks >= 0 && bt_stride >= 0, "block_size / num_blocks / bt_stride out of range");
    PA_REQUIRE(mask_heads == 1 || mask_heads == num_q_heads, "mask_heads=%d must be 1 or num_q_heads", mask_heads);
    PA_REQUIRE((int64_t)mask_words * 32 >= n_keys, "mask_words=%d hold fewer than n_keys=%d bits", mask_words, n_keys);
    PA_REQUIRE(batch <= 65535 && max_q_len <= 65535, "batch=%d / max_q_len=%d above 65535", batch, max_q_len);
    if (dtype != PA_F32 && dtype != PA_BF16 && dtype != PA_F16)
        return pa_fail(PA_ERR_UNSUPPORTED, "pa_attend_masked: dtype=%d is not F32, BF16 or F16", dtype);
    if (kv_dtype != dtype && !(kv_dtype == PA_FP8_E4M3 && dtype != PA_F32))
        return pa_fail(PA_ERR_UNSUPPORTED,
                       "pa_attend_masked: kv_dtype=%d must be the dtype of q (%d), or FP8_E4M3 with 16-bit q", kv_dtype, dtype);
    if (batch == 0 || max_q_len == 0) return PA_OK;
    PA_REQUIRE(q && out && ctx_lens && q_lens && q_starts && k_cache && v_cache, "NULL argument");
    PA_REQUIRE(kv_dtype != PA_FP8_E4M3 || (k_scale && v_scale), "fp8 KV needs k_scale and v_scale");
    PA_REQUIRE(mask || n_keys == 0, "NULL mask");
    PA_REQUIRE(block_tables || bt_stride == 0, "NULL block_tables with bt_stride=%lld", (long long)bt_stride);
    MaskedArgs a;
    a.q = q; a.k = k_cache; a.v = v_cache; a.out = out; a.bt = block_tables; a.bt_stride = bt_stride;
    a.ctx_lens = ctx_lens; a.q_lens = q_lens; a.q_starts = q_starts;
    a.mask = mask; a.mask_heads = mask_heads; a.mask_words = mask_words; a.n_keys = n_keys;
    a.hq = num_q_heads; a.hkv = num_kv_heads; a.d = head_dim; a.bs = block_size; a.num_blocks = num_blocks;
    a.scale_log2 = scale * 1.4426950408889634f;
    const dim3 grid((unsigned)num_q_heads, (unsigned)max_q_len, (unsigned)batch), block(kMThreads);
    hipStream_t s = (hipStream_t)stream;
    a.k_scale = k_scale; a.v_scale = v_scale;
    if (kv_dtype == PA_FP8_E4M3) {
        if (dtype == PA_BF16) attend_masked_kernel<pa_bf16, pa_fp8><<<grid, block, 0, s>>>(a);
        else attend_masked_kernel<pa_f16, pa_fp8><<<grid, block, 0, s>>>(a);
    } else if (dtype == PA_F32) attend_masked_kernel<float, float><<<grid, block, 0, s>>>(a);
    else if (dtype == PA_BF16) attend_masked_kernel<pa_bf16, pa_bf16><<<grid, block, 0, s>>>(a);
    else attend_masked_kernel<pa_f16, pa_f16><<<grid, block, 0, s>>>(a);
    PA_CHECK_LAUNCH("pa_attend_masked");
    return PA_OK;
}
