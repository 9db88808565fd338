// KV append (scatter by slot) and block-table gather: pure row copies,
// HBM-bound, bit-exact.  One thread moves one vector (16 B when the row and
// the pointers allow it, else 4 B) of the K row and the matching one of the V
// row, so consecutive lanes touch consecutive addresses on both sides.
#include "pa_common.h"

namespace {

template <typename V>
__global__ __launch_bounds__(256) void kv_scatter_kernel(
    V *__restrict__ k_cache, V *__restrict__ v_cache, const V *__restrict__ k_src,
    const V *__restrict__ v_src, const int64_t *__restrict__ slots, int64_t n_vec_total,
    int vec_per_row, int64_t total_slots) {
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= n_vec_total) return;
    const int64_t tok = gid / vec_per_row;
    const int j = (int)(gid - tok * vec_per_row);
    const int64_t slot = slots[tok];
    if (slot < 0 || slot >= total_slots) return;  // dropped row
    const int64_t dst = slot * vec_per_row + j;
    k_cache[dst] = k_src[gid];
    v_cache[dst] = v_src[gid];
}

template <typename V>
__global__ __launch_bounds__(256) void kv_gather_kernel(
    const V *__restrict__ k_cache, const V *__restrict__ v_cache, V *__restrict__ k_out,
    V *__restrict__ v_out, const int32_t *__restrict__ block_tables, int64_t bt_stride,
    const int32_t *__restrict__ seq_lens, int64_t n_vec_total, int64_t max_len, int vec_per_row,
    int64_t num_blocks, int block_size) {
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= n_vec_total) return;
    const int64_t row = gid / vec_per_row;  // = b * max_len + pos
    const int j = (int)(gid - row * vec_per_row);
    const int64_t b = row / max_len;
    const int64_t pos = row - b * max_len;
    V kv{}, vv{};
    if (pos < (int64_t)seq_lens[b]) {
        const int64_t blk = pos / block_size;
        if (blk < bt_stride) {
            const int64_t bid = block_tables[b * bt_stride + blk];
            if (bid >= 0 && bid < num_blocks) {
                const int64_t src = (bid * block_size + (pos - blk * block_size)) * vec_per_row + j;
                kv = k_cache[src];
                vv = v_cache[src];
            }
        }
    }
    k_out[gid] = kv;
    v_out[gid] = vv;
}

int check_row(int num_kv_heads, int head_dim, int elem_bytes, int64_t *row_bytes) {
    PA_REQUIRE(num_kv_heads > 0 && head_dim > 0, "num_kv_heads=%d head_dim=%d must be positive",
               num_kv_heads, head_dim);
    PA_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4, "elem_bytes=%d not in {1,2,4}",
               elem_bytes);
    *row_bytes = (int64_t)num_kv_heads * head_dim * elem_bytes;
    PA_REQUIRE(*row_bytes % 4 == 0, "row of %lld bytes is not a multiple of 4", (long long)*row_bytes);
    return PA_OK;
}

}  // namespace

extern "C" int pa_kv_scatter(void *k_cache, void *v_cache, const void *k_src, const void *v_src,
                             const int64_t *slots, int64_t n_tokens, int64_t total_slots,
                             int num_kv_heads, int head_dim, int elem_bytes, void *stream) {
    pa_clear_error();
    PA_REQUIRE(n_tokens >= 0, "n_tokens=%lld is negative", (long long)n_tokens);
    PA_REQUIRE(total_slots >= 0, "total_slots=%lld is negative", (long long)total_slots);
    int64_t row_bytes = 0;
    if (int rc = check_row(num_kv_heads, head_dim, elem_bytes, &row_bytes)) return rc;
    if (n_tokens == 0) return PA_OK;
    PA_REQUIRE(k_cache && v_cache && k_src && v_src && slots, "NULL buffer with n_tokens=%lld",
               (long long)n_tokens);
    PA_REQUIRE(((uintptr_t)slots & 7u) == 0, "slots is not 8-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const bool wide = row_bytes % 16 == 0 && pa_aligned16(k_cache) && pa_aligned16(v_cache) &&
                      pa_aligned16(k_src) && pa_aligned16(v_src);
    const int vec = wide ? 16 : 4;
    PA_REQUIRE(wide || (((uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)k_src | (uintptr_t)v_src) & 3u) == 0,
               "buffers are not 4-byte aligned");
    const int vec_per_row = (int)(row_bytes / vec);
    const int64_t n_vec = n_tokens * vec_per_row;
    const int64_t grid = (n_vec + 255) / 256;
    PA_REQUIRE(grid <= 0x7fffffff, "n_tokens=%lld is too large for one launch", (long long)n_tokens);
    if (wide)
        kv_scatter_kernel<uint4><<<dim3((unsigned)grid), dim3(256), 0, s>>>(
            (uint4 *)k_cache, (uint4 *)v_cache, (const uint4 *)k_src, (const uint4 *)v_src, slots, n_vec,
            vec_per_row, total_slots);
    else
        kv_scatter_kernel<uint32_t><<<dim3((unsigned)grid), dim3(256), 0, s>>>(
            (uint32_t *)k_cache, (uint32_t *)v_cache, (const uint32_t *)k_src, (const uint32_t *)v_src,
            slots, n_vec, vec_per_row, total_slots);
    PA_CHECK_LAUNCH("pa_kv_scatter");
    return PA_OK;
}

extern "C" int pa_kv_gather(const void *k_cache, const void *v_cache, void *k_out, void *v_out,
                            const int32_t *block_tables, int64_t bt_stride, const int32_t *seq_lens,
                            int batch, int64_t max_len, int64_t num_blocks, int block_size,
                            int num_kv_heads, int head_dim, int elem_bytes, void *stream) {
    pa_clear_error();
    PA_REQUIRE(batch >= 0 && max_len >= 0, "batch=%d max_len=%lld must be non-negative", batch,
               (long long)max_len);
    PA_REQUIRE(block_size > 0, "block_size=%d must be positive", block_size);
    PA_REQUIRE(num_blocks >= 0 && bt_stride >= 0, "num_blocks=%lld bt_stride=%lld must be non-negative",
               (long long)num_blocks, (long long)bt_stride);
    int64_t row_bytes = 0;
    if (int rc = check_row(num_kv_heads, head_dim, elem_bytes, &row_bytes)) return rc;
    if (batch == 0 || max_len == 0) return PA_OK;
    PA_REQUIRE(k_out && v_out && seq_lens, "NULL output or seq_lens");
    PA_REQUIRE(k_cache && v_cache, "NULL cache pointer");
    PA_REQUIRE(block_tables || bt_stride == 0, "NULL block_tables with bt_stride=%lld", (long long)bt_stride);
    hipStream_t s = (hipStream_t)stream;
    const bool wide = row_bytes % 16 == 0 && pa_aligned16(k_cache) && pa_aligned16(v_cache) &&
                      pa_aligned16(k_out) && pa_aligned16(v_out);
    const int vec = wide ? 16 : 4;
    PA_REQUIRE(wide || (((uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)k_out | (uintptr_t)v_out) & 3u) == 0,
               "buffers are not 4-byte aligned");
    const int vec_per_row = (int)(row_bytes / vec);
    const int64_t n_vec = (int64_t)batch * max_len * vec_per_row;
    const int64_t grid = (n_vec + 255) / 256;
    PA_REQUIRE(grid <= 0x7fffffff, "batch*max_len=%lld rows is too large for one launch",
               (long long)batch * max_len);
    if (wide)
        kv_gather_kernel<uint4><<<dim3((unsigned)grid), dim3(256), 0, s>>>(
            (const uint4 *)k_cache, (const uint4 *)v_cache, (uint4 *)k_out, (uint4 *)v_out, block_tables,
            bt_stride, seq_lens, n_vec, max_len, vec_per_row, num_blocks, block_size);
    else
        kv_gather_kernel<uint32_t><<<dim3((unsigned)grid), dim3(256), 0, s>>>(
            (const uint32_t *)k_cache, (const uint32_t *)v_cache, (uint32_t *)k_out, (uint32_t *)v_out,
            block_tables, bt_stride, seq_lens, n_vec, max_len, vec_per_row, num_blocks, block_size);
    PA_CHECK_LAUNCH("pa_kv_gather");
    return PA_OK;
}
