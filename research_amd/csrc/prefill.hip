// Host entry point of causal prefill attention over a paged context.
#include "prefill_mfma.h"
#include "prefill_plan.h"

namespace pa_decode_detail {
prefill_mfma_fn pa_prefill_asm_kernel(int dtype, int head_dim, bool lower_bounds, bool long_table);
constexpr int kWdTasks = 4, kWdCapGroups = 6144;  // (prefill_d256.h)
prefill_mfma_fn pa_prefill_d256_kernel(int dtype, bool lower_bounds, bool long_table);
}

using namespace pa_decode_detail;

namespace {

// Compute units of the current device (asked once per device).
int prefill_cus() {
    static int cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
    }
    return n;
}

// (the split rule, the workspace size and the groups a workgroup runs are host-testable arithmetic: prefill_plan.h)
int prefill_splits(int64_t workgroups, int cus, int64_t max_keys) {
    return plan_prefill_splits(workgroups, cus, max_keys, kPfKeys);
}
size_t prefill_ws_bytes(int64_t total_q, int num_q_heads, int head_dim, int splits) {
    return plan_prefill_ws_bytes(total_q, num_q_heads, head_dim, splits);
}

// Merge of the pieces of a split prefill launch: one thread per (row, head, four consecutive d).  The partial rows
// are d_part floats long (the head size the kernel is compiled for), the output rows d_head elements.
template <typename T>
__global__ __launch_bounds__(256) void prefill_merge_kernel(const float *part_o, const float *part_ml, T *out,
                                                            const int32_t *q_lens, const int32_t *q_starts, int hq,
                                                            int d_head, int d_part, int splits) {
    const int b = blockIdx.z, i = blockIdx.y;
    if (i >= q_lens[b]) return;
    const int item = blockIdx.x * 256 + threadIdx.x, v4 = d_head / 4;
    if (item >= hq * v4) return;
    const int h = item / v4, d = (item - h * v4) * 4;
    const int64_t row = (int64_t)q_starts[b] + i;
    const int64_t base = (row * hq + h) * splits;
    float m_all = -1.0e30f;
    for (int s = 0; s < splits; ++s)
        if (part_ml[(base + s) * 2 + 1] > 0.f) m_all = fmaxf(m_all, part_ml[(base + s) * 2]);
    float den = 0.f, num[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < splits; ++s) {
        const float l = part_ml[(base + s) * 2 + 1];
        if (!(l > 0.f)) continue;  // a piece in which the row saw no key wrote no O row
        const float w = __builtin_amdgcn_exp2f(part_ml[(base + s) * 2] - m_all);
        const float4 o = *reinterpret_cast<const float4 *>(part_o + (base + s) * d_part + d);
        den = fmaf(w, l, den);
        num[0] = fmaf(w, o.x, num[0]);
        num[1] = fmaf(w, o.y, num[1]);
        num[2] = fmaf(w, o.z, num[2]);
        num[3] = fmaf(w, o.w, num[3]);
    }
    const float inv = den > 0.f ? 1.f / den : 0.f;
    T *op = out + (row * hq + h) * d_head + d;
#pragma unroll
    for (int j = 0; j < 4; ++j) pa_scalar<T>::store(op + j, num[j] * inv);
}

int prefill_launch(bool force_rowwise, const void *q, const void *k_cache, const void *v_cache, void *out,
                   const int32_t *block_tables, int64_t bt_stride, const int32_t *ctx_lens, const int32_t *q_lens,
                   const int32_t *q_starts, const int32_t *row_first_key, int batch, int max_q_len, int num_q_heads,
                   int num_kv_heads, int head_dim, int block_size, int64_t num_blocks, float scale, int window,
                   int dtype, void *stream, int64_t total_q = 0, void *workspace = nullptr,
                   size_t workspace_bytes = 0) {
    pa_clear_error();
    PA_REQUIRE(batch >= 0 && max_q_len >= 0, "batch=%d max_q_len=%d must be non-negative", batch, max_q_len);
    PA_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && head_dim > 0, "head counts / head_dim must be positive");
    PA_REQUIRE(num_q_heads % num_kv_heads == 0, "num_q_heads=%d is not a multiple of num_kv_heads=%d",
               num_q_heads, num_kv_heads);
    PA_REQUIRE(block_size > 0, "block_size=%d must be positive", block_size);
    PA_REQUIRE(window >= 0, "window=%d is negative (0 = no sliding window)", window);
    PA_REQUIRE(num_blocks >= 0 && bt_stride >= 0, "num_blocks / bt_stride must be non-negative");
    PA_REQUIRE(num_blocks * (int64_t)block_size < (1ll << 40), "pool of %lld blocks is too large", (long long)num_blocks);
    PA_REQUIRE(dtype == PA_F32 || dtype == PA_BF16 || dtype == PA_F16, "dtype=%d is not F32, BF16 or F16", dtype);
    RowwiseArgs a;
    const int nrep_t = pa_fill_head_mapping(a.p, num_q_heads, num_kv_heads, head_dim, dtype);
    const KernelSet ks = nrep_t ? pa_pick_kernels(dtype, dtype, plan_pad_dim(head_dim), nrep_t) : KernelSet{};
    if (!ks.rowwise)
        return pa_fail(PA_ERR_UNSUPPORTED,
                       "pa_prefill_paged: no kernel for dtype=%d head_dim=%d (head_dim must be a multiple of 8 up to 256)",
                       dtype, head_dim);
    PA_REQUIRE(batch <= 65535 && max_q_len <= 65535, "batch=%d / max_q_len=%d above 65535", batch, max_q_len);
    if (batch == 0 || max_q_len == 0) return PA_OK;
    PA_REQUIRE(q && out && ctx_lens && q_lens && q_starts, "NULL q / out / ctx_lens / q_lens / q_starts");
    PA_REQUIRE(k_cache && v_cache, "NULL cache pointer");
    PA_REQUIRE(block_tables || bt_stride == 0, "NULL block_tables with bt_stride=%lld", (long long)bt_stride);
    PA_REQUIRE(pa_aligned16(k_cache) && pa_aligned16(v_cache), "cache pointers must be 16-byte aligned");

    a.p.k = k_cache; a.p.v = v_cache; a.p.bt = block_tables; a.p.bt_stride = bt_stride;
    a.p.k_scale = nullptr; a.p.v_scale = nullptr;
    a.p.bs = block_size; a.p.num_blocks = num_blocks;
    a.p.scale_log2 = scale * 1.4426950408889634f;
    a.p.window = window;
    a.q = q; a.out = out; a.ctx_lens = ctx_lens; a.q_lens = q_lens; a.q_starts = q_starts;
    a.row_lo = row_first_key;
    a.batch = batch; a.max_q_len = max_q_len;
    a.splits = 1; a.part_o = nullptr; a.part_ml = nullptr; a.groups_per_wg = 1;
    hipStream_t s = (hipStream_t)stream;
    // bf16 / fp16 with head_dim 32, 64, 128 (and 256, below) run on the matrix cores unless the caller asked for the
    // vector kernel
    // (the matrix-core softmax takes the running maximum of the unscaled logits, which needs scale > 0)
    prefill_mfma_fn mfma =
        force_rowwise || !(scale > 0.f) ? nullptr : pa_prefill_mfma_kernel(dtype, head_dim, block_size == 16);
    int split = 1;  // pieces per workgroup (the kernels with the assembly loop, given a workspace)
    // head_dim 128, 64 or 32, blocks of a multiple of 16 tokens (or one block per sequence, as dense prefill passes its
    // rows): the kernel whose whole tile loop is scheduled assembly (one instance without, one with sliding window /
    // per-row first keys).  Its LDS copy of the table holds pa_asm_cap_tiles() tiles from the workgroup's first tile
    // on, which bounds the table's length - or, under a sliding window, the stretch of keys that the rows of a
    // workgroup (at most kPfTasks blocks of kPfRows) see; longer tables take the instance that fills its copy again on
    // the way.
    // (a chunk's rows of q and out are addressed by 32-bit byte offsets from the sequence's first row)
    // Head sizes between the compiled ones (multiples of 8) run the next larger instance: rows in memory keep their
    // size, the chunks past a row's end are zero in Q^T and never stored.
    const int d_pad = plan_pad_dim(head_dim);
    const bool matrix_types = !force_rowwise && scale > 0.f && (dtype == PA_BF16 || dtype == PA_F16);
    if (matrix_types && head_dim % 8 == 0 && (d_pad == 128 || d_pad == 64 || d_pad == 32) &&
        (block_size % 16 == 0 || bt_stride == 1) &&
        num_blocks * (int64_t)block_size >= 16 && num_blocks * (int64_t)block_size < (1ll << 31) &&
        bt_stride * (int64_t)block_size < (1ll << 31) &&
        (int64_t)max_q_len * num_q_heads * head_dim * 2 < (1ll << 31)) {
        const int64_t cap_keys = (int64_t)pa_asm_cap_tiles(d_pad) * kPfKeys;
        const bool fits = bt_stride * (int64_t)block_size <= cap_keys ||
                          (window > 0 && (int64_t)window + kPfTasks * kPfRows + 3 * kPfKeys <= cap_keys);
        // With a workspace, a launch that cannot fill the chip has every workgroup's tiles cut into pieces (the
        // instance with lower bounds runs them: a piece is a later first tile and an earlier last key).
        if (workspace) {
            const int row_blocks = (max_q_len + kPfRows - 1) / kPfRows;
            const int64_t groups = (row_blocks * (int64_t)a.p.n_rep + kPfTasks - 1) / kPfTasks;
            int want = prefill_splits((int64_t)num_kv_heads * groups * batch, prefill_cus(),
                                      window > 0 ? (int64_t)window + kPfTasks * kPfRows : bt_stride * (int64_t)block_size);
            while (want > 1 && prefill_ws_bytes(total_q, num_q_heads, d_pad, want) > workspace_bytes) --want;
            split = want;
        }
        const bool lower_bounds = split > 1 || window > 0 || row_first_key != nullptr;
        mfma = pa_prefill_asm_kernel(dtype, d_pad, lower_bounds, !fits);
        if (!lower_bounds && fits) {
            // The plain instance runs several groups of one (sequence, kv head) per workgroup, which share the
            // set-up of lengths and slot tables: as many (up to 8) as leave a workgroup for every compute unit.
            const int row_blocks = (max_q_len + kPfRows - 1) / kPfRows;
            const int64_t groups = (row_blocks * (int64_t)a.p.n_rep + kPfTasks - 1) / kPfTasks;
            const int gpw = plan_groups_per_workgroup(num_kv_heads, groups, batch, prefill_cus());
            a.groups_per_wg = gpw;
        }
    }
    // head_dim 256: one 32-row task per wave, loads driven by a table of 16-key groups - which must lie inside one
    // pool block (block sizes that are multiples of 16, or a single block per sequence); the kernel fills its table
    // again whenever the context is longer than what LDS can hold of it
    int tasks_per_wg = kPfTasks;
    // (a pool of fewer than 16 rows has no slot a whole group could be loaded from: the vector kernel)
    if (matrix_types && head_dim % 8 == 0 && d_pad == 256 && (block_size % 16 == 0 || bt_stride == 1) &&
        num_blocks * (int64_t)block_size >= 16 && num_blocks * (int64_t)block_size < (1ll << 31) &&
        bt_stride * (int64_t)block_size < (1ll << 31)) {
        // (the tables hold kWdCapGroups groups of 16 keys from the workgroup's first tile on; under a sliding window
        // a workgroup's kWdTasks blocks of kPfRows rows, and the tiles its loads run ahead, bound what it needs)
        const bool fits = bt_stride * (int64_t)block_size <= (int64_t)kWdCapGroups * 16 ||
                          (window > 0 && (int64_t)window + kWdTasks * kPfRows + 10 * 32 <= (int64_t)kWdCapGroups * 16);
        if (workspace) {  // (as above; a workgroup of this kernel holds kWdTasks tasks)
            const int row_blocks = (max_q_len + kPfRows - 1) / kPfRows;
            const int64_t groups = (row_blocks * (int64_t)a.p.n_rep + kWdTasks - 1) / kWdTasks;
            int want = prefill_splits((int64_t)num_kv_heads * groups * batch, prefill_cus(),
                                      window > 0 ? (int64_t)window + kWdTasks * kPfRows : bt_stride * (int64_t)block_size);
            while (want > 1 && prefill_ws_bytes(total_q, num_q_heads, d_pad, want) > workspace_bytes) --want;
            split = want;
        }
        mfma = pa_prefill_d256_kernel(dtype, split > 1 || window > 0 || row_first_key != nullptr, !fits);
        tasks_per_wg = kWdTasks;
    }
    if (mfma) {
        PA_REQUIRE(pa_aligned16(q) && pa_aligned16(out), "q and out must be 16-byte aligned");
        const int row_blocks = (max_q_len + kPfRows - 1) / kPfRows;
        int groups = (row_blocks * a.p.n_rep + tasks_per_wg - 1) / tasks_per_wg;
        groups = (groups + a.groups_per_wg - 1) / a.groups_per_wg;  // workgroups along y: chunks of groups
        PA_REQUIRE((int64_t)groups * split <= 65535, "max_q_len=%d is too long for one launch", max_q_len);
        if (split > 1) {
            PA_REQUIRE(((uintptr_t)workspace & 255u) == 0, "workspace must be 256-byte aligned");
            a.splits = split;
            a.part_o = (float *)workspace;
            a.part_ml = a.part_o + (size_t)total_q * num_q_heads * split * d_pad;
        }
        mfma<<<dim3((unsigned)num_kv_heads, (unsigned)(groups * split), (unsigned)batch), dim3(kPfThreads), 0, s>>>(a);
        PA_CHECK_LAUNCH("pa_prefill_paged (matrix-core kernel)");
        if (split > 1) {
            const unsigned gx = (unsigned)((num_q_heads * (head_dim / 4) + 255) / 256);
            const dim3 mg(gx, (unsigned)max_q_len, (unsigned)batch);
            if (dtype == PA_BF16)
                prefill_merge_kernel<pa_bf16><<<mg, dim3(256), 0, s>>>(a.part_o, a.part_ml, (pa_bf16 *)out, q_lens, q_starts,
                                                                     num_q_heads, head_dim, d_pad, split);
            else
                prefill_merge_kernel<pa_f16><<<mg, dim3(256), 0, s>>>(a.part_o, a.part_ml, (pa_f16 *)out, q_lens, q_starts,
                                                                    num_q_heads, head_dim, d_pad, split);
            PA_CHECK_LAUNCH("pa_prefill_paged_ws (merge of the pieces)");
        }
        return PA_OK;
    }
    ks.rowwise<<<dim3((unsigned)(a.p.n_hgroups * a.p.n_rgroups), (unsigned)max_q_len, (unsigned)batch),
                 dim3(kThreads), 0, s>>>(a);
    PA_CHECK_LAUNCH("pa_prefill_paged");
    return PA_OK;
}

}  // namespace

#define PA_PREFILL_PARAMS                                                                                      \
    const void *q, const void *k_cache, const void *v_cache, void *out, const int32_t *block_tables,          \
        int64_t bt_stride, const int32_t *ctx_lens, const int32_t *q_lens, const int32_t *q_starts,            \
        const int32_t *row_first_key, int batch, int max_q_len, int num_q_heads, int num_kv_heads,             \
        int head_dim, int block_size, int64_t num_blocks, float scale, int window, int dtype, void *stream
#define PA_PREFILL_ARGS                                                                                        \
    q, k_cache, v_cache, out, block_tables, bt_stride, ctx_lens, q_lens, q_starts, row_first_key, batch,       \
        max_q_len, num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, scale, window, dtype, stream

extern "C" int pa_prefill_paged(PA_PREFILL_PARAMS) { return prefill_launch(false, PA_PREFILL_ARGS); }

extern "C" size_t pa_prefill_workspace_bytes(int batch, int max_q_len, int64_t total_q, int64_t bt_stride,
                                             int block_size, int window, int num_q_heads, int num_kv_heads,
                                             int head_dim, int dtype) {
    pa_clear_error();
    if (batch < 0 || max_q_len < 0 || total_q < 0 || bt_stride < 0 || block_size <= 0 || window < 0 ||
        num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads != 0 || head_dim <= 0) {
        pa_fail(PA_ERR_INVALID_ARG, "pa_prefill_workspace_bytes: negative size or inconsistent head counts");
        return 0;
    }
    // only the 16-bit kernels with the assembly loop split (head_dim a multiple of 8 up to 256; the partial rows have
    // the head size the kernel is compiled for); everything else needs none
    if ((dtype != PA_BF16 && dtype != PA_F16) || head_dim % 8 != 0 || head_dim > 256 || batch == 0 || max_q_len == 0)
        return 0;
    const int d_pad = plan_pad_dim(head_dim);
    const int n_rep = num_q_heads / num_kv_heads;
    const int row_blocks = (max_q_len + kPfRows - 1) / kPfRows;
    const int tasks = d_pad == 256 ? kWdTasks : kPfTasks;
    const int64_t groups = (row_blocks * (int64_t)n_rep + tasks - 1) / tasks;
    const int split = prefill_splits((int64_t)num_kv_heads * groups * batch, prefill_cus(),
                                     window > 0 ? (int64_t)window + tasks * kPfRows : bt_stride * (int64_t)block_size);
    return prefill_ws_bytes(total_q, num_q_heads, d_pad, split);
}

extern "C" int pa_prefill_paged_ws(PA_PREFILL_PARAMS, int64_t total_q, void *workspace, size_t workspace_bytes) {
    if (workspace && total_q <= 0) {
        pa_clear_error();
        return pa_fail(PA_ERR_INVALID_ARG, "pa_prefill_paged_ws: total_q=%lld must be positive with a workspace",
                       (long long)total_q);
    }
    return prefill_launch(false, PA_PREFILL_ARGS, total_q, workspace, workspace_bytes);
}
extern "C" int pa_prefill_paged_rowwise(PA_PREFILL_PARAMS) { return prefill_launch(true, PA_PREFILL_ARGS); }
