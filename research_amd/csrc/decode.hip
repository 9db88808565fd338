// Host entry points of paged decode attention: argument checks, split-K
// planning arithmetic, workspace layout and the two launches.  The kernels are
// in decode_impl.h and are instantiated per pool element type in
// decode_inst_*.hip.
#include <stdlib.h>

#include <mutex>

#include "decode_impl.h"

// Scratch of pa_decode_static: device memory the library itself holds (one copy per GPU, for the life of the
// process) so that callers which cannot allocate - code under HIP graph capture, serving loops with a fixed
// memory plan - still get the split pass's partial results somewhere.  In host code this name is only a handle
// for hipGetSymbolAddress; kernels receive the address that call returns.
constexpr size_t kStaticScratchBytes = (size_t)PA_DECODE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace pa_decode_detail {

KernelSet pa_pick_kernels(int q_dtype, int kv_dtype, int d, int nrep_t) {
    if (kv_dtype == PA_FP8_E4M3) return pa_kernels_fp8(q_dtype, d, nrep_t);
    if (q_dtype != kv_dtype) return KernelSet{};
    if (q_dtype == PA_BF16) return pa_kernels_bf16(d, nrep_t);
    if (q_dtype == PA_F16) return pa_kernels_f16(d, nrep_t);
    if (q_dtype == PA_F32) return pa_kernels_f32(d, nrep_t);
    return KernelSet{};
}

int pa_fill_head_mapping(PoolArgs &p, int num_q_heads, int num_kv_heads, int head_dim, int kv_dtype) {
    const HeadPlan h = plan_heads(num_q_heads, num_kv_heads, head_dim, pa_dtype_bytes(kv_dtype));
    if (!h.nrep_t) return 0;
    p.d = head_dim;
    p.hq = h.hq;
    p.hkv = h.hkv;
    p.n_rep = h.n_rep;
    p.hpw = h.hpw;
    p.tpw = h.tpw;
    p.n_hgroups = h.n_hgroups;
    p.n_rgroups = h.n_rgroups;
    return h.nrep_t;
}

}  // namespace pa_decode_detail

using namespace pa_decode_detail;

namespace {

static_assert(PA_DECODE_TICKET_BYTES == kPlanTicketBytes, "paged_attn.h and decode_plan.h disagree on the ticket region");
constexpr int kMaxSplitGrid = kPlanMaxSplitGrid;  // upper bound of the split pass's grid, fixes the workspace size

constexpr int kMaxDevices = 64;

// Compute units of the current device (asked once per device).
int num_cus() {
    static int cached[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    int n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
    }
    return n;
}

// Workgroups of the split pass per compute unit: two workgroups of four waves keep two waves on every SIMD,
// each with the loads of eight token steps in flight.
constexpr int kSplitWgsPerCu = 2;

int split_grid() {
    const int grid = num_cus() * kSplitWgsPerCu;
    return grid > kMaxSplitGrid ? kMaxSplitGrid : grid;
}

// Address of `scratch` on the current device.  Every GPU holds its own copy of the array at its own address,
// so the address is asked for once per device, with that device current, and kept.
int static_scratch(void **ptr) {
    static void *addr[kMaxDevices];
    static std::mutex mu;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return pa_fail(PA_ERR_HIP, "pa_decode_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices)
        return pa_fail(PA_ERR_UNSUPPORTED, "pa_decode_static: device index %d above %d", dev, kMaxDevices - 1);
    std::lock_guard<std::mutex> lock(mu);
    if (!addr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return pa_fail(PA_ERR_HIP, "pa_decode_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        addr[dev] = p;
    }
    *ptr = addr[dev];
    return PA_OK;
}

enum { kPhaseSplit = 1, kPhaseReduce = 2 };

int decode_launch(int phases, const void *q, const void *k_cache, const void *v_cache, void *out,
                  const int32_t *block_tables, int64_t bt_stride, const int32_t *seq_lens,
                  const int32_t *extra_zero_keys, const float *k_scale, const float *v_scale, int batch,
                  int num_q_heads, int num_kv_heads, int head_dim, int block_size, int64_t num_blocks, float scale,
                  int window, int q_dtype, int kv_dtype, void *workspace, size_t workspace_bytes, void *stream,
                  bool use_static = false) {
    pa_clear_error();
    PA_REQUIRE(batch >= 0, "batch=%d is negative", batch);
    PA_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && head_dim > 0, "head counts / head_dim must be positive");
    PA_REQUIRE(num_q_heads % num_kv_heads == 0, "num_q_heads=%d is not a multiple of num_kv_heads=%d",
               num_q_heads, num_kv_heads);
    PA_REQUIRE(block_size > 0, "block_size=%d must be positive", block_size);
    PA_REQUIRE(window >= 0, "window=%d is negative (0 = no sliding window)", window);
    PA_REQUIRE(window == 0 || !extra_zero_keys, "a sliding window cannot be combined with extra_zero_keys");
    PA_REQUIRE(num_blocks >= 0 && bt_stride >= 0, "num_blocks / bt_stride must be non-negative");
    PA_REQUIRE(num_blocks * (int64_t)block_size < (1ll << 40), "pool of %lld blocks is too large", (long long)num_blocks);
    PA_REQUIRE((int64_t)block_size * num_kv_heads * head_dim * 4 < (1ll << 31),
               "one block of %d tokens x %d heads x %d is too large", block_size, num_kv_heads, head_dim);
    DecodeArgs a;
    const int nrep_t = pa_fill_head_mapping(a.p, num_q_heads, num_kv_heads, head_dim, kv_dtype);
    const int d_pad = plan_pad_dim(head_dim);  // the head size the kernels are compiled for
    const KernelSet ks = nrep_t ? pa_pick_kernels(q_dtype, kv_dtype, d_pad, nrep_t) : KernelSet{};
    if (!ks.split)
        return pa_fail(PA_ERR_UNSUPPORTED,
                       "pa_decode: no kernel for q_dtype=%d kv_dtype=%d head_dim=%d (head_dim must be a multiple of 8, "
                       "of 16 for an fp8 pool, up to 256)", q_dtype, kv_dtype, head_dim);
    if (batch == 0) return PA_OK;
    PA_REQUIRE(q && out && seq_lens, "NULL q / out / seq_lens");
    PA_REQUIRE(k_cache && v_cache, "NULL cache pointer");
    PA_REQUIRE(block_tables || bt_stride == 0, "NULL block_tables with bt_stride=%lld", (long long)bt_stride);
    PA_REQUIRE(kv_dtype != PA_FP8_E4M3 || (k_scale && v_scale), "fp8 KV needs k_scale and v_scale");
    PA_REQUIRE(pa_aligned16(k_cache) && pa_aligned16(v_cache) && pa_aligned16(q),
               "q and cache pointers must be 16-byte aligned");
    PA_REQUIRE(head_dim * pa_dtype_bytes(q_dtype) % 16 == 0, "head_dim=%d: rows of q must be whole 16-byte vectors", head_dim);
    if (batch > kMaxBatch) {
        // The block prefix sums of a launch live in LDS: a larger batch is taken kMaxBatch sequences at a time, one
        // after the other on the stream, all through the same workspace (sized for kMaxBatch sequences).
        const size_t q_row = (size_t)num_q_heads * head_dim * pa_dtype_bytes(q_dtype);
        for (int at = 0; at < batch; at += kMaxBatch) {
            const int rc = decode_launch(
                phases, (const char *)q + at * q_row, k_cache, v_cache, (char *)out + at * q_row,
                block_tables ? block_tables + (int64_t)at * bt_stride : nullptr, bt_stride, seq_lens + at,
                extra_zero_keys ? extra_zero_keys + at : nullptr, k_scale, v_scale,
                batch - at < kMaxBatch ? batch - at : kMaxBatch, num_q_heads, num_kv_heads, head_dim, block_size,
                num_blocks, scale, window, q_dtype, kv_dtype, workspace, workspace_bytes, stream, use_static);
            if (rc != PA_OK) return rc;
        }
        return PA_OK;
    }
    PA_REQUIRE(plan_split_lds_bytes(batch, d_pad, pa_dtype_bytes(kv_dtype), nrep_t) <= 65536,
               "batch=%d needs more than 64 KB of LDS per workgroup", batch);
    const int grid = split_grid();
    // A caller's workspace is sized without asking the device (kMaxSplitGrid workgroups); the library's own
    // scratch is laid out for the grid this device really gets, which is what makes its fixed size go far.
    const HeadPlan plan = plan_heads(num_q_heads, num_kv_heads, head_dim, pa_dtype_bytes(kv_dtype));
    const WsPlan w = plan_workspace(batch, plan, d_pad, use_static ? grid : kMaxSplitGrid);
    if (use_static) {
        if (w.total > kStaticScratchBytes)
            return pa_fail(PA_ERR_WORKSPACE,
                           "pa_decode_static: these shapes need %zu bytes of scratch, the library holds %zu: use "
                           "pa_decode with a workspace of pa_decode_workspace_bytes()",
                           w.total, kStaticScratchBytes);
        const int rc = static_scratch(&workspace);
        if (rc != PA_OK) return rc;
    } else {
        if (!workspace || workspace_bytes < w.total)
            return pa_fail(PA_ERR_WORKSPACE, "pa_decode: workspace of %zu bytes, need %zu", workspace_bytes, w.total);
        PA_REQUIRE(((uintptr_t)workspace & 255u) == 0, "workspace must be 256-byte aligned");
    }

    a.p.k = k_cache; a.p.v = v_cache; a.p.bt = block_tables; a.p.bt_stride = bt_stride;
    a.p.k_scale = k_scale; a.p.v_scale = v_scale;
    a.p.bs = block_size; a.p.num_blocks = num_blocks;
    a.p.scale_log2 = scale * 1.4426950408889634f;
    a.p.window = window;
    a.q = q; a.out = out; a.seq_lens = seq_lens; a.extra_zero = extra_zero_keys;
    a.batch = batch;
    a.slot_cap = w.slots;
    char *ws = (char *)workspace;
    a.block_prefix = (int32_t *)(ws + w.prefix_off);
    a.tickets = (unsigned long long *)(ws + w.ticket_off);
    a.part_ml = (float *)(ws + w.ml_off);
    a.part_acc = (float *)(ws + w.acc_off);
    // Batches that leave a sequence few pieces are finished by the split pass alone.
    a.group_tickets = (unsigned long long *)(ws + kPlanGroupTicketOff);
    a.merge_in_split = phases == (kPhaseSplit | kPhaseReduce) && plan_merge_in_split(batch, plan, grid) ? 1 : 0;

    hipStream_t s = (hipStream_t)stream;
    a.split_grid = grid;
    if (phases & kPhaseSplit) {
        ks.split<<<dim3((unsigned)grid), dim3(kThreads), (size_t)(batch + 1) * sizeof(int), s>>>(a);
        PA_CHECK_LAUNCH("pa_decode split pass");
    }
    if ((phases & kPhaseReduce) && !a.merge_in_split) {
        // Many rows and therefore few pieces per sequence: one wave per row.
        const int64_t rows = (int64_t)batch * num_q_heads;
        if (rows >= 2 * (int64_t)grid)
            ks.reduce_wave<<<dim3((unsigned)((rows + kWaves - 1) / kWaves)), dim3(kThreads), 0, s>>>(a);
        else
            ks.reduce<<<dim3((unsigned)rows), dim3(kThreads), 0, s>>>(a);
        PA_CHECK_LAUNCH("pa_decode reduction pass");
    }
    return PA_OK;
}

}  // namespace

extern "C" size_t pa_decode_workspace_bytes(int batch, int num_q_heads, int num_kv_heads, int head_dim,
                                            int kv_dtype) {
    pa_clear_error();
    PoolArgs p;
    if (batch < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads != 0) {
        pa_fail(PA_ERR_INVALID_ARG, "pa_decode_workspace_bytes: negative batch or inconsistent head counts");
        return 0;
    }
    const int nrep_t = pa_fill_head_mapping(p, num_q_heads, num_kv_heads, head_dim, kv_dtype);
    if (!nrep_t) {
        pa_fail(PA_ERR_UNSUPPORTED, "pa_decode_workspace_bytes: no kernel for kv_dtype=%d head_dim=%d", kv_dtype,
                head_dim);
        return 0;
    }
    const HeadPlan plan = plan_heads(num_q_heads, num_kv_heads, head_dim, pa_dtype_bytes(kv_dtype));
    return plan_workspace(batch < kMaxBatch ? batch : kMaxBatch, plan, plan.d_pad, kMaxSplitGrid).total;
}

extern "C" int pa_decode_passes(int batch, int num_q_heads, int num_kv_heads, int head_dim, int kv_dtype) {
    pa_clear_error();
    const HeadPlan plan = plan_heads(num_q_heads, num_kv_heads, head_dim, pa_dtype_bytes(kv_dtype));
    if (batch < 0 || !plan.nrep_t) return pa_fail(PA_ERR_UNSUPPORTED, "pa_decode_passes: no kernel for these shapes");
    if (batch > kMaxBatch) batch = kMaxBatch;  // launches per group of kMaxBatch sequences
    return plan_merge_in_split(batch, plan, split_grid()) ? 1 : 2;
}

#define PA_DECODE_PARAMS                                                                                       \
    const void *q, const void *k_cache, const void *v_cache, void *out, const int32_t *block_tables,          \
        int64_t bt_stride, const int32_t *seq_lens, const int32_t *extra_zero_keys, const float *k_scale,      \
        const float *v_scale, int batch, int num_q_heads, int num_kv_heads, int head_dim, int block_size,      \
        int64_t num_blocks, float scale, int window, int q_dtype, int kv_dtype, void *workspace,                \
        size_t workspace_bytes, void *stream
#define PA_DECODE_ARGS                                                                                         \
    q, k_cache, v_cache, out, block_tables, bt_stride, seq_lens, extra_zero_keys, k_scale, v_scale, batch,     \
        num_q_heads, num_kv_heads, head_dim, block_size, num_blocks, scale, window, q_dtype, kv_dtype,         \
        workspace, workspace_bytes, stream

extern "C" int pa_decode(PA_DECODE_PARAMS) { return decode_launch(kPhaseSplit | kPhaseReduce, PA_DECODE_ARGS); }
extern "C" int pa_decode_split(PA_DECODE_PARAMS) { return decode_launch(kPhaseSplit, PA_DECODE_ARGS); }
extern "C" int pa_decode_reduce(PA_DECODE_PARAMS) { return decode_launch(kPhaseReduce, PA_DECODE_ARGS); }

extern "C" int pa_decode_static(const void *q, const void *k_cache, const void *v_cache, void *out,
                                const int32_t *block_tables, int64_t bt_stride, const int32_t *seq_lens,
                                const int32_t *extra_zero_keys, const float *k_scale, const float *v_scale, int batch,
                                int num_q_heads, int num_kv_heads, int head_dim, int block_size, int64_t num_blocks,
                                float scale, int window, int q_dtype, int kv_dtype, void *stream) {
    return decode_launch(kPhaseSplit | kPhaseReduce, q, k_cache, v_cache, out, block_tables, bt_stride, seq_lens,
                         extra_zero_keys, k_scale, v_scale, batch, num_q_heads, num_kv_heads, head_dim, block_size,
                         num_blocks, scale, window, q_dtype, kv_dtype, nullptr, 0, stream, true);
}
