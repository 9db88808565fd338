// Bookkeeping of the split pass of paged decode attention: how the (plane, sequence, block) space is cut into
// workgroup ranges, which workgroup owns a block, where a range's partial result goes in the workspace and how
// the workspace is laid out.  Integer arithmetic only; shared by the kernels (decode_impl.h), the host entry
// point (decode.hip) and a plain C++ replay of both passes that the CPU tests compile with g++ (no HIP needed).
#pragma once
#include <stddef.h>
#include <stdint.h>

#if defined(__HIPCC__)
#define PA_PLAN_FN __host__ __device__ inline __attribute__((always_inline))
#else
#define PA_PLAN_FN inline
#endif

namespace pa_decode_detail {

constexpr int kPlanMaxBatch = 8192;      // sequences per call (their block prefix sum lives in LDS)
constexpr int kPlanMaxSplitGrid = 4096;  // upper bound of the split pass's grid, fixes the caller's workspace size
constexpr int kPlanMinUnitsPerWorkgroup = 4;
// Arrival tickets of the merge inside the split pass: 64-bit counters in a region of fixed size at the start of
// every workspace, so that calls of any shape use the same bytes for the same purpose and nothing else is ever
// written there: kPlanTicketSlots counters per (plane, sequence), then 2 per workgroup of the largest grid for the
// groups that the pieces of a many-piece sequence are merged in.  The caller zero-fills the region once; every call
// leaves it at zero.
constexpr int kPlanTicketSlots = 65536;
constexpr size_t kPlanGroupTicketOff = (size_t)kPlanTicketSlots * 8;
constexpr size_t kPlanTicketBytes = kPlanGroupTicketOff + 2 * (size_t)kPlanMaxSplitGrid * 8 + 64 * 1024;  // 640 KiB

// How the heads are spread over wave loads and planes (a plane = one group of hpw kv heads x one group of <= nrep_t
// query heads per kv head).  lpr lanes of 16 bytes hold one K/V row; a wave load covers rpw = 64/lpr rows, mapped
// to hpw neighbouring kv heads of tpw consecutive tokens.
struct HeadPlan {
    int hq, hkv, n_rep;
    int hpw, tpw, n_hgroups, n_rgroups;
    int nrep_t;  // padded group size (kernel template parameter); 0 = no kernel for this head_dim / element size
    int d_pad;   // head_dim rounded up to the next of 32, 64, 128, 256: the head size the kernel is compiled for
    PA_PLAN_FN int planes() const { return n_hgroups * n_rgroups; }
    PA_PLAN_FN int heads_per_slot() const { return hpw * nrep_t; }
};

// The kernels are compiled for head sizes 32, 64, 128 and 256; any other head_dim up to 256 whose rows are whole
// 16-byte vectors runs the next larger one with the lanes past the row's end idle.
PA_PLAN_FN int plan_pad_dim(int head_dim) { return head_dim <= 32 ? 32 : head_dim <= 64 ? 64 : head_dim <= 128 ? 128 : 256; }

PA_PLAN_FN HeadPlan plan_heads(int num_q_heads, int num_kv_heads, int head_dim_real, int kv_elem_bytes) {
    HeadPlan h = {};
    if (kv_elem_bytes <= 0 || head_dim_real <= 0 || head_dim_real > 256 || head_dim_real * kv_elem_bytes % 16 != 0 ||
        head_dim_real % 8 != 0)
        return h;
    if (num_q_heads <= 0 || num_kv_heads <= 0 || num_q_heads % num_kv_heads != 0) return h;
    const int head_dim = plan_pad_dim(head_dim_real);
    h.d_pad = head_dim;
    const int lpr = head_dim * kv_elem_bytes / 16;  // lanes per K/V row
    const int rpw = 64 / lpr;                        // rows per wave load
    int hpw = 1;                                     // kv heads per wave load: power of two dividing num_kv_heads
    while (hpw * 2 <= rpw && num_kv_heads % (hpw * 2) == 0) hpw *= 2;
    const int n_rep = num_q_heads / num_kv_heads;
    int nrep_t = 1;
    while (nrep_t < n_rep && nrep_t < 8) nrep_t *= 2;
    h.hq = num_q_heads;
    h.hkv = num_kv_heads;
    h.n_rep = n_rep;
    h.hpw = hpw;
    h.tpw = rpw / hpw;
    h.n_hgroups = num_kv_heads / hpw;
    h.n_rgroups = (n_rep + nrep_t - 1) / nrep_t;
    h.nrep_t = nrep_t;
    return h;
}

// Blocks of a sequence of `len` keys that hold visible keys under a sliding window (0 = none): the query sits at
// position len-1 and sees keys j >= len - window, so blocks [first_key / bs, ceil(len / bs)) take part.
PA_PLAN_FN int plan_first_key(int len, int window) { return window > 0 && len > window ? len - window : 0; }
PA_PLAN_FN int plan_blocks_of(int len, int block_size, int window) {
    if (len <= 0) return 0;
    return (len + block_size - 1) / block_size - plan_first_key(len, window) / block_size;
}

// Workgroup w of a grid of G owns the flattened units [floor(w*T/G), floor((w+1)*T/G)) of T.
PA_PLAN_FN int64_t plan_unit_begin(int64_t w, int64_t total, int64_t grid) { return w * total / grid; }
PA_PLAN_FN int plan_owner_of(int64_t u, int64_t total, int64_t grid) { return (int)(((u + 1) * grid - 1) / total); }

// Workgroups that take part: with little work a workgroup per pool block would leave hundreds of one-block
// partials, so a workgroup gets at least kPlanMinUnitsPerWorkgroup units and the rest of the grid leaves at once.
PA_PLAN_FN int plan_effective_grid(int64_t total, int grid) {
    const int64_t g = total / kPlanMinUnitsPerWorkgroup;
    return g < 1 ? 1 : (g < grid ? (int)g : grid);
}

// Partial slot of the piece of (plane, sequence) that workgroup w computed: unique, because along the flattened
// order both w and plane*batch + sequence only grow.
PA_PLAN_FN int64_t plan_slot(int w, int plane, int batch, int b) { return (int64_t)w + (int64_t)plane * batch + b; }

// workspace = [tickets uint64[kPlanTicketSlots]] [block_prefix int32[batch+1]] [part_ml float[slots][heads][2]]
//             [part_acc float[slots][heads][D]], heads = hpw*nrep_t query heads of one plane,
// slots = grid_cap + planes*batch (slot indices stay below grid + planes*batch - 1).
struct WsPlan {
    size_t prefix_off, ticket_off, ml_off, acc_off, total;
    int64_t slots;
};
PA_PLAN_FN size_t plan_align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
PA_PLAN_FN WsPlan plan_workspace(int batch, const HeadPlan &h, int head_dim, int grid_cap) {
    WsPlan w;
    const size_t heads = (size_t)h.heads_per_slot();
    const size_t keys = (size_t)h.planes() * (size_t)batch;
    w.slots = (int64_t)grid_cap + (int64_t)keys;
    w.ticket_off = 0;
    w.prefix_off = kPlanTicketBytes;
    w.ml_off = w.prefix_off + plan_align_up((size_t)(batch + 1) * 4, 256);
    w.acc_off = w.ml_off + plan_align_up((size_t)w.slots * heads * 2 * 4, 256);
    w.total = w.acc_off + plan_align_up((size_t)w.slots * heads * (size_t)head_dim * 4, 256);
    return w;
}

// LDS of the merge of a workgroup's row-group partials (decode_impl.h: merge_rows): rows = 4 waves x rows per wave
// load, each D + 2 floats plus 3 floats of weights; as many query heads per round (8, 4, 2 or 1 of the nrep_t) as
// 28 KB hold.
constexpr int kPlanThreads = 256;
constexpr int kPlanMergeBudget = 28 * 1024;
PA_PLAN_FN constexpr int plan_merge_rows(int head_dim, int kv_elem_bytes) { return 4 * (64 / (head_dim * kv_elem_bytes / 16)); }
PA_PLAN_FN constexpr int plan_merge_heads_per_round(int head_dim, int kv_elem_bytes, int nrep_t) {
    const int per_head = plan_merge_rows(head_dim, kv_elem_bytes) * (head_dim + 2 + 3) * 4;
    return nrep_t >= 8 && 8 * per_head <= kPlanMergeBudget   ? 8
           : nrep_t >= 4 && 4 * per_head <= kPlanMergeBudget ? 4
           : nrep_t >= 2 && 2 * per_head <= kPlanMergeBudget ? 2
                                                             : 1;
}
PA_PLAN_FN constexpr int plan_merge_floats(int head_dim, int kv_elem_bytes, int nrep_t) {
    return plan_merge_heads_per_round(head_dim, kv_elem_bytes, nrep_t) * plan_merge_rows(head_dim, kv_elem_bytes) *
           (head_dim + 2 + 3);
}
// LDS of one workgroup of the split pass: the block prefix sums (dynamic), the scan scratch, the merge area, a flag.
PA_PLAN_FN constexpr size_t plan_split_lds_bytes(int batch, int head_dim, int kv_elem_bytes, int nrep_t) {
    return (size_t)(batch + 1) * 4 + kPlanThreads * 4 + (size_t)plan_merge_floats(head_dim, kv_elem_bytes, nrep_t) * 4 + 4;
}

// Whether the split pass merges the pieces of a sequence itself (the workgroup that delivers the last outstanding
// piece of a sequence, or of a group of its pieces, merges) instead of leaving them to a second launch: when the
// batch is so large that a (plane, sequence) has two pieces on average at most.  Measured on MI355X: 256 sequences
// (two pieces each) gain 1 % over the two launches; 64 sequences (four pieces each) lose 2 % - delivering a piece
// costs round trips to the memory side, about 9 us at the end of a 100 us launch where the second launch costs 7 -
// and a few long sequences spread over the whole grid are merged much faster by the second launch, whose
// workgroups take one output row each.
PA_PLAN_FN bool plan_merge_in_split(int batch, const HeadPlan &h, int grid) {
    const int64_t keys = (int64_t)h.planes() * batch;  // one ticket each
    return (int64_t)grid <= 2 * keys && keys <= kPlanTicketSlots;
}

}  // namespace pa_decode_detail
