// Replays, on the host and in plain C++, the index arithmetic of both passes of paged decode attention from
// research_amd/csrc/decode_plan.h (the header the kernels use): the split pass's walk over its range of
// (plane, sequence, block) units for every workgroup, the reduction pass's walk over the workgroups that hold
// pieces of a row, the partial-slot formula and the workspace layout.  Test infrastructure (compiled with g++ by
// tests/test_decode_plan.py); computes no attention.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <set>
#include <vector>

#include "../../research_amd/csrc/decode_plan.h"

using namespace pa_decode_detail;

#define FAIL(...)                               \
    do {                                        \
        snprintf(err, (size_t)errlen, __VA_ARGS__); \
        return 1;                               \
    } while (0)

// stats: [0] units, [1] workgroups taking part, [2] partial pieces, [3] rows finished in place, [4] largest slot,
//        [5] slot capacity, [6] most pieces of one (plane, sequence), [7] workspace bytes
extern "C" int pa_plan_replay(const int32_t *seq_lens, int batch, int num_q_heads, int num_kv_heads, int head_dim,
                              int kv_elem_bytes, int block_size, int window, int launch_grid, int grid_cap,
                              int64_t *stats, char *err, int errlen) {
    const HeadPlan h = plan_heads(num_q_heads, num_kv_heads, head_dim, kv_elem_bytes);
    if (!h.nrep_t) FAIL("no head plan");
    if (batch < 1 || batch > kPlanMaxBatch) FAIL("batch out of range");
    const WsPlan ws = plan_workspace(batch, h, head_dim, grid_cap);
    const int planes = h.planes();
    // ---- what every workgroup computes first: blocks before each sequence ----
    std::vector<int64_t> prefix(batch + 1, 0);
    for (int b = 0; b < batch; ++b) prefix[b + 1] = prefix[b] + plan_blocks_of(seq_lens[b], block_size, window);
    if (prefix[batch] > 0x7fffffffll) FAIL("block prefix sum leaves 32 bits");
    const int64_t per_plane = prefix[batch];
    const int64_t total = per_plane * planes;
    for (int i = 0; i < 8; ++i) stats[i] = 0;
    stats[0] = total;
    stats[5] = ws.slots;
    stats[7] = (int64_t)ws.total;
    if (plan_split_lds_bytes(batch, head_dim, kv_elem_bytes, h.nrep_t) > 65536) FAIL("workgroup LDS above 64 KB");
    // layout: regions in order, aligned, inside the total
    if (!(ws.ticket_off == 0 && ws.prefix_off >= kPlanTicketBytes && ws.ml_off >= ws.prefix_off + (size_t)(batch + 1) * 4 &&
          (!plan_merge_in_split(batch, h, launch_grid) || (size_t)planes * batch * 8 <= kPlanTicketBytes) &&
          ws.acc_off >= ws.ml_off + (size_t)ws.slots * h.heads_per_slot() * 8 &&
          ws.total >= ws.acc_off + (size_t)ws.slots * h.heads_per_slot() * head_dim * 4 && ws.prefix_off % 256 == 0 &&
          ws.ml_off % 256 == 0 && ws.acc_off % 256 == 0))
        FAIL("workspace regions overlap or are misaligned");
    if (total == 0) return 0;
    const int grid = plan_effective_grid(total, launch_grid);
    if (grid < 1 || grid > launch_grid) FAIL("effective grid %d outside [1, %d]", grid, launch_grid);
    stats[1] = grid;

    // ---- split pass ----
    std::vector<int> owner((size_t)total, -1);                 // workgroup that attended each unit
    std::set<int64_t> slots_written;                            // partial slots
    std::vector<std::vector<int>> pieces((size_t)planes * batch);  // workgroups that left a partial per (plane, sequence)
    std::vector<char> whole((size_t)planes * batch, 0);          // finished in place
    for (int w = 0; w < grid; ++w) {
        int64_t cur = plan_unit_begin(w, total, grid);
        const int64_t end = plan_unit_begin((int64_t)w + 1, total, grid);
        if (end - cur < 1) FAIL("workgroup %d of %d has no units (total %lld)", w, grid, (long long)total);
        while (cur < end) {
            const int plane = (int)(cur / per_plane);
            const int64_t off = cur - plane * per_plane;
            int lo = 0, hi = batch;  // the kernel's binary search: last b with prefix[b] <= off
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (prefix[mid] <= off) lo = mid; else hi = mid;
            }
            const int b = lo;
            const int64_t nblk = prefix[b + 1] - prefix[b];
            const int64_t blk0 = off - prefix[b];
            const int64_t blk1 = std::min(nblk, blk0 + (end - cur));
            if (nblk < 1 || blk0 < 0 || blk0 >= nblk || blk1 <= blk0)
                FAIL("workgroup %d: search landed on sequence %d (blocks %lld) with range [%lld, %lld)", w, b,
                     (long long)nblk, (long long)blk0, (long long)blk1);
            if (plane >= planes) FAIL("plane %d of %d", plane, planes);
            // the blocks it reads: first visible block + [blk0, blk1) must lie inside the sequence
            const int len = seq_lens[b];
            const int fb = plan_first_key(len, window) / block_size;
            if ((fb + blk1 - 1) * (int64_t)block_size >= len) FAIL("sequence %d: block %lld past its %d keys", b, (long long)(fb + blk1 - 1), len);
            for (int64_t u = cur; u < cur + (blk1 - blk0); ++u) {
                if (owner[(size_t)u] != -1) FAIL("unit %lld attended twice", (long long)u);
                owner[(size_t)u] = w;
                if (plan_owner_of(u, total, grid) != w) FAIL("owner_of(%lld) = %d, attended by %d", (long long)u, plan_owner_of(u, total, grid), w);
            }
            const size_t key = (size_t)plane * batch + b;
            if (blk0 == 0 && blk1 == nblk) {
                if (whole[key] || !pieces[key].empty()) FAIL("(plane %d, sequence %d) finished twice", plane, b);
                whole[key] = 1;
                ++stats[3];
            } else {
                const int64_t slot = plan_slot(w, plane, batch, b);
                if (slot < 0 || slot >= ws.slots) FAIL("slot %lld outside the workspace's %lld", (long long)slot, (long long)ws.slots);
                if (!slots_written.insert(slot).second) FAIL("slot %lld written twice", (long long)slot);
                if (whole[key]) FAIL("(plane %d, sequence %d) has pieces and was finished in place", plane, b);
                pieces[key].push_back(w);
                stats[4] = std::max(stats[4], slot);
                ++stats[2];
            }
            cur += blk1 - blk0;
        }
    }
    for (int64_t u = 0; u < total; ++u)
        if (owner[(size_t)u] == -1) FAIL("unit %lld attended by nobody", (long long)u);

    // ---- reduction pass (and the tickets of the merge inside the split pass): per output row ----
    for (int b = 0; b < batch; ++b)
        for (int qh = 0; qh < num_q_heads; ++qh) {
            const int kv = qh / h.n_rep, rep = qh - kv * h.n_rep;
            const int hg = kv / h.hpw, rg = rep / h.nrep_t;
            const int plane = rg * h.n_hgroups + hg;
            const int idx = (kv - hg * h.hpw) * h.nrep_t + (rep - rg * h.nrep_t);
            if (plane >= planes || idx < 0 || idx >= h.heads_per_slot()) FAIL("query head %d maps to plane %d, index %d", qh, plane, idx);
            const int64_t nblk = prefix[b + 1] - prefix[b];
            const size_t key = (size_t)plane * batch + b;
            if (nblk == 0) {
                if (whole[key] || !pieces[key].empty()) FAIL("empty sequence %d has results", b);
                continue;
            }
            const int64_t u0 = plane * per_plane + prefix[b];
            const int w0 = plan_owner_of(u0, total, grid), w1 = plan_owner_of(u0 + nblk - 1, total, grid);
            if (w0 == w1) {
                if (!whole[key]) FAIL("(plane %d, sequence %d): one owner but not finished in place", plane, b);
                continue;
            }
            if (whole[key]) FAIL("(plane %d, sequence %d): owners %d..%d but finished in place", plane, b, w0, w1);
            if ((int)pieces[key].size() != w1 - w0 + 1) FAIL("(plane %d, sequence %d): %d pieces written, %d expected", plane, b, (int)pieces[key].size(), w1 - w0 + 1);
            for (int w = w0; w <= w1; ++w) {
                if (pieces[key][(size_t)(w - w0)] != w) FAIL("(plane %d, sequence %d): piece of workgroup %d missing", plane, b, w);
                if (!slots_written.count(plan_slot(w, plane, batch, b))) FAIL("slot of workgroup %d not written", w);
            }
            stats[6] = std::max<int64_t>(stats[6], w1 - w0 + 1);
        }
    return 0;
}
