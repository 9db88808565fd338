// Replays, on the host and in plain C++, the bookkeeping of the matrix-core prefill launches from
// research_amd/csrc/prefill_plan.h (the header the host entry points and the kernels use): the pieces a
// workgroup's tiles are cut into, the groups a workgroup runs in turn, the split rule and the workspace size.
// Test infrastructure (compiled with g++ by tests/test_prefill_plan.py); computes no attention.
#include <cstdio>
#include <vector>

#include "../../research_amd/csrc/prefill_plan.h"

using namespace pa_decode_detail;

#define FAIL(...)                                   \
    do {                                            \
        snprintf(err, (size_t)errlen, __VA_ARGS__); \
        return 1;                                   \
    } while (0)

// The pieces of the n_all tiles from t0 on: consecutive, disjoint, covering, sizes within one of each other.
extern "C" int pa_plan_pieces(int t0, int n_all, int n_splits, char *err, int errlen) {
    int at = t0, smallest = 1 << 30, largest = 0;
    for (int piece = 0; piece < n_splits; ++piece) {
        int tb, te;
        plan_piece_tiles(t0, n_all, piece, n_splits, tb, te);
        if (tb != at) FAIL("piece %d of %d starts at tile %d, the piece before it ended at %d", piece, n_splits, tb, at);
        if (te < tb) FAIL("piece %d of %d ends before it starts", piece, n_splits);
        smallest = te - tb < smallest ? te - tb : smallest;
        largest = te - tb > largest ? te - tb : largest;
        at = te;
    }
    if (at != t0 + n_all) FAIL("the pieces end at tile %d, the tiles at %d", at, t0 + n_all);
    if (largest - smallest > 1) FAIL("pieces of %d and %d tiles", smallest, largest);
    return 0;
}

// The walk of every workgroup (chunk) of one (sequence, kv head) over its groups, as the kernel does it: every group
// below group_end is run by exactly one chunk, a chunk's groups grow, and no chunk runs more than `limit` of them.
// Returns the largest number of groups of a chunk through *most.
extern "C" int pa_plan_groups(int group_end, int n_chunks, int limit, int *most, char *err, int errlen) {
    std::vector<int> owner(group_end, -1);
    *most = 0;
    for (int c = 0; c < n_chunks; ++c) {
        if (plan_group_of(0, n_chunks, c) != c) FAIL("chunk %d does not start with group %d", c, c);
        if (c >= group_end) continue;  // (the kernel's workgroup leaves at once)
        int ran = 0, last = -1;
        for (int i = 0;; ++i) {
            const int g = plan_group_of(i, n_chunks, c);
            if (g >= group_end) break;
            if (g <= last) FAIL("chunk %d: group %d after group %d", c, g, last);
            if (owner[g] >= 0) FAIL("group %d is run by chunks %d and %d", g, owner[g], c);
            owner[g] = c;
            last = g;
            ++ran;
        }
        if (ran > limit) FAIL("chunk %d runs %d groups, the launch was sized for %d", c, ran, limit);
        *most = ran > *most ? ran : *most;
    }
    for (int g = 0; g < group_end; ++g)
        if (owner[g] < 0) FAIL("group %d of %d is run by nobody (%d chunks)", g, group_end, n_chunks);
    return 0;
}

extern "C" int pa_plan_splits(long long workgroups, int cus, long long max_keys, int tile_keys) {
    return plan_prefill_splits(workgroups, cus, max_keys, tile_keys);
}
extern "C" long long pa_plan_cost(long long workgroups, int cus, long long tiles, int s) {
    return plan_prefill_cost(workgroups, cus, tiles, s);
}
extern "C" unsigned long long pa_plan_ws_bytes(long long total_q, int num_q_heads, int head_dim, int splits) {
    return plan_prefill_ws_bytes(total_q, num_q_heads, head_dim, splits);
}
extern "C" int pa_plan_groups_per_workgroup(int num_kv_heads, long long groups, int batch, int cus) {
    return plan_groups_per_workgroup(num_kv_heads, groups, batch, cus);
}
