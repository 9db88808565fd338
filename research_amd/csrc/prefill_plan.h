// Bookkeeping of the matrix-core prefill launches: how many pieces a workgroup's tiles are cut into, which tiles a
// piece runs, how many groups of tasks a workgroup runs in turn and which ones, and the size of the workspace.
// Integer arithmetic only; shared by the host entry points (prefill.hip), the kernels (prefill_asm.h,
// prefill_d256.h) and a plain C++ replay that the CPU tests compile with g++ (no HIP needed).
#pragma once
#include <stddef.h>
#include <stdint.h>

#include "decode_plan.h"  // PA_PLAN_FN

namespace pa_decode_detail {

constexpr int kPlanMaxPrefillSplits = 8;
constexpr int kPlanMinTilesPerSplit = 24;  // a piece's set-up and write-out cost about six tiles of its loop
constexpr int kPlanPieceFixedTiles = 6;    // set-up and write-out of a workgroup, in tiles of its loop
constexpr int kPlanMaxGroupsPerWorkgroup = 8;

// What a launch costs with its workgroups' tiles cut into s pieces, in tile times: the launch takes rounds of
// `cus` workgroups, each lasting a piece's tiles plus its fixed cost.
PA_PLAN_FN int64_t plan_prefill_cost(int64_t workgroups, int cus, int64_t tiles, int s) {
    const int64_t rounds = (workgroups * s + cus - 1) / cus;
    return rounds * (tiles / s + kPlanPieceFixedTiles);
}

// Pieces to cut every workgroup's tiles into, from shapes alone.  The matrix-core kernels run one workgroup per
// compute unit, each owning 256 (head_dim 256: 128) row-head pairs and all their keys, so a launch of few rows
// leaves compute units idle however long the context is.  The split with the lowest cost wins (the smaller on
// ties), as long as a piece keeps kPlanMinTilesPerSplit tiles of the longest context the block tables can describe.
PA_PLAN_FN int plan_prefill_splits(int64_t workgroups, int cus, int64_t max_keys, int tile_keys) {
    const int64_t tiles = max_keys / tile_keys;
    int best = 1;
    int64_t best_cost = 0;
    for (int s = 1; s <= kPlanMaxPrefillSplits; ++s) {
        if (s > 1 && tiles / s < kPlanMinTilesPerSplit) break;
        const int64_t cost = plan_prefill_cost(workgroups, cus, tiles, s);
        if (s == 1 || cost < best_cost) {
            best_cost = cost;
            best = s;
        }
    }
    return best;
}

// workspace = [part_o float[row][head][piece][D]] [part_ml float[row][head][piece][2]]
PA_PLAN_FN size_t plan_prefill_ws_bytes(int64_t total_q, int num_q_heads, int head_dim, int splits) {
    return splits <= 1 ? 0 : (size_t)total_q * num_q_heads * splits * ((size_t)head_dim + 2) * sizeof(float);
}

// Piece `piece` of `n_splits` of the n_all tiles from tile t0 on runs the tiles [tb, te) (empty when there are
// fewer tiles than pieces): consecutive, disjoint, sizes that differ by one at most.
PA_PLAN_FN void plan_piece_tiles(int t0, int n_all, int piece, int n_splits, int &tb, int &te) {
    tb = t0 + (int)((int64_t)piece * n_all / n_splits);
    te = t0 + (int)((int64_t)(piece + 1) * n_all / n_splits);
}

// Groups (of 8 tasks) of one (sequence, kv head) that a workgroup of the plain assembly-loop instance runs in turn:
// they share the set-up of lengths and slot tables.  As many (up to 8) as leave a workgroup for every compute unit.
PA_PLAN_FN int plan_groups_per_workgroup(int num_kv_heads, int64_t groups, int batch, int cus) {
    int gpw = 1;
    for (int g = 2; g <= kPlanMaxGroupsPerWorkgroup && g <= groups; ++g)
        if ((int64_t)num_kv_heads * ((groups + g - 1) / g) * batch >= cus) gpw = g;
    return gpw;
}

// The i-th group of the workgroup that is chunk `wg_chunk` of `n_chunks`: one of every n_chunks consecutive groups,
// counted from the front in even rounds and from the back in odd ones, so that under the causal mask (later groups
// see more keys) the workgroups' totals come out equal.  Strictly increasing in i; a workgroup stops at its first
// group past the sequence's last.
PA_PLAN_FN int plan_group_of(int i, int n_chunks, int wg_chunk) {
    return i * n_chunks + ((i & 1) ? n_chunks - 1 - wg_chunk : wg_chunk);
}

}  // namespace pa_decode_detail
