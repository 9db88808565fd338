// Causal prefill attention over a paged context for head_dim 128, 64 and 32 (bf16 / fp16) with the whole tile loop in
// scheduled assembly (prefill_mfma_loop.inc, written by gen_prefill_loop.py).
//
// Same computation, work split, LDS ring and operand layouts as prefill_mfma_kernel (prefill_mfma.h); what
// differs is what surrounds the loop:
//   * the pool slots of the context's 16-key groups are looked up once per workgroup and kept in LDS behind the
//     ring (table A: slot of the group's first key; table B: first row of the group that does not exist, 16 =
//     none), so a tile's loads are a table read, a scalar multiply per group and one direct load per group and
//     tensor (head_dim 128: eight per wave and tile, head_dim 64: four, head_dim 32: two), for any block size that is a multiple
//     of 16;
//   * rows past the context end and absent blocks are loaded from a slot that exists (the group's own block,
//     or slot 0) and cleared in LDS before the tile is published; a zero key takes part with logit 0 and a
//     zero value row, which is what the other kernels do for absent blocks;
//   * every wave runs every tile of the workgroup with the causal / context-end mask applied where needed, so
//     there is no per-wave tail code: a wave past its last key multiplies exact zeros;
//   * sliding windows and per-row first keys have an instance of their own (LO): the out-of-line mask block also
//     applies the lower bound, a row that has seen no key yet takes its first maximum as reference, and the
//     workgroup starts at the tile of the first key its first row sees;
//   * block sizes that are not multiples of 16 are taken with one block per sequence (what dense prefill passes):
//     a group's load then runs into the next block's rows, which are cleared like rows past the context end,
//     and the one group at the end of the pool is fetched lane by lane when its tile is published;
//   * the tables hold pa_asm_cap_tiles() tiles from the workgroup's first tile on; the LONG instance fills them
//     again on the way when the workgroup runs more tiles than that;
//   * the host launches prefill_mfma_kernel for tables of several blocks that are not multiples of 16 keys long.
// Only the set-up, the first subtile's S^T and the write-out are compiled code, so the register allocator sees
// one asm statement with pinned operands and little else.
#pragma once
#include "prefill_mfma.h"
#include "prefill_plan.h"
#include "prefill_mfma_loop.inc"

namespace pa_decode_detail {


// LO: the instance that also applies lower bounds (sliding window, per-row first keys): the workgroup starts at
// the tile of the first key its first row sees, everything the loop counts in is relative to that tile.
// LONG: the instance for workgroups that run more tiles than the tables hold (the same code with a loop around the
// assembly that fills the tables again, which costs registers in the set-up).
template <typename T, bool LO, int D, bool LONG = false>
__global__ __launch_bounds__(kPfThreads) void prefill_asm_kernel(const RowwiseArgs a) {
    using M = Mfma16<T>;
    using X8 = typename M::x8;
    static_assert(D == 128 || D == 64 || D == 32, "the assembly loops are generated for these head sizes");
    using G = PfTile<D>;
    constexpr int KS = D / 16, DT = D / 32, NC = kPfCols;
    constexpr int GPT = kPfKeys / 16;  // 16-key groups per tile
    // A wave-wide direct load covers 1 KiB = RPL rows.  head_dim 128: wave w fetches four rows of each of the tile's
    // four groups (NG = 4 loads per tensor: groups 0, 1, 2, 3); head_dim 64: eight rows of two of them (NG = 2:
    // groups w/2 and w/2 + 2); head_dim 32: all sixteen rows of group w (NG = 1).  Load n lands 4 KiB behind load n-1.
    constexpr int NG = G::LOADS / kPfWaves, GSTEP = GPT / NG;
    typedef __attribute__((address_space(3))) char lds_char;
    constexpr int kRingBytes = kPfStages * 2 * G::BYTES;
    constexpr int kPaCapTiles = pa_asm_cap_tiles(D);
    constexpr int kTabABytes = kPaCapTiles * GPT * 4, kTabBBytes = (kPaCapTiles + 1) * GPT;
    static_assert(kPfStages == 4 && kPfKeys == 64 && kPfWaves == 4 && NC == 2, "the assembly loop is written for this shape");
    __shared__ __attribute__((aligned(1024))) char s_mem[kRingBytes + kTabABytes + kTabBBytes];
    __shared__ int s_special[kPfWaves];  // per wave: first tile with a row that does not exist
    const uint32_t lds_base = (uint32_t)(size_t)(lds_char *)s_mem;
    int32_t *tab_a = reinterpret_cast<int32_t *>(s_mem + kRingBytes);
    uint8_t *tab_b = reinterpret_cast<uint8_t *>(s_mem + kRingBytes + kTabABytes);

    const PoolArgs &p = a.p;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5, col = lane & 31;

    // workgroup -> (kv head, chunk of groups of 8 tasks, sequence), heaviest first when the prefix is short (the launch
    // order of prefill_mfma_kernel).  The plain instance runs the a.groups_per_wg groups of its chunk in turn:
    // lengths and slot tables are set up once (the groups of one sequence and kv head share them), which is a
    // third of what a group costs beside its loop and counts where the loop is short (prompts of a few hundred
    // tokens).
    const int kvh = blockIdx.x;
    const int n_splits = a.splits;  // pieces a workgroup's tiles are cut into (1: none; more only in the LO instance)
    const int gpw = (LO || LONG) ? 1 : a.groups_per_wg;  // groups per workgroup
    const int piece = (int)blockIdx.y % n_splits, chunk_y = (int)blockIdx.y / n_splits;
    const int n_chunks = gridDim.y / n_splits, n_seqs = gridDim.z;
    const int lin = chunk_y + n_chunks * blockIdx.z;
    const bool group_major = a.ctx_lens[0] - a.q_lens[0] < a.q_lens[0];
    const int wg_chunk = group_major ? n_chunks - 1 - lin / n_seqs : chunk_y;
    const int b = group_major ? lin % n_seqs : (int)blockIdx.z;
    // (read once and held in scalar registers: a load behind the direct-to-LDS requests would wait for all of them)
    const int q_len = __builtin_amdgcn_readfirstlane(a.q_lens[b]);
    const int ctx_len = __builtin_amdgcn_readfirstlane(a.ctx_lens[b]);
    const int q_start = __builtin_amdgcn_readfirstlane(a.q_starts[b]);
    const int prefix = ctx_len - q_len;
    const int n_rowblocks = (q_len + kPfRows - 1) / kPfRows;
    const int n_tasks = n_rowblocks * p.n_rep;
    // Groups of this workgroup: one of every n_chunks consecutive groups, the wg_chunk-th from the front in even
    // rounds and from the back in odd ones, so that under the causal mask (later groups see more keys) the
    // workgroups' totals come out equal.
    const int group_end = (n_tasks + kPfTasks - 1) / kPfTasks;
    if (wg_chunk >= group_end || q_len <= 0) return;  // uniform over the workgroup
    auto group_of = [&](int i) PF_INLINE { return plan_group_of(i, n_chunks, wg_chunk); };
    int first_special_tab = 0;  // (of the tables, which the workgroup's groups share)
    // Between two groups' loops the ring is empty and its four stages hold: stage 0 - tile 0 of the next group
    // (every group of the workgroup starts at key 0 of the same sequence and kv head); stages 1 and 2 - the next
    // group's Q rows, staged as whole rows (32 rows of each of a wave's two tasks); stage 3 - the rows being written
    // out, one task of each wave at a time.  The first group's Q rows are requested here; a later group's, and
    // its tile 0, before the write-out of the group before it, so that they travel while that group's rows are
    // normalised and stored.
    constexpr int QRB = D * 2, QCPR = QRB / 16, QRPI = 64 / QCPR;
    constexpr int kStoresPerTask = 32 / QRPI;  // store instructions of the write-out per task
    constexpr int kStageBytes = kRingBytes / kPfStages;
    const uint32_t q_stage = (uint32_t)kStageBytes + (uint32_t)wave * (NC * 32 * QRB);
    static_assert(kPfWaves * NC * 32 * QRB == 2 * kStageBytes, "the staged rows of the four waves fill two stages");
    static_assert(kPfWaves * 32 * QRB == kStageBytes, "one task's rows of the four waves fill one stage");
    // (32-bit byte offsets from the sequence's first row: the host checks that a chunk's rows span less than 2 GiB)
    // Head sizes between the compiled ones (p.d < D, a multiple of 8): rows in memory are p.d elements long, the
    // kernel's rows D.  The 16-byte chunks past a row's end are requested from chunk 0 instead (any finite data
    // does) and Q^T holds zeros there, so they add nothing to S^T; what they add to O^T is never stored.
    const uint32_t row_bytes = (uint32_t)p.d * 2;       // a (token, head) row in memory
    const uint32_t real_chunks = row_bytes / 16;        // its 16-byte chunks (<= QCPR)
    const bool padded = real_chunks != (uint32_t)QCPR;  // uniform
    auto real_chunk = [&](uint32_t chunk) PF_INLINE { return chunk < real_chunks ? chunk : 0u; };
    const uint32_t q_row_bytes = (uint32_t)p.hq * row_bytes;
    const uint32_t q_last_row = (uint32_t)(q_len - 1) * q_row_bytes;
    const char *q_seq = reinterpret_cast<const char *>(a.q) + (int64_t)q_start * p.hq * row_bytes;
    auto issue_q = [&](int grp) PF_INLINE {
        const int lrow = lane / QCPR, lslot = lane % QCPR;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int task = grp * kPfTasks + wave * NC + c;
            const bool lv = task < n_tasks;
            const int rb = lv ? task / p.n_rep : 0;
            const int qhead = kvh * p.n_rep + (lv ? task - rb * p.n_rep : 0);
            const char *qb = pf_scalar_ptr(q_seq + qhead * row_bytes);
            const uint32_t row_ofs = (uint32_t)(rb * kPfRows + lrow) * q_row_bytes;
#pragma unroll
            for (int i = 0; i < 32 / QRPI; ++i) {
                const int r = i * QRPI + lrow;
                // (rows past the chunk's end read its last row: they are computed and never stored)
                const uint32_t ofs = min(row_ofs + (uint32_t)(i * QRPI) * q_row_bytes, q_last_row);
                pf_dma16(lds_base + q_stage + (uint32_t)((c * 32 + i * QRPI) * QRB), qb,
                         ofs + real_chunk((uint32_t)(lslot ^ (r & (QCPR - 1)))) * 16);
            }
        }
    };
    issue_q(wg_chunk);
    int prev_stores = 0;  // store instructions this wave issued behind the current group's Q loads
    bool tile0_ahead = false;  // (uniform) tile 0 of the current group was requested with its Q rows

    for (int gi = 0;;) {  // uniform control flow, stated to the compiler
    const int group = __builtin_amdgcn_readfirstlane(group_of(gi));
    const int task0 = group * kPfTasks;
    bool live[NC];
    int row0[NC], qh[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int task = task0 + wave * NC + c;
        live[c] = task < n_tasks;
        const int rb = live[c] ? task / p.n_rep : 0;
        const int rep = live[c] ? task - rb * p.n_rep : 0;
        row0[c] = rb * kPfRows;
        qh[c] = kvh * p.n_rep + rep;
    }
    const int last_task = min(n_tasks, task0 + kPfTasks) - 1;
    int wg_keys = min(ctx_len, prefix + min(q_len, (last_task / p.n_rep) * kPfRows + kPfRows));
    // subtiles that reach past this key hold keys some row of the wave must not see
    const int mask_from = min(prefix + min(row0[0], row0[1]) + 1, ctx_len);
    // a lane's last visible key per column tile, less the 4 keys its half of the wave is ahead by
    int lim[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) lim[c] = min(ctx_len - 1, prefix + row0[c] + col) - 4 * half;
    // Lower bounds (see prefill_mfma_kernel): a row's first visible key under the window and / or the per-row
    // first keys, clamped so that the row always sees its own position; non-decreasing along a sequence.
    int t0 = 0;             // first tile of the workgroup
    int lo_mask_until = 0;  // subtiles that start below this key hold keys some row of the wave cannot see any more
    int lo[NC] = {0, 0};    // a lane's first visible key per column tile, less 4 * half like lim
    if constexpr (LO) {
        const int win = p.window;
        const int32_t *rlo = a.row_lo ? a.row_lo + q_start : nullptr;
        auto row_first = [&](int row) PF_INLINE {
            const int pos = prefix + row;
            int first = win > 0 ? pos - win + 1 : 0;
            if (rlo) first = max(first, rlo[min(row, q_len - 1)]);
            return min(max(first, 0), min(pos, ctx_len - 1));
        };
        t0 = row_first((task0 / p.n_rep) * kPfRows) / kPfKeys;
        lo_mask_until = row_first(min(q_len, max(row0[0], row0[1]) + kPfRows) - 1);
#pragma unroll
        for (int c = 0; c < NC; ++c) lo[c] = row_first(row0[c] + col) - 4 * half;
    }
    if constexpr (LO) {
        if (n_splits > 1) {
            // This workgroup runs piece `piece` of the tiles [t0, t0 + n_all): a later first tile and an earlier
            // last key, nothing else changes (rows that see none of the piece's keys end with an empty sum).
            const int n_all = (wg_keys + kPfKeys - 1) / kPfKeys - t0;
            int tb, te;
            plan_piece_tiles(t0, n_all, piece, n_splits, tb, te);
            if (tb >= te) {  // uniform: fewer tiles than pieces - an empty partial for every row
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const int row = row0[c] + col;
                    if (live[c] && row < q_len && half == 0) {
                        const int64_t at = ((((int64_t)q_start + row) * p.hq + qh[c]) * n_splits + piece) * 2;
                        a.part_ml[at] = kNegBig;
                        a.part_ml[at + 1] = 0.f;
                    }
                }
                return;
            }
            t0 = tb;
            wg_keys = min(wg_keys, te * kPfKeys);
        }
    }
    // tiles the loop runs (>= 1), counted from t0 like every tile number below
    const int n_tiles = (wg_keys + kPfKeys - 1) / kPfKeys - t0;
    // The tables hold kPaCapTiles tiles from a first tile `base` on.  They are filled for base = 0 here and, in the
    // LONG instance, again every kSegTiles tiles: the assembly loop is left and entered again, which is free of side
    // conditions because every pass of its body leaves the state the next one starts from.  (The host launches the
    // other instance when the whole block table fits, or when a sliding window bounds the tiles a workgroup can see.)
    constexpr int kSegTiles = (kPaCapTiles - kPfStages) / kPfStages * kPfStages;  // (the loop starts in ring slot 0)
    const int cap_rel = kPaCapTiles;

    // ---- slot tables (in flight together with the Q rows) ----
    const int64_t pool_rows = p.num_blocks * p.bs;  // >= 16, < 2^31 (the host checks)
    // Blocks that are not multiples of 16 keys long (one block per sequence, as dense prefill passes its rows):
    // a 16-key group may run into the rows of the next block - harmless, they are cleared before the tile is
    // published - but the last group of the pool's last block would run past the end of the pool.  That one
    // group (at most one per workgroup) is loaded from slot 0 instead and its existing rows are copied from
    // where they are, lane by lane, when its tile is published.
    int edge_tile = -1, edge_group = 0, edge_rows = 0;  // tile relative to t0
    int64_t edge_slot = 0;
    if (p.bs % 16 != 0) {  // (then bt_stride is 1)
        const int64_t bid = p.bt[(int64_t)b * p.bt_stride];
        const int n_keys = min(ctx_len, p.bs);
        const int key_last = (n_keys - 1) / 16 * 16;
        if (bid >= 0 && bid < p.num_blocks && bid * p.bs + key_last + 16 > pool_rows && key_last / kPfKeys >= t0) {
            edge_tile = key_last / kPfKeys - t0;
            edge_group = key_last / 16 % GPT;
            edge_rows = n_keys - key_last;
            edge_slot = bid * p.bs + key_last;
        }
    }
    // the tables hold the tiles of this group, or of the whole sequence when the workgroup runs several groups
    const int tab_tiles =
        gpw == 1 ? n_tiles : (ctx_len + kPfKeys - 1) / kPfKeys - t0;  // (several groups: every key of the sequence)
    auto fill_tables = [&](int base) PF_INLINE {
        const int32_t *bt_seq = p.bt + (int64_t)b * p.bt_stride;
        const int n_rest = tab_tiles - base;           // tiles still to run (>= 1)
        const int n_real = min(n_rest, kPaCapTiles);   // those of them with table entries
        const int n_entries = n_real * GPT;  // (the loads of tiles past the last fetch tile 0 again: it has entries)
        int first_special = n_rest;
        for (int i = tid; i < n_entries; i += kPfThreads) {
            const int key = 16 * ((t0 + base) * GPT + i), blk = key / p.bs;
            int64_t bid = -1;
            if (blk < p.bt_stride) bid = bt_seq[blk];
            const bool present = bid >= 0 && bid < p.num_blocks;
            // rows of the group that exist: inside the context and inside the group's block (a block that is not
            // a multiple of 16 keys long is the only block of its sequence: what follows it is absent)
            const int rows = present ? min(max(min(ctx_len, (blk + 1) * p.bs) - key, 0), 16) : 0;
            int64_t slot = present ? bid * p.bs + key % p.bs : 0;
            if (slot + 16 > pool_rows) slot = 0;  // (the group at the end of the pool: see edge_tile below)
            tab_a[i] = (int32_t)slot;
            tab_b[i] = (uint8_t)rows;
            if (rows < 16) first_special = min(first_special, i / GPT);
        }
        if (tid < GPT) tab_b[cap_rel * GPT + tid] = 0;  // tiles past the tables: nothing exists
        if (n_rest > n_real) first_special = min(first_special, n_real);
        // minimum over the wave here, over the waves behind the next barrier (read_special)
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) first_special = min(first_special, __shfl_xor(first_special, d, 64));
        if (lane == 0) s_special[wave] = first_special;
    };
    // first tile (counted from the tables' base) with a row that does not exist
    auto read_special = [&]() PF_INLINE {
        return __builtin_amdgcn_readfirstlane(min(min(s_special[0], s_special[1]), min(s_special[2], s_special[3])));
    };
    const bool first_group = gi == 0;  // uniform
    if (first_group) {
        fill_tables(0);
        pf_wait_loads<0>();
    } else if (prev_stores == 2 * kStoresPerTask) {
        // this group's Q rows were requested before the last group's stores: wait for them, not for the stores
        pf_wait_loads<2 * kStoresPerTask>();
    } else if (prev_stores == kStoresPerTask) {
        pf_wait_loads<kStoresPerTask>();
    } else {
        pf_wait_loads<0>();
    }
    const float sc = p.scale_log2;
    X8 qreg[NC][KS];
    uint4 q_raw[NC][KS];  // (all reads first: one LDS round trip)
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int slot = (2 * ks + half) ^ (col & (QCPR - 1));
            q_raw[c][ks] = *reinterpret_cast<const uint4 *>(s_mem + q_stage + (c * 32 + col) * QRB + slot * 16);
        }
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const uint4 raw = q_raw[c][ks];
            // scaled by softmax scale * log2(e) here, once per workgroup: S^T then comes out of the products in
            // the units of the exponential's argument (one more rounding of q to its 16-bit type)
            const X8 q8 = __builtin_bit_cast(X8, raw);
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = M::pack((float)q8[2 * e] * sc, (float)q8[2 * e + 1] * sc);
            if (padded && (uint32_t)(2 * ks + half) >= real_chunks) w[0] = w[1] = w[2] = w[3] = 0;  // past the row's end
            qreg[c][ks] = __builtin_bit_cast(X8, uint4{w[0], w[1], w[2], w[3]});
        }
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(qreg[c][ks]));
    __syncthreads();  // the tables are complete and the staged rows have been read: the ring may overwrite them
    if (first_group) first_special_tab = read_special();
    int first_special = min(first_special_tab, n_tiles);  // (a group before the last runs fewer tiles than the tables hold)

    // ---- loads of a tile: wave w fetches rows w*RPL .. w*RPL + RPL-1 of the tile and, NG-1 times, the rows 4*RPL on ----
    const int64_t tok_stride = (int64_t)p.hkv * row_bytes;
    const char *pool_k = reinterpret_cast<const char *>(p.k) + (int64_t)kvh * row_bytes;
    const char *pool_v = reinterpret_cast<const char *>(p.v) + (int64_t)kvh * row_bytes;
    const int ld_row = lane / G::CPR, ld_slot = lane % G::CPR;
    const int tile_row = wave * G::RPL + ld_row;  // this lane's row of the tile in the wave's first load
    const int g0 = (wave * G::RPL) / 16;          // the 16-key group of that load; load n: group g0 + n * GSTEP
    const int arow = tile_row % 16;               // this lane's row inside its 16-key group
    const uint32_t lane_k = (uint32_t)(arow * tok_stride) + real_chunk((uint32_t)(ld_slot ^ G::swz_k(tile_row))) * 16;
    const uint32_t lane_v = (uint32_t)(arow * tok_stride) + real_chunk((uint32_t)(ld_slot ^ G::swz_v(tile_row))) * 16;
    const uint32_t m0w = lds_base + (uint32_t)wave * (G::RPL * G::RB);
    constexpr int kLoadStep = kPfWaves * G::RPL * G::RB;  // LDS bytes between a wave's consecutive loads
    static_assert(kLoadStep == 4096, "the assembly loops place a wave's loads 4 KiB apart");
    auto issue = [&](int tile) PF_INLINE {
        const int src = tile < min(n_tiles, kPaCapTiles) ? tile : 0;
        const uint32_t dst0 = m0w + (uint32_t)(tile % kPfStages) * 2 * G::BYTES;
        int32_t slots[NG];  // (read together: one wait for the table instead of one per load)
#pragma unroll
        for (int n = 0; n < NG; ++n) slots[n] = tab_a[src * GPT + g0 + n * GSTEP];
#pragma unroll
        for (int n = 0; n < NG; ++n) {
            const uint32_t slot = (uint32_t)__builtin_amdgcn_readfirstlane(slots[n]);
            const uint64_t ofs = (uint64_t)slot * (uint32_t)tok_stride;
            pf_dma16(dst0 + n * kLoadStep, pf_scalar_ptr(pool_k + ofs), lane_k);
            pf_dma16(dst0 + G::BYTES + n * kLoadStep, pf_scalar_ptr(pool_v + ofs), lane_v);
        }
    };
    // this wave's load of the group at the end of the pool, as an LDS offset behind the wave's first load (-1: none)
    const int edge_n = edge_group - g0;
    const int edge_ofs = edge_tile >= 0 && edge_n >= 0 && edge_n % GSTEP == 0 ? edge_n / GSTEP * kLoadStep : -1;
    auto mend_tile0 = [&]() PF_INLINE {  // (the loop does this for later tiles)
        if (first_special == 0) {  // clear the rows of tile 0 that do not exist
#pragma unroll
            for (int n = 0; n < NG; ++n)
                if (arow >= tab_b[g0 + n * GSTEP]) {
                    const uint32_t at = (m0w - lds_base) + n * kLoadStep + lane * 16;
                    *reinterpret_cast<uint4 *>(s_mem + at) = uint4{0, 0, 0, 0};
                    *reinterpret_cast<uint4 *>(s_mem + at + G::BYTES) = uint4{0, 0, 0, 0};
                }
        }
        if (edge_tile == 0 && edge_ofs >= 0 && arow < edge_rows) {
            const uint32_t at = (m0w - lds_base) + edge_ofs + lane * 16;
            *reinterpret_cast<uint4 *>(s_mem + at) = *reinterpret_cast<const uint4 *>(pool_k + edge_slot * tok_stride + lane_k);
            *reinterpret_cast<uint4 *>(s_mem + at + G::BYTES) =
                *reinterpret_cast<const uint4 *>(pool_v + edge_slot * tok_stride + lane_v);
        }
    };
    if (tile0_ahead) {
        // tile 0 landed with the Q rows and the barrier above published it
        issue(1);
        issue(2);
        if (first_special == 0 || edge_tile == 0) {  // uniform, rare: a context of less than a tile, an absent first block
            mend_tile0();
            __syncthreads();
        }
    } else {
        issue(0);
        issue(1);
        issue(2);
        pf_wait_loads<4 * NG>();  // tile 0 has landed
        mend_tile0();
        __syncthreads();  // tile 0 is visible
    }

    // ---- operand read addresses (stage 0), as in prefill_mfma_kernel ----
    uint32_t kad[KS], vad[DT];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kad[ks] = lds_base + col * G::RB + (((2 * ks + half) ^ G::swz_k(col)) * 16);
    {
        const int g16 = lane >> 4, s16 = lane & 15;
        const int v_key = 4 * (g16 >> 1) + (s16 >> 2);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            vad[dt] = lds_base + G::BYTES + v_key * G::RB +
                      ((((4 * dt) ^ G::swz_v(v_key)) + 2 * (g16 & 1) + ((s16 & 3) >> 1)) * 16) + 8 * (s16 & 1);
    }

    // ---- first subtile: S^T, mask, row maxima; K operands of the second subtile ----
    f32x16 s0[NC];
    X8 ka[KS];
    float mx[NC];
    {
        auto read_k = [&](int kt) PF_INLINE {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                ka[ks] = __builtin_bit_cast(X8, *reinterpret_cast<const __attribute__((address_space(3))) uint4 *>(
                                                    (const lds_char *)(size_t)kad[ks] + kt * 32 * G::RB));
        };
        read_k(0);
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int i = 0; i < 16; ++i) s0[c][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int c = 0; c < NC; ++c) s0[c] = M::mma(ka[ks], qreg[c][ks], s0[c]);
        read_k(1);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            float m = kNegBig;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int idx = 8 * (i >> 2) + (i & 3) + kPfKeys * t0;  // (+ 4 * half: folded into lim and lo)
                if (idx > lim[c] || (LO && idx < lo[c])) s0[c][i] = -INFINITY;
                m = fmaxf(m, s0[c][i]);
            }
            const uint32_t u = __builtin_bit_cast(uint32_t, m);
            const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
            mx[c] = fmaxf(__builtin_bit_cast(float, (uint32_t)sw[0]), __builtin_bit_cast(float, (uint32_t)sw[1]));
        }
    }
    // The reference maximum of a row starts as the maximum of its first subtile.  From here on S^T is kept
    // relative to the reference: the loop's first product of each column tile accumulates onto ref[c] = minus
    // the reference in all 16 registers, the exponentials take S^T as it is, and mx is the maximum relative to
    // the reference (0 now).  The reference moves up only when a later maximum exceeds it by more than kPfSlack
    // (lazy rescale: see prefill_mfma_kernel).  Without lower bounds every row sees key 0, so the maximum is
    // finite; with them a row may see nothing of the first subtile: its reference stays unset (thr = a large
    // negative number instead of the slack) until a maximum of visible keys arrives, which then becomes the
    // reference whatever its sign.
    f32x16 ref[NC];
    float thr[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const bool seen = mx[c] > kNegBig;
        const float m0 = seen ? mx[c] : 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s0[c][i] -= m0;
            ref[c][i] = -m0;
        }
        if (seen) mx[c] = 0.f;
        thr[c] = seen ? kPfSlack : kNegBig;
    }
    f32x16 o[NC][DT];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[c][dt][i] = 0.f;
    float l_run[NC] = {0.f, 0.f};  // running sums

    {
        // (wave-uniform values the compiler may hold in vector registers are moved to scalar ones for the "s" operands)
        auto uni = [](int v) PF_INLINE { return __builtin_amdgcn_readfirstlane(v); };
        const uint32_t tab_a_base = lds_base + kRingBytes + 4 * g0;  // (the wave's first group folded in)
        const uint32_t tab_b_base = lds_base + kRingBytes + kTabABytes;
        const uint32_t cap_tiles = (uint32_t)uni(cap_rel), mask_from_u = (uint32_t)uni(mask_from);
        const uint32_t lane16 = (uint32_t)lane * 16, arow_u = (uint32_t)arow;
        const uint64_t pk = reinterpret_cast<uint64_t>(pool_k), pv = reinterpret_cast<uint64_t>(pool_v);
        const uint32_t pklo = __builtin_amdgcn_readfirstlane((uint32_t)pk), pkhi = __builtin_amdgcn_readfirstlane((uint32_t)(pk >> 32));
        const uint32_t pvlo = __builtin_amdgcn_readfirstlane((uint32_t)pv), pvhi = __builtin_amdgcn_readfirstlane((uint32_t)(pv >> 32));
        const uint32_t stride = (uint32_t)tok_stride;
        const uint32_t edge_slot_u = (uint32_t)uni((int)edge_slot);
        const uint32_t edge_rows_u = (uint32_t)uni(edge_rows), edge_ofs_u = (uint32_t)uni(edge_ofs);
        const float slack = kPfSlack;  // in the units of S^T here: log2 of the factor a row's reference may lag by
#define PA_LOOP_COMMON_OUT(...)                                                                                      \
      "+{v[0:15]}"(s0[0]), "+{v[16:31]}"(s0[1]), "+{v[118:133]}"(ref[0]), "+{v[134:149]}"(ref[1]),                    \
      [mx0] "+&v"(mx[0]), [mx1] "+&v"(mx[1]), [l0] "+&v"(l_run[0]), [l1] "+&v"(l_run[1]),                             \
      [ntiles] "+&s"(n_left), [sT] "+&s"(s_t), [sP] "+&s"(s_p), [srem] "+&s"(s_rem) __VA_ARGS__
#define PA_LOOP_COMMON_IN(...)                                                                                        \
      [lanek] "v"(lane_k), [lanev] "v"(lane_v), [lane16] "v"(lane16),                                                   \
      [arow] "v"(arow_u), [lim0] "v"(lim[0]), [lim1] "v"(lim[1]), [slack] "s"(slack),                                   \
      [pklo] "s"(pklo), [pkhi] "s"(pkhi), [pvlo] "s"(pvlo), [pvhi] "s"(pvhi), [stride] "s"(stride), [m0w] "s"(m0w),     \
      [nreal] "s"(n_real_u), [tabA] "s"(tab_a_base), [tabB] "s"(tab_b_base), [splo] "s"(sp_lo),                       \
      [spspan] "s"(sp_span), [captiles] "s"(cap_tiles), [maskfrom] "s"(mask_from_u),                                \
      [edgetile] "s"(edge_tile_u), [edgeslot] "s"(edge_slot_u), [edgerows] "s"(edge_rows_u),                          \
      [edgeofs] "s"(edge_ofs_u) __VA_ARGS__                       \
    : "v32", "v33", "v34", "v35", "v36", "v37", "v38", "v39", "v40", "v41", "v42", "v43", "v44", "v45", "v46", "v47",  \
      "v48", "v49", "v50", "v51", "v52", "v53", "v54", "v55", "v56", "v57", "v58", "v59", "v60", "v61", "v62", "v63",  \
      "v64", "v65", "v66", "v67", "v68", "v69", "v70", "v71", "v72", "v73", "v74", "v75", "v76", "v77", "v78", "v79",  \
      "v80", "v81", "v82", "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95",  \
      "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105", "v106", "v107", "v108", "v109",      \
      "v110", "v111", "v112", "v113", "v114", "v115", "v116", "a224", "a225", "a226", "a227", "a228", "a229", "a230",  \
      "a231", "a232", "a233", "a234", "a235", "a236", "a237", "a238", "a239", "a240", "a241", "a242", "a243", "a244",  \
      "a245", "a246", "a247", "a248", "a249", "a250", "a251", "a252", "a253", "a254", "a255", "s40", "s41", "s42",     \
      "s43", "s44", "s45", "s46", "s47", "s48", "s49", "s50", "s51", "s52", "s53", "s54", "s55", "s56", "s57", "s58",  \
      "s59", "s60", "s61", "s62", "s63", "vcc", "scc", "memory"
// head_dim 128: o[c][dt] at a[16*(4c+dt)], q[c][ks] at a[128 + 4*(8c+ks)], ka[ks] at a[192 + 4*ks] (Q^T is only read;
// as read-write operands its registers stay where they are when the statement sits in a loop)
#define PA_LOOP_OPERANDS(MORE_OUT, MORE_IN)                                                                           \
    : "+{a[0:15]}"(o[0][0]), "+{a[16:31]}"(o[0][1]), "+{a[32:47]}"(o[0][2]), "+{a[48:63]}"(o[0][3]),                    \
      "+{a[64:79]}"(o[1][0]), "+{a[80:95]}"(o[1][1]), "+{a[96:111]}"(o[1][2]), "+{a[112:127]}"(o[1][3]),                \
      "+{a[192:195]}"(ka[0]), "+{a[196:199]}"(ka[1]), "+{a[200:203]}"(ka[2]), "+{a[204:207]}"(ka[3]),                   \
      "+{a[208:211]}"(ka[4]), "+{a[212:215]}"(ka[5]), "+{a[216:219]}"(ka[6]), "+{a[220:223]}"(ka[7]),                   \
      "+{a[128:131]}"(qreg[0][0]), "+{a[132:135]}"(qreg[0][1]), "+{a[136:139]}"(qreg[0][2]), "+{a[140:143]}"(qreg[0][3]), \
      "+{a[144:147]}"(qreg[0][4]), "+{a[148:151]}"(qreg[0][5]), "+{a[152:155]}"(qreg[0][6]), "+{a[156:159]}"(qreg[0][7]), \
      "+{a[160:163]}"(qreg[1][0]), "+{a[164:167]}"(qreg[1][1]), "+{a[168:171]}"(qreg[1][2]), "+{a[172:175]}"(qreg[1][3]), \
      "+{a[176:179]}"(qreg[1][4]), "+{a[180:183]}"(qreg[1][5]), "+{a[184:187]}"(qreg[1][6]), "+{a[188:191]}"(qreg[1][7]), \
      PA_LOOP_COMMON_OUT(MORE_OUT)                                                                                    \
    : [kad0] "v"(kad[0]), [kad1] "v"(kad[1]), [kad2] "v"(kad[2]), [kad3] "v"(kad[3]), [kad4] "v"(kad[4]),               \
      [kad5] "v"(kad[5]), [kad6] "v"(kad[6]), [kad7] "v"(kad[7]), [vad0] "v"(vad[0]), [vad1] "v"(vad[1]),               \
      [vad2] "v"(vad[2]), [vad3] "v"(vad[3]), PA_LOOP_COMMON_IN(MORE_IN)
// head_dim 64: o[c][dt] at a[16*(2c+dt)], q[c][ks] at a[128 + 4*(4c+ks)], ka[ks] at a[192 + 4*ks]; bshift: the bit
// of the wave's first group in a tile's row of table B
#define PA_LOOP_OPERANDS_D64(MORE_OUT, MORE_IN)                                                                       \
    : "+{a[0:15]}"(o[0][0]), "+{a[16:31]}"(o[0][1]), "+{a[32:47]}"(o[1][0]), "+{a[48:63]}"(o[1][1]),                    \
      "+{a[192:195]}"(ka[0]), "+{a[196:199]}"(ka[1]), "+{a[200:203]}"(ka[2]), "+{a[204:207]}"(ka[3]),                   \
      PA_LOOP_COMMON_OUT(MORE_OUT)                                                                                    \
    : "{a[128:131]}"(qreg[0][0]), "{a[132:135]}"(qreg[0][1]), "{a[136:139]}"(qreg[0][2]), "{a[140:143]}"(qreg[0][3]),   \
      "{a[144:147]}"(qreg[1][0]), "{a[148:151]}"(qreg[1][1]), "{a[152:155]}"(qreg[1][2]), "{a[156:159]}"(qreg[1][3]),   \
      [kad0] "v"(kad[0]), [kad1] "v"(kad[1]), [kad2] "v"(kad[2]), [kad3] "v"(kad[3]), [vad0] "v"(vad[0]),               \
      [vad1] "v"(vad[1]), [bshift] "s"(b_shift), PA_LOOP_COMMON_IN(MORE_IN)
// head_dim 32: o[c][0] at a[16*c], q[c][ks] at a[128 + 4*(2c+ks)], ka[ks] at a[192 + 4*ks]
#define PA_LOOP_OPERANDS_D32(MORE_OUT, MORE_IN)                                                                       \
    : "+{a[0:15]}"(o[0][0]), "+{a[16:31]}"(o[1][0]), "+{a[192:195]}"(ka[0]), "+{a[196:199]}"(ka[1]),                    \
      PA_LOOP_COMMON_OUT(MORE_OUT)                                                                                    \
    : "{a[128:131]}"(qreg[0][0]), "{a[132:135]}"(qreg[0][1]), "{a[136:139]}"(qreg[1][0]), "{a[140:143]}"(qreg[1][1]),   \
      [kad0] "v"(kad[0]), [kad1] "v"(kad[1]), [vad0] "v"(vad[0]), [bshift] "s"(b_shift), PA_LOOP_COMMON_IN(MORE_IN)
#define PA_NOTHING
#define PA_LO_OUT , [thr0] "+&v"(thr[0]), [thr1] "+&v"(thr[1]), [slo] "+&s"(s_lo)
#define PA_LO_IN , [lo0] "v"(lo[0]), [lo1] "v"(lo[1]), [negbig] "s"(neg_big)
        const float neg_big = kNegBig;
        constexpr bool BF = std::is_same<T, pa_bf16>::value;
        const int n_tiles_u = uni(n_tiles);
        for (int base = 0;;) {  // one pass per fill of the tables (uniform control flow, stated to the compiler)
        const int n_rest = n_tiles_u - base;
        const int n_seg = LONG ? uni(min(n_rest, kSegTiles)) : n_rest;  // tiles of this pass
        int n_left = uni(n_seg - 1);  // tiles after the current one
        uint32_t s_t = 3, s_p = 1;    // (the loop counts tiles from the tables' base)
        int s_rem = uni(mask_from - kPfKeys * (t0 + base));      // mask_from - 64 * (absolute) tile
        int s_lo = uni(lo_mask_until - kPfKeys * (t0 + base));   // the same for the lower bound
        // tiles in [sp_lo, sp_lo + sp_span) are checked before they are published (the pass publishes tiles 1 .. n_seg)
        const uint32_t sp_lo = (uint32_t)uni(first_special);
        const uint32_t sp_span = (uint32_t)uni(max(min(n_rest, n_seg + 1) - first_special, 0));
        const uint32_t n_real_u = (uint32_t)uni(min(n_rest, kPaCapTiles));
        const uint32_t edge_tile_u = (uint32_t)uni(edge_tile >= base ? edge_tile - base : -1);
        if constexpr (D == 128 && LO) {
            if constexpr (BF) {
                asm volatile(PF_LOOP_ASM_BF16_LO PA_LOOP_OPERANDS(PA_LO_OUT, PA_LO_IN));
            } else {
                asm volatile(PF_LOOP_ASM_F16_LO PA_LOOP_OPERANDS(PA_LO_OUT, PA_LO_IN));
            }
        } else if constexpr (D == 128) {
            (void)s_lo; (void)neg_big;
            if constexpr (BF) {
                asm volatile(PF_LOOP_ASM_BF16 PA_LOOP_OPERANDS(PA_NOTHING, PA_NOTHING));
            } else {
                asm volatile(PF_LOOP_ASM_F16 PA_LOOP_OPERANDS(PA_NOTHING, PA_NOTHING));
            }
        } else if constexpr (D == 32 && LO) {
            const uint32_t b_shift = (uint32_t)uni(8 * g0);
            if constexpr (BF) {
                asm volatile(PF_LOOP_ASM_D32_BF16_LO PA_LOOP_OPERANDS_D32(PA_LO_OUT, PA_LO_IN));
            } else {
                asm volatile(PF_LOOP_ASM_D32_F16_LO PA_LOOP_OPERANDS_D32(PA_LO_OUT, PA_LO_IN));
            }
        } else if constexpr (D == 32) {
            (void)s_lo; (void)neg_big;
            const uint32_t b_shift = (uint32_t)uni(8 * g0);
            if constexpr (BF) {
                asm volatile(PF_LOOP_ASM_D32_BF16 PA_LOOP_OPERANDS_D32(PA_NOTHING, PA_NOTHING));
            } else {
                asm volatile(PF_LOOP_ASM_D32_F16 PA_LOOP_OPERANDS_D32(PA_NOTHING, PA_NOTHING));
            }
        } else if constexpr (LO) {
            const uint32_t b_shift = (uint32_t)uni(8 * g0);
            if constexpr (BF) {
                asm volatile(PF_LOOP_ASM_D64_BF16_LO PA_LOOP_OPERANDS_D64(PA_LO_OUT, PA_LO_IN));
            } else {
                asm volatile(PF_LOOP_ASM_D64_F16_LO PA_LOOP_OPERANDS_D64(PA_LO_OUT, PA_LO_IN));
            }
        } else {
            (void)s_lo; (void)neg_big;
            const uint32_t b_shift = (uint32_t)uni(8 * g0);
            if constexpr (BF) {
                asm volatile(PF_LOOP_ASM_D64_BF16 PA_LOOP_OPERANDS_D64(PA_NOTHING, PA_NOTHING));
            } else {
                asm volatile(PF_LOOP_ASM_D64_F16 PA_LOOP_OPERANDS_D64(PA_NOTHING, PA_NOTHING));
            }
        }
        if constexpr (!LONG) break;
        base = uni(base + n_seg);
        if (base >= n_tiles_u) break;
        __syncthreads();  // every wave has left the loop: nobody reads the tables
        fill_tables(base);
        __syncthreads();
        first_special = read_special();
        }
#undef PA_LOOP_OPERANDS
#undef PA_LOOP_OPERANDS_D64
#undef PA_LOOP_OPERANDS_D32
#undef PA_LOOP_COMMON_OUT
#undef PA_LOOP_COMMON_IN
#undef PA_NOTHING
#undef PA_LO_OUT
#undef PA_LO_IN
    }

    if constexpr (LO) {
        if (n_splits > 1) {
            // ---- a piece: the row's reference maximum, sum and unnormalised O^T go to the workspace ----
            // (the accumulators sit in the registers the assembly loop pins them to; they leave through a multiply
            // by a one the compiler cannot see through, as they do through the normalisation in the write-out below -
            // a plain copy of such an element is mis-selected by this compiler)
            float one = 1.f;
            asm volatile("" : "+v"(one));
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const float l_tot = l_run[c] + __shfl_xor(l_run[c], 32, 64);
                const int row = row0[c] + col;
                if (!live[c] || row >= q_len) continue;
                const int64_t at = (((int64_t)q_start + row) * p.hq + qh[c]) * n_splits + piece;
                float *po = a.part_o + at * D + 4 * half;  // lane owns d = 32*dt + 8*g + 4*half + j
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        *reinterpret_cast<float4 *>(po + 32 * dt + 8 * g) =
                            float4{o[c][dt][4 * g] * one, o[c][dt][4 * g + 1] * one, o[c][dt][4 * g + 2] * one,
                                   o[c][dt][4 * g + 3] * one};
                if (half == 0) {
                    a.part_ml[at * 2] = l_tot > 0.f ? -(ref[c][0] * one) : kNegBig;  // (a row that saw no key has no maximum)
                    a.part_ml[at * 2 + 1] = l_tot;
                }
            }
            return;
        }
    }
    // ---- normalise; rows go through LDS so that every store instruction writes whole 256-byte rows ----
    __syncthreads();  // every wave is done with the ring
    const int group_next = __builtin_amdgcn_readfirstlane(group_of(gi + 1));
    tile0_ahead = false;
    if (group_next < group_end) {  // (uniform) the next group's Q rows and its tile 0 travel during the write-out
        issue_q(group_next);
        if constexpr (!LO && !LONG) {
            issue(0);
            tile0_ahead = true;
        }
    }
    const uint32_t out_stage = 3u * kStageBytes + (uint32_t)wave * (32 * QRB);  // this wave's 32 rows of a task
    // Stores through a descriptor of the sequence's rows: a row past the chunk's length falls outside it and is
    // dropped, so every task costs exactly kStoresPerTask store instructions - the count the next group's wait
    // for its Q rows (requested before these stores) relies on.
    const __amdgpu_buffer_rsrc_t rout = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(reinterpret_cast<char *>(a.out) + (int64_t)q_start * q_row_bytes), 0, q_len * (int)q_row_bytes, 0x00020000);
    prev_stores = 0;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        if (!live[c]) continue;  // uniform
        const float l_tot = l_run[c] + __shfl_xor(l_run[c], 32, 64);
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        // lane owns row col, d = 32*dt + 8*g + 4*half + j: the 8 bytes are half `half` of 16-byte chunk 4*dt + g,
        // chunks swizzled by row so that the 32 rows of a store spread over the banks
        char *rowp = s_mem + out_stage + col * QRB;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                uint2 w;
                w.x = M::pack(o[c][dt][4 * g] * inv, o[c][dt][4 * g + 1] * inv);
                w.y = M::pack(o[c][dt][4 * g + 2] * inv, o[c][dt][4 * g + 3] * inv);
                *reinterpret_cast<uint2 *>(rowp + (((4 * dt + g) ^ (col & (QCPR - 1))) * 16) + 8 * half) = w;
            }
        // (a wave reads only what it wrote itself, and LDS serves a wave in order: no barrier)
        const int r_in = lane / QCPR, chunk = lane % QCPR;  // QRPI rows per instruction, 16 bytes per lane
        prev_stores += kStoresPerTask;
        uint4 rows[32 / QRPI];  // (all reads before the first store: one LDS round trip, not one per store)
#pragma unroll
        for (int i = 0; i < 32 / QRPI; ++i) {
            const int r = i * QRPI + r_in;
            rows[i] = *reinterpret_cast<const uint4 *>(s_mem + out_stage + r * QRB + ((chunk ^ (r & (QCPR - 1))) * 16));
        }
        // (a chunk past the end of the row in memory gets an offset outside the descriptor: dropped)
        const int out_ofs = (uint32_t)chunk < real_chunks
                                ? (int)(((uint32_t)(row0[c] + r_in) * p.hq + qh[c]) * row_bytes) + chunk * 16
                                : (int)0x80000000u;
#pragma unroll
        for (int i = 0; i < 32 / QRPI; ++i)
            __builtin_amdgcn_raw_buffer_store_b128(pa_u4{rows[i].x, rows[i].y, rows[i].z, rows[i].w}, rout,
                                                   out_ofs + i * QRPI * (int)q_row_bytes, 0, 0);
    }
    gi = __builtin_amdgcn_readfirstlane(gi + 1);
    if (group_next >= group_end) break;
    // (no barrier: until the next group's barrier behind its Q^T read, a wave touches only its own staged rows)
    }  // groups of the workgroup
}

// nullptr unless the element type has this kernel; `lower_bounds`: the instance for sliding windows and per-row
// first keys; `long_table`: the instance that fills its tables more than once
prefill_mfma_fn pa_prefill_asm_kernel(int dtype, int head_dim, bool lower_bounds, bool long_table);

}  // namespace pa_decode_detail
