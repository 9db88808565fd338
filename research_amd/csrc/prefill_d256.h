// Causal prefill attention over a paged context on the gfx950 matrix cores for head_dim 256 (bf16 / fp16).
//
// The computation and the operand layouts are those of prefill_mfma_kernel (prefill_mfma.h): S^T = K . Q^T and
// O^T += V^T . P^T with v_mfma_f32_32x32x16, a query row per lane, lazy rescaling.  What head_dim 256 changes is
// the budget.  The accumulators of 32 query rows already fill 128 registers and their Q^T operands 64, so a wave
// owns ONE column tile of 32 rows (a workgroup = 4 waves = 4 tasks), and 64 keys of K and V are 64 KiB, so the
// LDS ring holds stages of 32 keys (one subtile): 4 stages x 32 KiB.
//
// With so little LDS per stage the order in which data is needed decides how far ahead the loads can run.  The
// software pipeline multiplies S^T of subtile g+1 while subtile g is exponentiated, so K of a subtile is read
// two subtiles before its V^T.  Stage s of the ring therefore holds V of tile s and K of tile s+1: everything a
// stage holds has been read by the middle of subtile s, which is where the barrier of the subtile sits, and
// behind that barrier the loads of stage s+4 go into the same slot while stages s+1 .. s+3 are resident or in
// flight: three subtiles of load latency are hidden with 128 KiB of LDS.
//
// Loads are table driven, as in prefill_asm_kernel: the pool slot of every 16-key group of the context is looked
// up once per workgroup and kept in LDS behind the ring (with the number of rows of the group that exist); rows
// past the context end or in absent blocks are fetched from a slot that exists and cleared in LDS before the
// stage is published, so every wave issues the same number of loads per stage and the waits are plain counts.
// A group must lie inside one pool block: block sizes that are multiples of 16, or one block per sequence of any
// length (what dense prefill passes).  In the second case a group's load may run into the next block's rows -
// they are cleared like rows past the context end - and the one group at the end of the pool is fetched lane
// by lane when the stages that hold it are published.
//
// The subtile loop is scheduled assembly (prefill_d256_loop.inc, written by gen_prefill_loop_d256.py), in one
// instance without and one with lower bounds (LO: sliding window, per-row first keys); the set-up, the first
// subtile's S^T and the write-out are compiled code.
// Every wave runs every subtile of the workgroup, with the masks applied where needed: a wave past its last
// visible key multiplies exact zeros.
#pragma once
#include "prefill_mfma.h"
#include "prefill_plan.h"
#include "prefill_d256_loop.inc"

namespace pa_decode_detail {

constexpr int kWdKeys = 32;          // keys per ring stage
constexpr int kWdStages = 4;
constexpr int kWdTasks = kPfWaves;   // tasks (32 query rows of one head) per workgroup: one per wave
constexpr int kWdCapGroups = 6144;   // 16-key groups the slot tables hold, from the workgroup's first tile on

// LONG: the instance for workgroups that run more tiles than the tables hold (it fills them again on the way; the
// other instance is the same code without that loop around the assembly, which costs it registers in the set-up).
template <typename T, bool LO, bool LONG>
__global__ __launch_bounds__(kPfThreads) void prefill_d256_kernel(const RowwiseArgs a) {
    using M = Mfma16<T>;
    using X8 = typename M::x8;
    using X4 = typename M::x4;
    constexpr int D = 256, KS = D / 16, DT = D / 32;
    constexpr int RB = D * 2;               // row bytes
    constexpr int CPR = RB / 16;            // 16-byte chunks per row
    constexpr int TENSOR = kWdKeys * RB;    // K (or V) of one stage
    constexpr int STAGE = 2 * TENSOR;       // K of tile s+1, then V of tile s
    constexpr int kRingBytes = kWdStages * STAGE;
    constexpr int CAP = kWdCapGroups;       // entry CAP of both tables: a group of which nothing exists
    constexpr int NL = 4;                   // direct loads per wave, stage and tensor (2 rows each)
    typedef __attribute__((address_space(3))) char lds_char;
    constexpr int kTabEntries = CAP + 4;    // (entries CAP .. CAP+3: groups of which nothing exists)
    __shared__ __attribute__((aligned(1024))) char s_mem[kRingBytes + kTabEntries * 4 + kTabEntries];
    __shared__ int s_special[kPfWaves];
    const uint32_t lds_base = (uint32_t)(size_t)(lds_char *)s_mem;
    int32_t *tab_a = reinterpret_cast<int32_t *>(s_mem + kRingBytes);            // pool slot of the group's first key
    uint8_t *tab_b = reinterpret_cast<uint8_t *>(s_mem + kRingBytes + kTabEntries * 4);  // rows of the group that exist

    const PoolArgs &p = a.p;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5, col = lane & 31;

    // workgroup -> (kv head, group of 4 tasks, sequence): the launch order of prefill_mfma_kernel
    const int kvh = blockIdx.x;
    const int n_splits = a.splits;  // pieces a workgroup's tiles are cut into (1: none; more only in the LO instances)
    const int piece = (int)blockIdx.y % n_splits, group_y = (int)blockIdx.y / n_splits;
    const int n_groups = gridDim.y / n_splits, n_seqs = gridDim.z;
    const int lin = group_y + n_groups * blockIdx.z;
    const bool group_major = a.ctx_lens[0] - a.q_lens[0] < a.q_lens[0];
    const int group = group_major ? n_groups - 1 - lin / n_seqs : group_y;
    const int b = group_major ? lin % n_seqs : (int)blockIdx.z;
    const int q_len = a.q_lens[b];
    const int ctx_len = a.ctx_lens[b];
    const int prefix = ctx_len - q_len;
    const int n_rowblocks = (q_len + kPfRows - 1) / kPfRows;
    const int n_tasks = n_rowblocks * p.n_rep;
    const int task0 = group * kWdTasks;
    if (task0 >= n_tasks || q_len <= 0) return;  // uniform over the workgroup

    const int task = task0 + wave;
    const bool live = task < n_tasks;
    const int rb = live ? task / p.n_rep : 0;
    const int row0 = rb * kPfRows;
    const int qh = kvh * p.n_rep + (live ? task - rb * p.n_rep : 0);
    const int last_task = min(n_tasks, task0 + kWdTasks) - 1;
    const int wg_keys = min(ctx_len, prefix + min(q_len, (last_task / p.n_rep) * kPfRows + kPfRows));
    int n_tiles = (wg_keys + kWdKeys - 1) / kWdKeys;  // >= 1; the workgroup runs tiles t0 .. n_tiles-1
    // lower bounds (sliding window, per-row first keys): see prefill_mfma_kernel
    const int win = p.window;
    const int32_t *rlo = a.row_lo ? a.row_lo + a.q_starts[b] : nullptr;
    const bool bounded = win > 0 || rlo != nullptr;  // uniform
    auto row_first = [&](int row) PF_INLINE {
        const int pos = prefix + row;
        int lo = win > 0 ? pos - win + 1 : 0;
        if (rlo) lo = max(lo, rlo[min(row, q_len - 1)]);
        return min(max(lo, 0), min(pos, ctx_len - 1));
    };
    const int wg_first_key = bounded ? row_first((task0 / p.n_rep) * kPfRows) : 0;
    int t0 = wg_first_key / kWdKeys;  // first tile of the workgroup (< n_tiles)
    if constexpr (LO) {
        if (n_splits > 1) {
            // This workgroup runs piece `piece` of the tiles [t0, n_tiles): a later first tile and an earlier last
            // one, nothing else changes (rows that see none of the piece's keys end with an empty sum).
            const int n_all = n_tiles - t0;
            int tb, te;
            plan_piece_tiles(t0, n_all, piece, n_splits, tb, te);
            if (tb >= te) {  // uniform: fewer tiles than pieces - an empty partial for every row
                const int row = row0 + col;
                if (live && row < q_len && half == 0) {
                    const int64_t at = ((((int64_t)a.q_starts[b] + row) * p.hq + qh) * n_splits + piece) * 2;
                    a.part_ml[at] = kNegBig;
                    a.part_ml[at + 1] = 0.f;
                }
                return;
            }
            t0 = tb;
            n_tiles = te;
        }
    }
    const int mask_from = min(prefix + row0 + 1, ctx_len);  // subtiles reaching past this key are masked
    const int lo_mask_until = bounded ? row_first(min(q_len, row0 + kPfRows) - 1) : 0;  // subtiles starting below it too
    // a lane's last and first visible key, less the 4 keys its half of the wave is ahead by
    const int lim = min(ctx_len - 1, prefix + row0 + col) - 4 * half;
    const int lo_lim = (bounded ? row_first(row0 + col) : 0) - 4 * half;

    // ---- Q^T operands, staged through the (still empty) ring as whole rows: see prefill_mfma_kernel ----
    constexpr int QRPI = 64 / CPR;  // rows per wave-wide load
    const uint32_t q_stage = (uint32_t)wave * (32 * RB);
    // Head sizes between 128 and 256 (p.d < D, a multiple of 8): rows in memory are p.d elements long, the kernel's
    // rows D.  The 16-byte chunks past a row's end are requested from chunk 0 instead (any finite data does) and
    // Q^T holds zeros there, so they add nothing to S^T; what they add to O^T is never stored.
    const int64_t row_bytes = (int64_t)p.d * 2;          // a (token, head) row in memory
    const uint32_t real_chunks = (uint32_t)row_bytes / 16;  // its 16-byte chunks (<= CPR)
    const bool padded = real_chunks != (uint32_t)CPR;       // uniform
    auto real_chunk = [&](uint32_t chunk) PF_INLINE { return chunk < real_chunks ? chunk : 0u; };
    {
        const int lrow = lane / CPR, lslot = lane % CPR;
        const char *qb = reinterpret_cast<const char *>(a.q) + ((int64_t)a.q_starts[b] * p.hq + qh) * row_bytes;
#pragma unroll
        for (int i = 0; i < 32 / QRPI; ++i) {
            const int r = i * QRPI + lrow;
            const int64_t grow = min(row0 + r, q_len - 1);
            pf_dma16(lds_base + q_stage + (uint32_t)(i * QRPI * RB),
                     qb + grow * p.hq * row_bytes + real_chunk((uint32_t)(lslot ^ (r & (CPR - 1)))) * 16);
        }
    }
    // ---- slot tables (in flight together with the Q rows) ----
    const int64_t pool_rows = p.num_blocks * p.bs;  // >= 16, < 2^31 (the host checks)
    // Blocks that are not multiples of 16 keys long (one block per sequence): the last 16-key group of the pool's
    // last block would be loaded from past the end of the pool.  The assembly instances load that one group (at
    // most one per workgroup) from slot 0 instead and copy its existing rows from where they are, lane by lane,
    // when the stages that hold it are published (see prefill_asm_kernel).
    int edge_tile = -1, edge_group = 0, edge_rows = 0;
    int64_t edge_slot = 0;
    if (p.bs % 16 != 0) {  // (then bt_stride is 1)
        const int64_t bid = p.bt[(int64_t)b * p.bt_stride];
        const int n_keys = min(ctx_len, p.bs);
        const int key_last = (n_keys - 1) / 16 * 16;
        if (bid >= 0 && bid < p.num_blocks && bid * p.bs + key_last + 16 > pool_rows) {
            edge_tile = key_last / kWdKeys;
            edge_group = key_last / 16 % 2;
            edge_rows = n_keys - key_last;
            edge_slot = bid * p.bs + key_last;
        }
    }
    // (entries of kLookahead tiles past the workgroup's last one follow as groups of which nothing exists: the
    // loads run that far ahead and past the end, so that every wave issues the same loads per stage)
    constexpr int kLookahead = 6;
    // The tables hold the groups of kWdCapGroups / 2 tiles, counted from a first tile `base` (entry i: keys
    // 16 * (2 * base + i) ..).  They are filled for base = t0 here, and in the LONG instance again every kSegTiles
    // tiles: the loop below is left and entered again, which is free of side conditions because every pass of its
    // body leaves the state the next one starts from.  (The host launches the other instance when the whole block
    // table fits, or when a sliding window bounds the tiles a workgroup can see.)
    constexpr int kSegTiles = (CAP / 2 - kLookahead - 2) / kWdStages * kWdStages;  // (the loop starts in ring slot 0)
    auto fill_tables = [&](int base) PF_INLINE {
        const int n_rest = n_tiles - base;  // tiles still to run
        const int n_entries = min(2 * (n_rest + kLookahead), CAP);
        const int32_t *bt_seq = p.bt + (int64_t)b * p.bt_stride;
        int first_special = n_rest;
        for (int i = tid; i < n_entries; i += kPfThreads) {
            const int key = 16 * (2 * base + i), blk = key / p.bs;
            int64_t bid = -1;
            if (i < 2 * n_rest && blk < p.bt_stride) bid = bt_seq[blk];
            const bool present = bid >= 0 && bid < p.num_blocks;
            // rows of the group that exist: inside the context and inside the group's block (a block that is not
            // a multiple of 16 keys long is the only block of its sequence: what follows it is absent)
            const int rows = present ? min(min(max(ctx_len - key, 0), 16), (blk + 1) * p.bs - key) : 0;
            int64_t slot = present ? bid * p.bs + key % p.bs : 0;
            if (slot + 16 > pool_rows) slot = 0;  // (the group at the end of the pool: see edge_tile below)
            tab_a[i] = (int32_t)slot;
            tab_b[i] = (uint8_t)rows;
            if (rows < 16) first_special = min(first_special, i / 2);
        }
        if (tid < 4) { tab_a[CAP + tid] = 0; tab_b[CAP + tid] = 0; }
        if (2 * n_rest > CAP) first_special = min(first_special, CAP / 2);
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) first_special = min(first_special, __shfl_xor(first_special, d, 64));
        if (lane == 0) s_special[wave] = first_special;
    };
    // first tile (counted from the tables' base) with a row that does not exist; every tile from there on is checked
    // before it is published.  Valid behind a barrier after fill_tables.
    auto read_special = [&]() PF_INLINE {
        return __builtin_amdgcn_readfirstlane(min(min(s_special[0], s_special[1]), min(s_special[2], s_special[3])));
    };
    fill_tables(t0);
    pf_wait_loads<0>();
    X8 qreg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int slot = (2 * ks + half) ^ (col & (CPR - 1));
        const uint4 raw = *reinterpret_cast<const uint4 *>(s_mem + q_stage + col * RB + slot * 16);
        // scaled by softmax scale * log2(e) here, once per workgroup: S^T then comes out of the products in the
        // units of the exponential's argument (one more rounding of q to its 16-bit type)
        const X8 q8 = __builtin_bit_cast(X8, raw);
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = M::pack((float)q8[2 * e] * p.scale_log2, (float)q8[2 * e + 1] * p.scale_log2);
        if (padded && (uint32_t)(2 * ks + half) >= real_chunks) w[0] = w[1] = w[2] = w[3] = 0;  // past the row's end
        qreg[ks] = __builtin_bit_cast(X8, uint4{w[0], w[1], w[2], w[3]});
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(qreg[ks]));  // (product operands live in AGPRs)
    __syncthreads();  // the tables are complete and the staged rows have been read: the ring may overwrite them
    int first_special_rel = read_special();
    const int first_special = t0 + first_special_rel;

    // ---- loads: wave w fetches rows 8w .. 8w+7 of a stage's K and V, two rows (1 KiB) per direct load ----
    const int64_t tok_stride = (int64_t)p.hkv * row_bytes;
    const char *pool_k = reinterpret_cast<const char *>(p.k) + (int64_t)kvh * row_bytes;
    const char *pool_v = reinterpret_cast<const char *>(p.v) + (int64_t)kvh * row_bytes;
    const int ld_row = lane / CPR, ld_slot = lane % CPR;
    const int arow0 = (wave & 1) * 8 + ld_row;  // this lane's row inside its 16-key group for load 0; +2 per load
    // K: 16 consecutive rows read the same chunk -> chunk index swizzled by row % 16;
    // V: 4 consecutive rows each read 4 consecutive chunks -> swizzled by 4 * (row % 4)
    uint32_t lane_k[NL], lane_v[NL];
#pragma unroll
    for (int n = 0; n < NL; ++n) {
        const int r = arow0 + 2 * n;
        lane_k[n] = (uint32_t)(r * tok_stride) + real_chunk((uint32_t)(ld_slot ^ (r & 15))) * 16;
        lane_v[n] = (uint32_t)(r * tok_stride) + real_chunk((uint32_t)(ld_slot ^ ((r & 3) * 4))) * 16;
    }
    const uint32_t wave_rows = (uint32_t)wave * (8 * RB);  // the wave's rows inside a tensor of a stage
    // table entry of the wave's group of tile `tile` (>= 0, at most kLookahead - 1 past the last tile)
    const int wave_group = wave >> 1;
    auto entry_of = [&](int tile) PF_INLINE { return min(2 * (tile - t0) + wave_group, CAP); };
    // one tensor's rows of one tile into LDS at byte offset `dst` of s_mem (always NL direct loads)
    auto issue_rows = [&](const char *pool, const uint32_t (&lane_ofs)[NL], int tile, uint32_t dst) PF_INLINE {
        const int slot = __builtin_amdgcn_readfirstlane(tab_a[entry_of(tile)]);
        const uint64_t ofs = (uint64_t)(uint32_t)slot * (uint32_t)tok_stride;  // 32 x 32 -> 64 bits, scalar
        const char *base = pf_scalar_ptr(pool + ofs);
#pragma unroll
        for (int n = 0; n < NL; ++n) pf_dma16(lds_base + dst + n * 2 * RB, base, lane_ofs[n]);
    };
    // (ring slots are counted from the workgroup's first tile: the assembly loop starts in slot 0)
    auto stage_ofs = [&](int s) PF_INLINE { return (uint32_t)((s - t0) & (kWdStages - 1)) * STAGE; };
    auto issue_k = [&](int s) PF_INLINE { issue_rows(pool_k, lane_k, s + 1, stage_ofs(s) + wave_rows); };
    auto issue_v = [&](int s) PF_INLINE { issue_rows(pool_v, lane_v, s, stage_ofs(s) + TENSOR + wave_rows); };
    // The loop's loads: a direct load adds its immediate offset to the LDS address and to the global address alike,
    // so with the global side compensated in the per-lane offsets the four loads of a tensor share one LDS base
    // (one write of m0).
    uint32_t lane_kb[NL], lane_vb[NL];
#pragma unroll
    for (int n = 0; n < NL; ++n) {
        lane_kb[n] = lane_k[n] + (NL - 1 - n) * 2 * RB;
        lane_vb[n] = lane_v[n] + (NL - 1 - n) * 2 * RB;
    }
    const char *pool_kb = pool_k - (NL - 1) * 2 * RB, *pool_vb = pool_v - (NL - 1) * 2 * RB;
    // clear the rows this wave loaded that do not exist (after its loads have landed, before the barrier)
    auto clear_rows = [&](int tile, uint32_t dst) PF_INLINE {
        const int rows = tab_b[entry_of(tile)];
#pragma unroll
        for (int n = 0; n < NL; ++n)
            if (arow0 + 2 * n >= rows) *reinterpret_cast<uint4 *>(s_mem + dst + n * 2 * RB + lane * 16) = uint4{0, 0, 0, 0};
    };
    // the rows of the group at the end of the pool that this wave holds, copied from where they are
    auto edge_copy = [&](const char *pool, const uint32_t (&lane_ofs)[NL], uint32_t dst) PF_INLINE {
        if (wave_group != edge_group) return;
#pragma unroll
        for (int n = 0; n < NL; ++n)
            if (arow0 + 2 * n < edge_rows)
                *reinterpret_cast<uint4 *>(s_mem + dst + n * 2 * RB + lane * 16) =
                    *reinterpret_cast<const uint4 *>(pool + edge_slot * tok_stride + lane_ofs[n]);
    };
    auto fix_k = [&](int s) PF_INLINE {
        if (s + 1 >= first_special) clear_rows(s + 1, stage_ofs(s) + wave_rows);
        if (s + 1 == edge_tile) edge_copy(pool_k, lane_k, stage_ofs(s) + wave_rows);
    };
    auto fix_v = [&](int s) PF_INLINE {
        if (s >= first_special) clear_rows(s, stage_ofs(s) + TENSOR + wave_rows);
        if (s == edge_tile) edge_copy(pool_v, lane_v, stage_ofs(s) + TENSOR + wave_rows);
    };

    // ---- per-lane byte offsets of the operand reads inside a stage ----
    // K operand of k-step ks: key row `col`, chunk 2*ks + half; k-steps 8..15 are 256 bytes behind 0..7
    int k_ofs[KS / 2];
#pragma unroll
    for (int ks = 0; ks < KS / 2; ++ks) k_ofs[ks] = col * RB + (((2 * ks + half) ^ (col & 15)) * 16);
    // V^T transpose read (see prefill_mfma_kernel); d tiles 4..7 are 256 bytes behind 0..3
    const int g16 = lane >> 4, s16 = lane & 15;
    const int v_key = 4 * (g16 >> 1) + (s16 >> 2);
    int v_ofs[DT / 2];
#pragma unroll
    for (int dt = 0; dt < DT / 2; ++dt)
        v_ofs[dt] = TENSOR + v_key * RB + ((((4 * dt) ^ ((v_key & 3) * 4)) + 2 * (g16 & 1) + ((s16 & 3) >> 1)) * 16) + 8 * (s16 & 1);

    auto read_k = [&](int s, X8 (&ka)[KS]) PF_INLINE {  // K of tile s+1
        const uint32_t base = lds_base + stage_ofs(s);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint32_t adr = base + k_ofs[ks & 7];
            ka[ks] = __builtin_bit_cast(X8, *reinterpret_cast<const __attribute__((address_space(3))) uint4 *>(
                                                (const lds_char *)(size_t)adr + (ks >> 3) * 256));
        }
    };
    // V^T of keys 16*step .. +16 of tile s, d tile dt (two transposing reads)
    auto read_v_one = [&](int s, int step, int dt, X8 &dst) PF_INLINE {
        const lds_char *at = (const lds_char *)(size_t)(lds_base + stage_ofs(s) + v_ofs[dt & 3]) + (dt >> 2) * 256 + 16 * step * RB;
        const X4 lo = __builtin_bit_cast(X4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((pa_s16x4 __attribute__((address_space(3))) *)at));
        const X4 hi = __builtin_bit_cast(
            X4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((pa_s16x4 __attribute__((address_space(3))) *)(at + 8 * RB)));
#pragma unroll
        for (int e = 0; e < 4; ++e) { dst[e] = lo[e]; dst[4 + e] = hi[e]; }
    };
    // mask of S^T of the subtile that starts at key_base: value i of a lane is key 8*(i/4) + i%4 (+ 4*half)
    auto mask_s = [&](f32x16 &s, int key_base) PF_INLINE {
        const int limit = lim - key_base, first = lo_lim - key_base;
        if (bounded) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int idx = 8 * (i >> 2) + (i & 3);
                s[i] = idx <= limit && idx >= first ? s[i] : -INFINITY;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) s[i] = 8 * (i >> 2) + (i & 3) <= limit ? s[i] : -INFINITY;
        }
    };
    auto max_piece = [&](f32x16 &s, int h, float &mx) PF_INLINE {
        asm volatile("" : "+v"(s));
        float m = fmaxf(s[8 * h], s[8 * h + 1]);
#pragma unroll
        for (int i = 2; i < 8; ++i) m = fmaxf(m, s[8 * h + i]);
        if (h == 0) {
            mx = m;
        } else {
            m = fmaxf(m, mx);
            const uint32_t u = __builtin_bit_cast(uint32_t, m);
            const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
            mx = fmaxf(__builtin_bit_cast(float, (uint32_t)sw[0]), __builtin_bit_cast(float, (uint32_t)sw[1]));
        }
        asm volatile("" : "+v"(mx));
    };

    // ---- fill the ring: K of tile t0 (the K part of stage t0-1), then stages t0 .. t0+2 ----
    issue_k(t0 - 1);
    issue_k(t0); issue_v(t0);
    issue_k(t0 + 1); issue_v(t0 + 1);
    issue_k(t0 + 2); issue_v(t0 + 2);
    pf_wait_loads<4 * NL>();  // K of t0 and stage t0 have landed
    fix_k(t0 - 1);
    fix_k(t0); fix_v(t0);
    __syncthreads();

    f32x16 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
    // S^T is kept relative to the row's reference maximum (see prefill_mfma_kernel): the first product of a
    // subtile accumulates onto ref = minus the reference in all 16 registers, the exponentials take S^T as it
    // is, mx is relative too.
    f32x16 ref;
#pragma unroll
    for (int i = 0; i < 16; ++i) ref[i] = 0.f;
    float l_run = 0.f, mx = kNegBig;
    X8 ka[KS], va0[DT / 2];
    f32x16 sb0;  // S^T of the first subtile

    // ---- first subtile: S^T, mask, row maximum; K operands of the second; V^T of the first k-step ----
    read_k(t0 - 1, ka);
    PF_FENCE();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) sb0 = M::mma(ka[ks], qreg[ks], ks == 0 ? ref : sb0);
    PF_FENCE();
    read_k(t0, ka);
    PF_FENCE();
    if (32 * (t0 + 1) > mask_from || 32 * t0 < lo_mask_until) mask_s(sb0, 32 * t0);
    max_piece(sb0, 0, mx);
    max_piece(sb0, 1, mx);
    PF_FENCE();
    // every wave has read K of tile t0: its slot takes stage t0+3
    __builtin_amdgcn_s_waitcnt((15) | (7 << 4) | (0 << 8) | (3 << 14));  // lgkmcnt(0)
    __syncthreads();
    issue_k(t0 + 3); issue_v(t0 + 3);
    PF_FENCE();

    {
        // The subtile loop as scheduled assembly (prefill_d256_loop.inc).  S^T of the first subtile becomes relative
        // to its row maximum, which is the reference from here on.  Without lower bounds every row has seen key
        // 0; with them a row may have seen nothing yet: its reference stays unset (thr = a large negative number
        // instead of the slack) until a maximum of visible keys arrives (see prefill_asm_kernel).  The loop takes
        // the first half of the first V^T operands read.
        static_assert(kWdStages == 4 && kWdKeys == 32 && CAP == 2 * 3072 && kSegTiles % kWdStages == 0,
                      "the assembly loop is written for this shape");
        const bool seen = mx > kNegBig;
        const float m0 = seen ? mx : 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            sb0[i] -= m0;
            ref[i] = -m0;
        }
        if (seen) mx = 0.f;
        float thr = seen ? kPfSlack : kNegBig;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) read_v_one(t0, 0, dt, va0[dt]);
        auto uni = [](int v) PF_INLINE { return __builtin_amdgcn_readfirstlane(v); };
        const uint32_t tab_a_w = lds_base + kRingBytes + 4 * wave_group;
        const uint32_t tab_b_w = lds_base + kRingBytes + kTabEntries * 4 + wave_group;
        const uint32_t mask_from_u = (uint32_t)uni(mask_from);
        const uint32_t m0w = lds_base + wave_rows, lane16 = (uint32_t)lane * 16, arow_u = (uint32_t)arow0;
        uint32_t kad[KS / 2], vad[DT / 2];
#pragma unroll
        for (int ks = 0; ks < KS / 2; ++ks) kad[ks] = lds_base + k_ofs[ks];
#pragma unroll
        for (int dt = 0; dt < DT / 2; ++dt) vad[dt] = lds_base + v_ofs[dt];
        const uint64_t pk = reinterpret_cast<uint64_t>(pool_kb), pv = reinterpret_cast<uint64_t>(pool_vb);
        const uint32_t pklo = uni((uint32_t)pk), pkhi = uni((uint32_t)(pk >> 32));
        const uint32_t pvlo = uni((uint32_t)pv), pvhi = uni((uint32_t)(pv >> 32));
        const uint32_t stride = (uint32_t)tok_stride;
        const uint32_t edge_slot_u = (uint32_t)uni((int)edge_slot), edge_rows_u = (uint32_t)uni(edge_rows);
        const float slack = kPfSlack, neg_big = kNegBig;
#define WD_NOTHING
#define WD_LO_OUT , [thr0] "+&v"(thr), [slo] "+&s"(s_lo)
#define WD_LO_IN , [lo0] "v"(lo_lim), [negbig] "s"(neg_big)
        constexpr bool BF = std::is_same<T, pa_bf16>::value;
        const int n_tiles_u = uni(n_tiles);
        for (int base = uni(t0);;) {  // one pass per fill of the tables (uniform control flow, stated to the compiler)
            const int n_seg = uni(min(n_tiles_u - base, kSegTiles));
            int n_left = uni(n_seg - 1);  // tiles after the current one
            uint32_t s_t = 4, s_p = 1;    // (the loop counts tiles from the tables' base)
            int s_rem = uni(mask_from - kWdKeys * base);
            int s_lo = uni(lo_mask_until - kWdKeys * base);
            const uint32_t sp_lo = (uint32_t)uni(max(first_special_rel - 1, 0));
            // (only the waves that load rows of the group at the end of the pool see its tile)
            const uint32_t edge_tile_u = (uint32_t)uni(wave_group == edge_group && edge_tile >= base ? edge_tile - base : -1);
            if constexpr (LO) {
                if constexpr (BF) {
                    asm volatile(WD_LOOP_ASM_BF16_LO WD_LOOP_OPERANDS(WD_LO_OUT, WD_LO_IN));
                } else {
                    asm volatile(WD_LOOP_ASM_F16_LO WD_LOOP_OPERANDS(WD_LO_OUT, WD_LO_IN));
                }
            } else {
                (void)thr; (void)s_lo; (void)neg_big;
                if constexpr (BF) {
                    asm volatile(WD_LOOP_ASM_BF16 WD_LOOP_OPERANDS(WD_NOTHING, WD_NOTHING));
                } else {
                    asm volatile(WD_LOOP_ASM_F16 WD_LOOP_OPERANDS(WD_NOTHING, WD_NOTHING));
                }
            }
            if constexpr (!LONG) break;
            base = uni(base + n_seg);
            if (base >= n_tiles_u) break;
            __syncthreads();  // every wave has left the loop: nobody reads the tables
            fill_tables(base);
            __syncthreads();
            first_special_rel = read_special();
        }
#undef WD_NOTHING
#undef WD_LO_OUT
#undef WD_LO_IN
    }
    pf_wait_loads<0>();  // (loads of the stages past the last tile: nothing may arrive after the workgroup has ended)

    // ---- normalise and write: lane owns row (row0+col), d = 32*dt + 4*half + 8*g + j ----
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int row = row0 + col;
    if (!live || row >= q_len) return;
    if constexpr (LO) {
        if (n_splits > 1) {
            // a piece: the row's reference maximum, sum and unnormalised O^T go to the workspace (through a multiply
            // by a one the compiler cannot see through: see prefill_asm_kernel)
            float one = 1.f;
            asm volatile("" : "+v"(one));
            const int64_t at = (((int64_t)a.q_starts[b] + row) * p.hq + qh) * n_splits + piece;
            float *po = a.part_o + at * D + 4 * half;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    *reinterpret_cast<float4 *>(po + 32 * dt + 8 * g) =
                        float4{o[dt][4 * g] * one, o[dt][4 * g + 1] * one, o[dt][4 * g + 2] * one, o[dt][4 * g + 3] * one};
            if (half == 0) {
                a.part_ml[at * 2] = l_tot > 0.f ? -(ref[0] * one) : kNegBig;  // (a row that saw no key has no maximum)
                a.part_ml[at * 2 + 1] = l_tot;
            }
            return;
        }
    }
    T *orow = reinterpret_cast<T *>(a.out) + (((int64_t)a.q_starts[b] + row) * p.hq + qh) * p.d;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            uint2 w;
            w.x = M::pack(o[dt][4 * g] * inv, o[dt][4 * g + 1] * inv);
            w.y = M::pack(o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv);
            // (p.d is a multiple of 8: the four elements lie on one side of the row's end)
            if (32 * dt + 4 * half + 8 * g < p.d) *reinterpret_cast<uint2 *>(orow + 32 * dt + 4 * half + 8 * g) = w;
        }
}

// nullptr unless the element type has this kernel; `lower_bounds`: the instance for sliding windows and per-row
// first keys; `long_table`: the instance that fills its tables more than once
prefill_mfma_fn pa_prefill_d256_kernel(int dtype, bool lower_bounds, bool long_table);
prefill_mfma_fn pa_prefill_d256_kernel_long(int dtype, bool lower_bounds);

}  // namespace pa_decode_detail
