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
// A group must lie inside one pool block: block sizes that are multiples of 16, or one block per sequence.
// CHECKED: the instance for block sizes that are not multiples of 16 (one block per sequence), where a sequence's
// last group can reach past the end of the pool: such a group is fetched lane by lane with clamped rows; its
// subtile loop is compiled code with the instruction order written out and fenced.  With blocks of a multiple of
// 16 keys no group can reach past the pool, and the subtile loop is scheduled assembly (ASM; prefill_d256_loop.inc,
// written by gen_prefill_loop_d256.py), in one instance without and one with lower bounds (LO: sliding window,
// per-row first keys).
// Every wave runs every subtile of the workgroup, with the masks applied where needed: a wave past its last
// visible key multiplies exact zeros.
#pragma once
#include "prefill_mfma.h"
#include "prefill_d256_loop.inc"

namespace pa_decode_detail {

constexpr int kWdKeys = 32;          // keys per ring stage
constexpr int kWdStages = 4;
constexpr int kWdTasks = kPfWaves;   // tasks (32 query rows of one head) per workgroup: one per wave
constexpr int kWdCapGroups = 6144;   // 16-key groups the slot tables hold: contexts of up to 98304 keys

template <typename T, bool CHECKED, bool ASM, bool LO>
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
    const int n_groups = gridDim.y, n_seqs = gridDim.z;
    const int lin = blockIdx.y + n_groups * blockIdx.z;
    const bool group_major = a.ctx_lens[0] - a.q_lens[0] < a.q_lens[0];
    const int group = group_major ? n_groups - 1 - lin / n_seqs : (int)blockIdx.y;
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
    const int n_tiles = (wg_keys + kWdKeys - 1) / kWdKeys;  // >= 1
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
    const int t0 = wg_first_key / kWdKeys;  // first tile of the workgroup (< n_tiles)
    const int mask_from = min(prefix + row0 + 1, ctx_len);  // subtiles reaching past this key are masked
    const int lo_mask_until = bounded ? row_first(min(q_len, row0 + kPfRows) - 1) : 0;  // subtiles starting below it too
    // a lane's last and first visible key, less the 4 keys its half of the wave is ahead by
    const int lim = min(ctx_len - 1, prefix + row0 + col) - 4 * half;
    const int lo_lim = (bounded ? row_first(row0 + col) : 0) - 4 * half;

    // ---- Q^T operands, staged through the (still empty) ring as whole rows: see prefill_mfma_kernel ----
    constexpr int QRPI = 64 / CPR;  // rows per wave-wide load
    const uint32_t q_stage = (uint32_t)wave * (32 * RB);
    {
        const int lrow = lane / CPR, lslot = lane % CPR;
        const char *qb = reinterpret_cast<const char *>(a.q) + ((int64_t)a.q_starts[b] * p.hq + qh) * RB;
#pragma unroll
        for (int i = 0; i < 32 / QRPI; ++i) {
            const int r = i * QRPI + lrow;
            const int64_t grow = min(row0 + r, q_len - 1);
            pf_dma16(lds_base + q_stage + (uint32_t)(i * QRPI * RB), qb + grow * p.hq * RB + ((lslot ^ (r & (CPR - 1))) * 16));
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
    if (ASM && p.bs % 16 != 0) {  // (then bt_stride is 1)
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
    const int n_entries = min(2 * (n_tiles + kLookahead), CAP);
    {
        const int32_t *bt_seq = p.bt + (int64_t)b * p.bt_stride;
        int first_special = n_tiles;
        for (int i = tid; i < n_entries; i += kPfThreads) {
            const int key = 16 * i, blk = key / p.bs;
            int64_t bid = -1;
            if (i < 2 * n_tiles && blk < p.bt_stride) bid = bt_seq[blk];
            const bool present = bid >= 0 && bid < p.num_blocks;
            // rows of the group that exist: inside the context and inside the group's block (a block that is not
            // a multiple of 16 keys long is the only block of its sequence: what follows it is absent)
            const int rows = present ? min(min(max(ctx_len - key, 0), 16), (blk + 1) * p.bs - key) : 0;
            int64_t slot = present ? bid * p.bs + key % p.bs : 0;
            if (ASM && slot + 16 > pool_rows) slot = 0;  // (the group at the end of the pool: see edge_tile below)
            tab_a[i] = (int32_t)slot;
            tab_b[i] = (uint8_t)rows;
            if (rows < 16) first_special = min(first_special, i / 2);
        }
        if (tid < 4) { tab_a[CAP + tid] = 0; tab_b[CAP + tid] = 0; }
        if (2 * n_tiles > CAP) first_special = min(first_special, CAP / 2);
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) first_special = min(first_special, __shfl_xor(first_special, d, 64));
        if (lane == 0) s_special[wave] = first_special;
    }
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
        qreg[ks] = __builtin_bit_cast(X8, uint4{w[0], w[1], w[2], w[3]});
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(qreg[ks]));  // (product operands live in AGPRs)
    __syncthreads();  // the tables are complete and the staged rows have been read: the ring may overwrite them
    // first tile with a row that does not exist; every tile from there on is checked before it is published
    const int first_special =
        __builtin_amdgcn_readfirstlane(min(min(s_special[0], s_special[1]), min(s_special[2], s_special[3])));

    // ---- loads: wave w fetches rows 8w .. 8w+7 of a stage's K and V, two rows (1 KiB) per direct load ----
    const int64_t tok_stride = (int64_t)p.hkv * RB;
    const char *pool_k = reinterpret_cast<const char *>(p.k) + (int64_t)kvh * RB;
    const char *pool_v = reinterpret_cast<const char *>(p.v) + (int64_t)kvh * RB;
    const int ld_row = lane / CPR, ld_slot = lane % CPR;
    const int arow0 = (wave & 1) * 8 + ld_row;  // this lane's row inside its 16-key group for load 0; +2 per load
    // K: 16 consecutive rows read the same chunk -> chunk index swizzled by row % 16;
    // V: 4 consecutive rows each read 4 consecutive chunks -> swizzled by 4 * (row % 4)
    uint32_t lane_k[NL], lane_v[NL];
#pragma unroll
    for (int n = 0; n < NL; ++n) {
        const int r = arow0 + 2 * n;
        lane_k[n] = (uint32_t)(r * tok_stride) + (uint32_t)((ld_slot ^ (r & 15)) * 16);
        lane_v[n] = (uint32_t)(r * tok_stride) + (uint32_t)((ld_slot ^ ((r & 3) * 4)) * 16);
    }
    const uint32_t wave_rows = (uint32_t)wave * (8 * RB);  // the wave's rows inside a tensor of a stage
    // table entry of the wave's group of tile `tile` (>= 0, at most kLookahead - 1 past the last tile)
    const int wave_group = wave >> 1;
    auto entry_of = [&](int tile) PF_INLINE { return min(2 * tile + wave_group, CAP); };
    // one tensor's rows of one tile into LDS at byte offset `dst` of s_mem (always NL direct loads)
    auto issue_rows = [&](const char *pool, const uint32_t (&lane_ofs)[NL], int chunk_swz_mask, int tile, uint32_t dst) PF_INLINE {
        const int slot = __builtin_amdgcn_readfirstlane(tab_a[entry_of(tile)]);
        if (!CHECKED || __builtin_expect((int64_t)slot + 16 <= pool_rows, 1)) {
            const uint64_t ofs = (uint64_t)(uint32_t)slot * (uint32_t)tok_stride;  // 32 x 32 -> 64 bits, scalar
            const char *base = pf_scalar_ptr(pool + ofs);
#pragma unroll
            for (int n = 0; n < NL; ++n) pf_dma16(lds_base + dst + n * 2 * RB, base, lane_ofs[n]);
        } else {
            // the group reaches past the end of the pool (its last rows do not exist): such lanes fetch the
            // pool's last row instead; the rows are cleared before the stage is published
#pragma unroll
            for (int n = 0; n < NL; ++n) {
                const int r = arow0 + 2 * n;
                const int64_t row = min((int64_t)slot + r, pool_rows - 1);
                const int swz = chunk_swz_mask == 15 ? (r & 15) : (r & 3) * 4;
                pf_dma16(lds_base + dst + n * 2 * RB, pool + row * tok_stride + ((ld_slot ^ swz) * 16));
            }
        }
    };
    // (ring slots are counted from the workgroup's first tile: the assembly loop starts in slot 0)
    auto stage_ofs = [&](int s) PF_INLINE { return (uint32_t)((s - t0) & (kWdStages - 1)) * STAGE; };
    auto issue_k = [&](int s) PF_INLINE { issue_rows(pool_k, lane_k, 15, s + 1, stage_ofs(s) + wave_rows); };
    auto issue_v = [&](int s) PF_INLINE { issue_rows(pool_v, lane_v, 3, s, stage_ofs(s) + TENSOR + wave_rows); };
    // The same inside the loop, trimmed: the two table entries are read one subtile ahead (pre_k, pre_v), and the
    // eight loads of a stage are one block of instructions.  A direct load adds its immediate offset to the LDS
    // address and to the global address alike, so with the global side compensated in the per-lane offsets the
    // four loads of a tensor share one LDS base (one write of m0).
    int pre_k = 0, pre_v = 0;
    auto prefetch_entries = [&](int s) PF_INLINE { pre_k = tab_a[entry_of(s + 1)]; pre_v = tab_a[entry_of(s)]; };
    uint32_t lane_kb[NL], lane_vb[NL];
#pragma unroll
    for (int n = 0; n < NL; ++n) {
        lane_kb[n] = lane_k[n] + (NL - 1 - n) * 2 * RB;
        lane_vb[n] = lane_v[n] + (NL - 1 - n) * 2 * RB;
    }
    const char *pool_kb = pool_k - (NL - 1) * 2 * RB, *pool_vb = pool_v - (NL - 1) * 2 * RB;
    const int slot_max = (int)max(pool_rows - 16, (int64_t)-1);  // last slot a whole group can start at
    auto dma_one = [&](uint32_t dst, const char *base, uint32_t lane_ofs, int n) PF_INLINE {
        if (n == 0) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %1 offset:0" : : "s"(dst), "s"(base), "v"(lane_ofs) : "memory", "m0");
        if (n == 1) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %1 offset:1024" : : "s"(dst), "s"(base), "v"(lane_ofs) : "memory", "m0");
        if (n == 2) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %1 offset:2048" : : "s"(dst), "s"(base), "v"(lane_ofs) : "memory", "m0");
        if (n == 3) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %1 offset:3072" : : "s"(dst), "s"(base), "v"(lane_ofs) : "memory", "m0");
    };
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
        if (ASM && s + 1 == edge_tile) edge_copy(pool_k, lane_k, stage_ofs(s) + wave_rows);
    };
    auto fix_v = [&](int s) PF_INLINE {
        if (s >= first_special) clear_rows(s, stage_ofs(s) + TENSOR + wave_rows);
        if (ASM && s == edge_tile) edge_copy(pool_v, lane_v, stage_ofs(s) + TENSOR + wave_rows);
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
    auto read_v = [&](int s, int step, X8 (&va)[DT]) PF_INLINE {  // V^T of keys 16*step .. +16 of tile s
        const uint32_t base = lds_base + stage_ofs(s);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const lds_char *at = (const lds_char *)(size_t)(base + v_ofs[dt & 3]) + (dt >> 2) * 256 + 16 * step * RB;
            const X4 lo = __builtin_bit_cast(X4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((pa_s16x4 __attribute__((address_space(3))) *)at));
            const X4 hi = __builtin_bit_cast(
                X4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((pa_s16x4 __attribute__((address_space(3))) *)(at + 8 * RB)));
#pragma unroll
            for (int e = 0; e < 4; ++e) { va[dt][e] = lo[e]; va[dt][4 + e] = hi[e]; }
        }
    };
    // the same reads one operand at a time (the loop spreads them between the products)
    auto read_k_one = [&](int s, int ks, X8 &dst) PF_INLINE {
        const uint32_t adr = lds_base + stage_ofs(s) + k_ofs[ks & 7];
        dst = __builtin_bit_cast(X8, *reinterpret_cast<const __attribute__((address_space(3))) uint4 *>(
                                         (const lds_char *)(size_t)adr + (ks >> 3) * 256));
    };
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
    // is, mx is relative too; m_thr is what mx must exceed for a rescale (kNegBig until the row has seen a key).
    f32x16 ref;
#pragma unroll
    for (int i = 0; i < 16; ++i) ref[i] = 0.f;
    float m_thr = kNegBig, l_run = 0.f, mx = kNegBig;
    X8 ka[KS], va0[DT], va1[DT];
    f32x16 sb[2];  // S^T of the current and of the next subtile, swapping roles every subtile

    // ---- first subtile: S^T, mask, row maximum; K operands of the second; V^T of the first k-step ----
    read_k(t0 - 1, ka);
    PF_FENCE();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) sb[0] = M::mma(ka[ks], qreg[ks], ks == 0 ? ref : sb[0]);
    PF_FENCE();
    read_k(t0, ka);
    PF_FENCE();
    if (32 * (t0 + 1) > mask_from || 32 * t0 < lo_mask_until) mask_s(sb[0], 32 * t0);
    max_piece(sb[0], 0, mx);
    max_piece(sb[0], 1, mx);
    PF_FENCE();
    // every wave has read K of tile t0: its slot takes stage t0+3
    __builtin_amdgcn_s_waitcnt((15) | (7 << 4) | (0 << 8) | (3 << 14));  // lgkmcnt(0)
    __syncthreads();
    issue_k(t0 + 3); issue_v(t0 + 3);
    prefetch_entries(t0 + 4);
    PF_FENCE();

    // One subtile g (= tile g, stage g); PAR = parity of g - t0: which S^T buffer is the current one.
    auto subtile = [&](int g, auto par_tag) PF_INLINE {
        constexpr int PAR = decltype(par_tag)::value ? 1 : 0;
        f32x16 &s = sb[PAR];
        f32x16 &s_nx = sb[PAR ^ 1];
        const bool mask_next = 32 * (g + 2) > mask_from || 32 * (g + 1) < lo_mask_until;
        uint32_t pp[8];
        float sum = 0.f;
        // exponentials of S^T values 2*j, 2*j+1, packed as a P^T operand word
        auto exp_piece = [&](int j) PF_INLINE {
            const float p0 = __builtin_amdgcn_exp2f(s[2 * j]);
            const float p1 = __builtin_amdgcn_exp2f(s[2 * j + 1]);
            sum += p0 + p1;
            uint32_t w = M::pack(p0, p1);
            asm volatile("" : "+v"(w), "+v"(sum));
            pp[j] = w;
        };
        // ---- the row maximum outgrew its reference by more than the slack (rare): rescale ----
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(mx > m_thr) != 0, 0)) {
            // the reference moves by delta: up to the new maximum, or - for a row that had seen no key so far
            // (sum and accumulators still zero) - to its first maximum, whatever its sign
            const bool unset = m_thr == kNegBig;
            const bool seen = mx > kNegBig;
            const float delta = unset ? (seen ? mx : 0.f) : fmaxf(mx, 0.f);
            const float alpha = unset ? 1.f : __builtin_amdgcn_exp2f(-delta);
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                ref[i] -= delta;
                s[i] -= delta;  // formed against the old reference
            }
            mx -= delta;
            if (seen) m_thr = kPfSlack;
        }
        PF_FENCE();
        // ---- (a) S^T of subtile g+1, with the exponentials of subtile g between the products ----
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            s_nx = M::mma(ka[ks], qreg[ks], ks == 0 ? ref : s_nx);
            PF_FENCE();
            // V^T of this subtile: the first k-step's (consumed in (b)) behind the first eight products, the second's
            // (consumed in (c)) behind the others
            if (ks < 8) read_v_one(g, 0, ks, va0[ks]);
            else read_v_one(g, 1, ks - 8, va1[ks - 8]);
            if (ks & 1) exp_piece(ks >> 1);
            PF_FENCE();
        }
        // ---- publish stage g+1; the loads of stage g+4 go into the slot of stage g (every read of it is done) ----
        pf_wait_loads<4 * NL>();  // loads in flight, oldest first: stages g+1, g+2, g+3
        fix_k(g + 1); fix_v(g + 1);
        __builtin_amdgcn_s_waitcnt((15) | (7 << 4) | (0 << 8) | (3 << 14));  // lgkmcnt(0): this wave's reads of stage g
        __syncthreads();
        // the loads of stage g+4, one behind each product of (b); a group that reaches past the end of the pool
        // takes the per-lane path here instead
        const int slot_k = __builtin_amdgcn_readfirstlane(pre_k), slot_v = __builtin_amdgcn_readfirstlane(pre_v);
        const bool fast = !CHECKED || max(slot_k, slot_v) <= slot_max;
        const uint32_t dst_k = lds_base + stage_ofs(g + 4) + wave_rows, dst_v = dst_k + TENSOR;
        const char *bk = pf_scalar_ptr(pool_kb + (uint64_t)(uint32_t)slot_k * (uint32_t)tok_stride);
        const char *bv = pf_scalar_ptr(pool_vb + (uint64_t)(uint32_t)slot_v * (uint32_t)tok_stride);
        if (CHECKED && __builtin_expect(!fast, 0)) { issue_k(g + 4); issue_v(g + 4); }
        prefetch_entries(g + 5);
        PF_FENCE();
        // ---- (b) O^T += V^T . P^T, first k-step ----
        {
            const X8 pb = __builtin_bit_cast(X8, uint4{pp[0], pp[1], pp[2], pp[3]});
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                o[dt] = M::mma(va0[dt], pb, o[dt]);
                PF_FENCE();
                if (fast) dma_one(dt < 4 ? dst_k : dst_v, dt < 4 ? bk : bv, dt < 4 ? lane_kb[dt & 3] : lane_vb[dt & 3], dt & 3);
                read_k_one(g + 1, dt, ka[dt]);  // K of subtile g+2 (k-steps 0..7 here, 8..15 in (c)): consumed in (a) of g+1
                PF_FENCE();
            }
        }
        if (mask_next) mask_s(s_nx, 32 * (g + 1));
        PF_FENCE();
        // ---- (c) second k-step, with the next subtile's row maximum ----
        {
            const X8 pb = __builtin_bit_cast(X8, uint4{pp[4], pp[5], pp[6], pp[7]});
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                o[dt] = M::mma(va1[dt], pb, o[dt]);
                PF_FENCE();
                read_k_one(g + 1, 8 + dt, ka[8 + dt]);
                if (dt == 1) max_piece(s_nx, 0, mx);
                if (dt == 3) max_piece(s_nx, 1, mx);
                PF_FENCE();
            }
        }
        l_run += sum;
        PF_FENCE();
    };
    if constexpr (ASM) {
        // The subtile loop as scheduled assembly (prefill_d256_loop.inc).  S^T of the first subtile becomes relative
        // to its row maximum, which is the reference from here on.  Without lower bounds every row has seen key
        // 0; with them a row may have seen nothing yet: its reference stays unset (thr = a large negative number
        // instead of the slack) until a maximum of visible keys arrives (see prefill_asm_kernel).  The loop takes
        // the first half of the first V^T operands read.
        static_assert(!CHECKED && kWdStages == 4 && kWdKeys == 32 && CAP == 2 * 3072, "the assembly loop is written for this shape");
        const bool seen = mx > kNegBig;
        const float m0 = seen ? mx : 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            sb[0][i] -= m0;
            ref[i] = -m0;
        }
        if (seen) mx = 0.f;
        float thr = seen ? kPfSlack : kNegBig;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) read_v_one(t0, 0, dt, va0[dt]);
        f32x16 &sb0 = sb[0];
        auto uni = [](int v) PF_INLINE { return __builtin_amdgcn_readfirstlane(v); };
        int n_left = uni(n_tiles - t0 - 1);  // tiles after the current one
        uint32_t s_t = (uint32_t)uni(t0 + 4), s_p = (uint32_t)uni(t0 + 1);
        int s_rem = uni(mask_from - kWdKeys * t0);
        int s_lo = uni(lo_mask_until - kWdKeys * t0);
        const uint32_t tab_a_w = lds_base + kRingBytes + 4 * wave_group;
        const uint32_t tab_b_w = lds_base + kRingBytes + kTabEntries * 4 + wave_group;
        const uint32_t sp_lo = (uint32_t)uni(max(first_special - 1, 0)), mask_from_u = (uint32_t)uni(mask_from);
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
        // (only the waves that load rows of the group at the end of the pool see its tile)
        const uint32_t edge_tile_u = (uint32_t)uni(wave_group == edge_group ? edge_tile : -1);
        const uint32_t edge_slot_u = (uint32_t)uni((int)edge_slot), edge_rows_u = (uint32_t)uni(edge_rows);
        const float slack = kPfSlack, neg_big = kNegBig;
#define WD_NOTHING
#define WD_LO_OUT , [thr0] "+&v"(thr), [slo] "+&s"(s_lo)
#define WD_LO_IN , [lo0] "v"(lo_lim), [negbig] "s"(neg_big)
        constexpr bool BF = std::is_same<T, pa_bf16>::value;
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
#undef WD_NOTHING
#undef WD_LO_OUT
#undef WD_LO_IN
    } else {
        for (int g = t0; g < n_tiles; g += 2) {
            subtile(g, PfBool<false>{});
            if (g + 1 < n_tiles) subtile(g + 1, PfBool<true>{});
        }
    }
    pf_wait_loads<0>();  // (loads of the stages past the last tile: nothing may arrive after the workgroup has ended)

    // ---- normalise and write: lane owns row (row0+col), d = 32*dt + 4*half + 8*g + j ----
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int row = row0 + col;
    if (!live || row >= q_len) return;
    T *orow = reinterpret_cast<T *>(a.out) + (((int64_t)a.q_starts[b] + row) * p.hq + qh) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            uint2 w;
            w.x = M::pack(o[dt][4 * g] * inv, o[dt][4 * g + 1] * inv);
            w.y = M::pack(o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv);
            *reinterpret_cast<uint2 *>(orow + 32 * dt + 4 * half + 8 * g) = w;
        }
}

// nullptr unless the element type has this kernel
prefill_mfma_fn pa_prefill_d256_kernel(int dtype, bool checked, bool lower_bounds);

}  // namespace pa_decode_detail
