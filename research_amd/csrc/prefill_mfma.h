// Causal prefill attention over a paged context on the gfx950 matrix cores
// (bf16 / fp16, head_dim 32, 64 or 128).
//
// Shape of the computation (flash-attention style, everything transposed so
// that a query row lives in a lane):
//   S^T[key][row] = K[key][:] . Q[row][:]      v_mfma_f32_32x32x16, A = K tile, B = Q^T
//   O^T[d][row]  += V^T[d][key] . P^T[key][row]  A = V^T (LDS transpose read), B = P^T
// In the 32x32 result layout a lane owns column (lane % 32) = one query row and
// 16 of the 32 keys (or d values), so the softmax statistics of a row are
// in-lane except for one exchange between the two half-waves, and rescaling
// O^T by a per-row factor is a plain per-lane multiply.  The 16 S^T values a
// lane holds for a 32-key subtile are, in register order, exactly the P^T
// operand of the two k-steps of the second product once V^T uses the same key
// order, so P never moves between lanes.
//
// Work split
//   workgroup = 4 waves, one per SIMD; a wave owns two 32-row column tiles (tasks): 64 query rows of one or two
//   (row block, query head of the kv head) pairs, so every K / V^T operand it reads from LDS feeds two products.
//   Accumulators (128 registers), Q^T operands (64) and S^T (2 x 32) fill the 512 registers a lane has, which is
//   why there is one wave per SIMD and why the instruction order below is written out: nothing but the wave's
//   own order hides latency.  The 8 tasks of a workgroup are consecutive (row block, head) pairs of one kv
//   head, so they share every K/V tile (GQA packing: K/V are fetched once per kv head, not per query head).
//   grid.x = kv head (fastest): with 8 XCDs a kv head's K/V stays in one XCD's L2 while all sequences and row
//   blocks that share prefix blocks re-read it.
//   K/V tiles of 64 keys go global -> LDS directly (global_load_lds, 16 bytes per lane, no staging registers)
//   into a ring of four stages: the loads of tile t+3 are in flight while tile t is multiplied, and there is
//   one barrier per tile.  A direct load puts lane i's 16 bytes at base + 16*i, so rows cannot be padded;
//   instead each lane fetches the chunk that belongs at its position under an XOR swizzle of the chunk index by
//   the row, chosen so that the 128-bit operand reads (16 rows, same chunk) and the transpose reads (4 rows x
//   64 bytes) each touch all 64 banks once.
#pragma once
#include "decode_impl.h"

namespace pa_decode_detail {

typedef float f32x16 __attribute__((ext_vector_type(16)));

typedef short pa_s16x4 __attribute__((ext_vector_type(4)));
// LDS transpose read of 16-bit elements: inside each group of 16 lanes, lane i
// receives element (i % 4) of the 8 bytes addressed by lanes i/4, i/4+4, i/4+8, i/4+12.
__device__ __forceinline__ pa_s16x4 pa_tr16_b64(const void *lds) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((pa_s16x4 __attribute__((address_space(3))) *)lds);
}

template <typename T> struct Mfma16;
template <> struct Mfma16<pa_bf16> {
    typedef __bf16 x8 __attribute__((ext_vector_type(8)));
    typedef __bf16 x4 __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ f32x16 mma(x8 a, x8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ x4 tr_read(const void *lds) {
        return __builtin_bit_cast(x4, pa_tr16_b64(lds));
    }
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) { return Pk16<pa_bf16>::pack(lo, hi); }
};
template <> struct Mfma16<pa_f16> {
    typedef _Float16 x8 __attribute__((ext_vector_type(8)));
    typedef _Float16 x4 __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ f32x16 mma(x8 a, x8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ x4 tr_read(const void *lds) {
        return __builtin_bit_cast(x4, pa_tr16_b64(lds));
    }
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) { return Pk16<pa_f16>::pack(lo, hi); }
};

constexpr int kPfKeys = 64;   // keys per K/V tile
constexpr int kPfSub = kPfKeys / 32;  // 32-key subtiles per tile
constexpr int kPfStages = 4;  // K/V tiles held in LDS (a ring)
constexpr int kPfRows = 32;   // query rows per task (one MFMA column tile)
constexpr int kPfCols = 2;    // tasks (column tiles) per wave
constexpr int kPfWaves = 4;
constexpr int kPfTasks = kPfWaves * kPfCols;  // tasks per workgroup
constexpr int kPfThreads = kPfWaves * 64;
constexpr float kPfSlack = 8.f;  // log2 of the factor by which a row's reference maximum may lag

// LDS tile geometry and swizzles for head_dim D (rows of D*2 bytes = CPR chunks of 16 bytes).
// Tiles of 64 keys the slot tables of prefill_asm_kernel hold (they live in LDS behind the ring, which is 128 KiB at
// head_dim 128 and smaller below), from the workgroup's first tile on: 102 400 keys at head_dim 128, 262 144 at 64 and
// 32.  Workgroups that run more tiles take the instance that fills the tables again on the way.
constexpr int pa_asm_cap_tiles(int head_dim) { return head_dim == 128 ? 1600 : 4096; }

template <int D> struct PfTile {
    static constexpr int RB = D * 2;            // row bytes
    static constexpr int CPR = D / 8;           // 16-byte chunks per row
    static constexpr int RPL = 64 / CPR;        // rows one wave-wide direct load covers
    static constexpr int LOADS = kPfKeys / RPL;  // wave-wide direct loads per tile and tensor
    static constexpr int BYTES = kPfKeys * RB;  // one tensor's tile
    static constexpr int RDIV = 16 / CPR;       // rows that share a 256-byte bank line
    // K: 16 consecutive rows read the same chunk -> 16 distinct 16-byte bank groups
    static __device__ __forceinline__ int swz_k(int row) { return (row / RDIV) % CPR; }
    // V: 4 consecutive rows each read 4 consecutive chunks -> 4 distinct 64-byte bank groups
    static __device__ __forceinline__ int swz_v(int row) { return CPR >= 8 ? ((row / RDIV) % (CPR / 4)) * 4 : 0; }
};

// A wave-uniform pointer, held in scalar registers.
__device__ __forceinline__ const char *pf_scalar_ptr(const char *ptr) {
    const uint64_t v = reinterpret_cast<uint64_t>(ptr);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const char *>(((uint64_t)hi << 32) | lo);
}

// Direct global -> LDS load of 16 bytes per lane: lane i's bytes land at LDS address lds_dst + 16*i.
// Issued as inline assembly on purpose.  The compiler cannot tell which LDS bytes such a load writes when
// the destination is computed, and would make every later LDS read wait for all loads in flight - the
// opposite of prefetching.  The kernel below waits for these loads itself (pf_wait_loads) before the
// barrier that publishes a tile.
__device__ __forceinline__ void pf_dma16(uint32_t lds_dst, const char *scalar_base, uint32_t lane_ofs) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_dst), "v"(lane_ofs), "s"(scalar_base)
                 : "memory", "m0");
}
__device__ __forceinline__ void pf_dma16(uint32_t lds_dst, const char *lane_ptr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_dst), "v"(lane_ptr) : "memory", "m0");
}
// One table entry per lane, loaded behind the compiler's back like the tile loads (a load the compiler knows
// about would make it wait for ALL loads in flight wherever it cannot prove the value has arrived).  The load
// and the wait for it (which is a wait for every load of the wave in flight) are one statement: the
// compiler never sees the register while the value is still on its way.
__device__ __forceinline__ int pf_load_i32_wait(const int32_t *lane_ptr) {
    int v;
    asm volatile("global_load_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(lane_ptr) : "memory");
    return v;
}
// Wait until at most N of this wave's vector memory loads are outstanding (they complete in order).
template <int N> __device__ __forceinline__ void pf_wait_loads() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));  // expcnt / lgkmcnt: no wait
}

template <bool B> struct PfBool { static constexpr bool value = B; };

// Nothing may be moved across this point by the instruction scheduler: the order of the groups of matrix,
// vector and LDS instructions written below is the order they issue in.
#define PF_FENCE() __builtin_amdgcn_sched_barrier(0)
#define PF_INLINE __attribute__((always_inline))

template <typename T, int D, bool BS16>
__global__ __launch_bounds__(kPfThreads) void prefill_mfma_kernel(const RowwiseArgs a) {
    using M = Mfma16<T>;
    using X8 = typename M::x8;
    using X4 = typename M::x4;
    using G = PfTile<D>;
    constexpr int KS = D / 16;  // k-steps of the first product
    constexpr int DT = D / 32;  // 32-wide d tiles of the second product
    constexpr int NC = kPfCols;
    typedef __attribute__((address_space(3))) char lds_char;
    // Ring of kPfStages K/V tiles: stage s holds K at s*2*BYTES and V behind it.
    __shared__ __attribute__((aligned(1024))) char s_kv[kPfStages * 2 * G::BYTES];
    const uint32_t lds_base = (uint32_t)(size_t)(lds_char *)s_kv;

    const PoolArgs &p = a.p;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;  // which 16 of the 32 keys / d values of a result tile
    const int col = lane & 31;   // query row inside a 32-row column tile

    const int kvh = blockIdx.x;
    // Launch order (workgroups start in the order x, y, z).  With a causal mask the last rows of a sequence have
    // the most keys.  When the prefix is shorter than the chunk (dense prefill: no prefix at all) the groups of
    // row blocks differ several-fold in work, and the heaviest groups of all sequences go first (+8 % on dense
    // causal prefill).  Otherwise the groups are about equal and sequences stay the slow index, so that the
    // workgroups in flight on an XCD (one kv head each) belong to few sequences and their keys stay in that
    // XCD's L2.  The first sequence decides for the launch, every workgroup reads the same two numbers.
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
    const int task0 = group * kPfTasks;
    if (task0 >= n_tasks || q_len <= 0) return;  // uniform over the workgroup

    // this wave's tasks (task = row block * n_rep + query head of the kv head) and the last key any wave needs
    bool live[NC];
    int row0[NC], qh[NC], my_keys[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int task = task0 + wave * NC + c;
        live[c] = task < n_tasks;
        const int rb = live[c] ? task / p.n_rep : 0;
        const int rep = live[c] ? task - rb * p.n_rep : 0;
        row0[c] = rb * kPfRows;
        qh[c] = kvh * p.n_rep + rep;
        my_keys[c] = live[c] ? min(ctx_len, prefix + min(q_len, row0[c] + kPfRows)) : 0;  // keys [0, my_keys)
    }
    const int wave_keys = max(my_keys[0], my_keys[1]);
    const int n_sub = (wave_keys + 31) / 32;  // 32-key subtiles this wave multiplies
    const int mask_from = min(prefix + min(row0[0], row0[1]) + 1, ctx_len);  // subtiles reaching past this key are masked
    const int last_task = min(n_tasks, task0 + kPfTasks) - 1;
    const int wg_keys = min(ctx_len, prefix + min(q_len, (last_task / p.n_rep) * kPfRows + kPfRows));
    const int n_tiles = (wg_keys + kPfKeys - 1) / kPfKeys;
    // Lower bounds.  Sliding window: a row at position pos sees keys j > pos - window.  Per-row first keys (packed
    // documents): row i sees keys j >= row_lo[i].  Both bounds are non-decreasing along a sequence, so the
    // workgroup starts at the tile that holds the first key its first row can see (earlier tiles are never
    // loaded); keys below a row's own bound are masked.  Waves whose rows start later see a fully masked first
    // subtile, which contributes nothing.
    const int win = p.window;
    const int32_t *rlo = a.row_lo ? a.row_lo + a.q_starts[b] : nullptr;
    const bool bounded = win > 0 || rlo != nullptr;  // uniform
    // a row's first visible key, clamped so that the row always sees its own position
    auto row_first = [&](int row) PF_INLINE {
        const int pos = prefix + row;
        int lo = win > 0 ? pos - win + 1 : 0;
        if (rlo) lo = max(lo, rlo[min(row, q_len - 1)]);
        return min(max(lo, 0), min(pos, ctx_len - 1));
    };
    const int wg_first_key = bounded ? row_first((task0 / p.n_rep) * kPfRows) : 0;
    const int t0 = wg_first_key / kPfKeys;  // first tile of the workgroup
    // subtiles that start below this key hold keys that some row of the wave cannot see any more
    const int lo_mask_until = bounded ? row_first(min(q_len, max(row0[0], row0[1]) + kPfRows) - 1) : 0;
    int lo_row[NC];  // this lane's rows
#pragma unroll
    for (int c = 0; c < NC; ++c) lo_row[c] = bounded ? row_first(row0[c] + col) : 0;

    // ---- Q^T operands: row = row0 + col, d = 16*ks + 8*half .. +8 ----
    // A lane's operands are 16-byte pieces of 32 different rows, hq*D elements apart: loaded directly, every
    // instruction touches 32 cache lines.  The rows are staged through LDS instead (the ring is still empty):
    // wave-wide direct loads of whole rows into the wave's own area, 16-byte chunks swizzled by row so that the
    // operand reads are free of bank conflicts.  Rows past the chunk's end repeat its last row; they are never
    // written out.
    X8 qreg[NC][KS];
    {
        constexpr int QRB = D * 2;       // bytes of a Q row of one head
        constexpr int QCPR = QRB / 16;   // 16-byte chunks per row
        constexpr int QRPI = 64 / QCPR;  // rows per wave-wide load
        const uint32_t q_stage = (uint32_t)wave * (NC * 32 * QRB);  // this wave's staging area, bytes into s_kv
        const int lrow = lane / QCPR, lslot = lane % QCPR;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const char *qb = reinterpret_cast<const char *>(a.q) + ((int64_t)a.q_starts[b] * p.hq + qh[c]) * (D * 2);
#pragma unroll
            for (int i = 0; i < 32 / QRPI; ++i) {
                const int r = i * QRPI + lrow;  // row of the column tile this lane fills
                const int64_t grow = min(row0[c] + r, q_len - 1);
                pf_dma16(lds_base + q_stage + (uint32_t)((c * 32 + i * QRPI) * QRB),
                         qb + grow * p.hq * (D * 2) + ((lslot ^ (r & (QCPR - 1))) * 16));
            }
        }
        pf_wait_loads<0>();
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int slot = (2 * ks + half) ^ (col & (QCPR - 1));
                const uint4 raw = *reinterpret_cast<const uint4 *>(s_kv + q_stage + (c * 32 + col) * QRB + slot * 16);
                // scaled by softmax scale * log2(e) here, once per workgroup: S^T then comes out of the products
                // in the units of the exponential's argument (one more rounding of q to its 16-bit type)
                const X8 q8 = __builtin_bit_cast(X8, raw);
                uint32_t w[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = M::pack((float)q8[2 * e] * p.scale_log2, (float)q8[2 * e + 1] * p.scale_log2);
                qreg[c][ks] = __builtin_bit_cast(X8, uint4{w[0], w[1], w[2], w[3]});
            }
    }

    // (used here, so that the compiler waits for them here and knows inside the loop that they have arrived)
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+a"(qreg[c][ks]));  // (product operands live in AGPRs)
    __syncthreads();  // every wave has read its staged rows: the ring may overwrite them

    f32x16 o[NC][DT];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[c][dt][i] = 0.f;
    // S^T is kept relative to a reference maximum per row, in base-2 units (Q^T is scaled): the first product
    // of a column tile accumulates onto ref[c] = minus the reference in all 16 registers of a lane, so the
    // exponentials take the S^T values as they are, and a row's maximum mx is relative to its reference too.
    // The reference is allowed to lag behind the true running maximum by up to 2^kPfSlack (as a factor on the
    // probabilities): sums and accumulators are rescaled only when a row's maximum grows by more than that,
    // which it rarely does, instead of on nearly every subtile.  The result is the same quotient either way;
    // probabilities stay below 2^kPfSlack, far inside the range of fp32 sums and of the 16-bit operand types.
    // m_thr is what mx must exceed for a rescale: kNegBig while the row has seen no key yet (its reference is
    // then set by the first maximum, whatever its sign), kPfSlack afterwards.
    f32x16 ref[NC];
    float m_thr[NC], l_run[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        m_thr[c] = kNegBig;
        l_run[c] = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) ref[c][i] = 0.f;
    }

    // ---- tile loader: wave-wide direct load l covers rows l*RPL .. of the tile; wave w issues l = w, w+4, ... ----
    const int32_t *bt_row = p.bt + (int64_t)b * p.bt_stride;
    const int64_t tok_stride = (int64_t)p.hkv * D * 2;
    const char *pool_k = reinterpret_cast<const char *>(p.k) + (int64_t)kvh * D * 2;
    const char *pool_v = reinterpret_cast<const char *>(p.v) + (int64_t)kvh * D * 2;
    const int ld_row = lane / G::CPR, ld_slot = lane % G::CPR;
    constexpr int NLW = (G::LOADS + kPfWaves - 1) / kPfWaves;  // direct loads per wave, tile and tensor
    static_assert(G::LOADS % kPfWaves == 0, "every wave issues the same number of loads");
    // Pools of 16-token blocks: a wave-wide load lies inside one pool block, and the position of a lane's
    // 16 bytes inside that block (token, swizzled chunk) is the same for every load the wave issues.  The
    // address is then a scalar block base plus one per-lane constant.  Block ids come from a window of 64
    // table entries (16 tiles) held one per lane and read out with v_readlane.
    constexpr int BPT = kPfKeys / 16;     // pool blocks per tile
    constexpr int WIN = 64 / BPT;         // tiles per block-id window
    const int64_t block_bytes = 16 * tok_stride;
    uint32_t lane_k = 0, lane_v = 0;
    if (BS16) {
        const int row = wave * G::RPL + ld_row;  // row of the tile for the wave's first load; +16 rows per further load
        const uint32_t tok_ofs = (uint32_t)((row % 16) * tok_stride);
        lane_k = tok_ofs + (uint32_t)((ld_slot ^ G::swz_k(row)) * 16);
        lane_v = tok_ofs + (uint32_t)((ld_slot ^ G::swz_v(row)) * 16);
    }
    int bid_win = -1;
    // Other block sizes (dense prefill hands over whole sequences as single blocks): the loads of a wave walk
    // the context 64 keys per tile, so (table entry, offset in the block) of each of the wave's loads is
    // advanced incrementally; block ids come from a window of 64 table entries starting at win_base.  A tile is
    // regular for the wave when its rows exist, no load straddles a block boundary and every block is present.
    const uint32_t lane_g = (uint32_t)(ld_row * tok_stride);  // + the swizzled chunk, per tensor, below
    int g_blk[NLW], g_off[NLW];  // of the next tile this wave issues
    int win_base = -(1 << 30);
    if (!BS16) {
#pragma unroll
        for (int n = 0; n < NLW; ++n) {
            const int key_first = t0 * kPfKeys + (n * kPfWaves + wave) * G::RPL;
            g_blk[n] = key_first / p.bs;
            g_off[n] = key_first % p.bs;
        }
    }
    // Loads of one tile into its ring stage.  Returns true if the wave issued exactly 2*NLW direct loads and no
    // other vector memory operation after them (what the load-count waits below rely on).
    auto issue = [&](int tile) PF_INLINE -> bool {
        const uint32_t dst0 = lds_base + (uint32_t)(tile % kPfStages) * 2 * G::BYTES;
        if (BS16) {
            if (tile % WIN == 0 || tile == t0) {  // next window of block ids (once per 16 tiles: latency not hidden)
                const int idx = (tile - tile % WIN) * BPT + lane;
                int v = -1;
                if (idx < p.bt_stride) v = pf_load_i32_wait(bt_row + idx);
                bid_win = v;
            }
            const int first = (tile % WIN) * BPT;  // lane of the window that holds the tile's first block
            const bool mine = lane >= first && lane < first + BPT;
            const bool bad = mine && !(bid_win >= 0 && bid_win < p.num_blocks);
            if ((tile + 1) * kPfKeys <= ctx_len && __builtin_amdgcn_ballot_w64(bad) == 0) {
                // whole tile inside the context and every block present (the common case): straight-line loads
                uint32_t lk = lane_k, lv = lane_v;
                asm volatile("" : "+v"(lk), "+v"(lv));
#pragma unroll
                for (int n = 0; n < NLW; ++n) {
                    const int l = n * kPfWaves + wave;  // uniform
                    const uint32_t bid = (uint32_t)__builtin_amdgcn_readlane(bid_win, first + (l * G::RPL) / 16);
                    const uint64_t ofs = (uint64_t)bid * (uint32_t)block_bytes;  // 32 x 32 -> 64 bits on the scalar unit
                    pf_dma16(dst0 + l * G::RPL * G::RB, pf_scalar_ptr(pool_k + ofs), lk);
                    pf_dma16(dst0 + G::BYTES + l * G::RPL * G::RB, pf_scalar_ptr(pool_v + ofs), lv);
                }
                return true;
            }
        } else {
            bool regular = (tile + 1) * kPfKeys <= ctx_len && g_blk[NLW - 1] < p.bt_stride &&
                           g_blk[NLW - 1] - g_blk[0] < 64 && (int64_t)p.num_blocks * p.bs <= 0xffffffffll;
            if (regular && (g_blk[0] < win_base || g_blk[NLW - 1] >= win_base + 64)) {  // move the id window
                win_base = g_blk[0];
                const int idx = win_base + lane;
                int v = -1;
                if (idx < p.bt_stride) v = pf_load_i32_wait(bt_row + idx);
                bid_win = v;
            }
            uint32_t g_row[NLW];  // pool row (slot) of the first row of each load
#pragma unroll
            for (int n = 0; n < NLW; ++n) {
                g_row[n] = 0;
                if (regular) {
                    const int64_t bid = __builtin_amdgcn_readlane(bid_win, g_blk[n] - win_base);
                    regular = g_off[n] + G::RPL <= p.bs && bid >= 0 && bid < p.num_blocks;
                    g_row[n] = (uint32_t)(bid * p.bs + g_off[n]);
                }
            }
            // advance to the next tile (tiles are issued in increasing order, each exactly once)
#pragma unroll
            for (int n = 0; n < NLW; ++n) {
                g_off[n] += kPfKeys;
                if (p.bs >= kPfKeys) {
                    if (g_off[n] >= p.bs) { g_off[n] -= p.bs; g_blk[n] += 1; }
                } else {
                    g_blk[n] += g_off[n] / p.bs;
                    g_off[n] %= p.bs;
                }
            }
            if (regular) {
#pragma unroll
                for (int n = 0; n < NLW; ++n) {
                    const int l = n * kPfWaves + wave;  // uniform
                    const int row = l * G::RPL + ld_row;  // row of the tile this lane fills (its swizzle)
                    const uint64_t ofs = (uint64_t)g_row[n] * (uint32_t)tok_stride;  // 32 x 32 -> 64 bits, scalar
                    uint32_t lk = lane_g + (uint32_t)((ld_slot ^ G::swz_k(row)) * 16);
                    uint32_t lv = lane_g + (uint32_t)((ld_slot ^ G::swz_v(row)) * 16);
                    asm volatile("" : "+v"(lk), "+v"(lv));
                    pf_dma16(dst0 + l * G::RPL * G::RB, pf_scalar_ptr(pool_k + ofs), lk);
                    pf_dma16(dst0 + G::BYTES + l * G::RPL * G::RB, pf_scalar_ptr(pool_v + ofs), lv);
                }
                return true;
            }
        }
        // tile with rows past the context end, missing blocks or loads across block boundaries: per-lane addresses
#pragma unroll
        for (int n = 0; n < NLW; ++n) {
            const int l = n * kPfWaves + wave;  // uniform
            const uint32_t dst_k = dst0 + l * G::RPL * G::RB, dst_v = dst_k + G::BYTES;
            const int row = l * G::RPL + ld_row;  // row of the tile this lane fills
            const int key = tile * kPfKeys + row;
            int64_t bid = -1;
            if (BS16) {
                bid = __builtin_amdgcn_readlane(bid_win, (tile % WIN) * BPT + (l * G::RPL) / 16);
            } else if (key < ctx_len && key / p.bs < p.bt_stride) {
                bid = bt_row[key / p.bs];
            }
            if (key < ctx_len && bid >= 0 && bid < p.num_blocks) {
                const int64_t off = (bid * p.bs + key % p.bs) * tok_stride;
                pf_dma16(dst_k, pool_k + off + ((ld_slot ^ G::swz_k(row)) * 16));
                pf_dma16(dst_v, pool_v + off + ((ld_slot ^ G::swz_v(row)) * 16));
            } else {
                // past the context end or a missing block: all-zero key and value rows
                *reinterpret_cast<uint4 *>(s_kv + (dst_k - lds_base) + lane * 16) = uint4{0, 0, 0, 0};
                *reinterpret_cast<uint4 *>(s_kv + (dst_v - lds_base) + lane * 16) = uint4{0, 0, 0, 0};
            }
        }
        return false;
    };

    // ---- per-lane byte offsets of the operand reads inside a tile ----
    int k_ofs[KS];  // K operand: key row `col` (+32 per subtile), chunk 2*ks + half
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_ofs[ks] = col * G::RB + (((2 * ks + half) ^ G::swz_k(col)) * 16);
    // V^T transpose read: 16-lane group g covers d = 16*(g%2).., keys 4*(g/2)..; source lane s of the group
    // supplies the 8 bytes at key +s/4, d +4*(s%4)
    const int g16 = lane >> 4, s16 = lane & 15;
    const int v_key = 4 * (g16 >> 1) + (s16 >> 2);
    int v_ofs[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
        v_ofs[dt] = v_key * G::RB + ((((4 * dt) ^ G::swz_v(v_key)) + 2 * (g16 & 1) + ((s16 & 3) >> 1)) * 16) + 8 * (s16 & 1);

    // LDS addresses are 32-bit integers: a tile's stage base is added to the per-lane offsets once per tile,
    // and every operand read of the tile is that register plus an immediate offset.
    uint32_t k_adr[KS], v_adr[DT];
    auto set_k_tile = [&](int tile) PF_INLINE {
        const uint32_t base = lds_base + (uint32_t)(tile % kPfStages) * 2 * G::BYTES;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) { k_adr[ks] = base + k_ofs[ks]; asm volatile("" : "+v"(k_adr[ks])); }
    };
    auto set_v_tile = [&](int tile) PF_INLINE {
        const uint32_t base = lds_base + (uint32_t)(tile % kPfStages) * 2 * G::BYTES + G::BYTES;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) { v_adr[dt] = base + v_ofs[dt]; asm volatile("" : "+v"(v_adr[dt])); }
    };
    // K operands of the 32-key subtile `kt` of the tile k_adr points at (shared by the wave's column tiles)
    auto read_k = [&](int kt, X8 (&ka)[KS]) PF_INLINE {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            ka[ks] = __builtin_bit_cast(X8, *reinterpret_cast<const __attribute__((address_space(3))) uint4 *>(
                                                (const lds_char *)(size_t)k_adr[ks] + kt * 32 * G::RB));
    };
    // V^T operands of k-step ks2 of subtile kt (keys 32*kt + 16*ks2 .. +16) of the tile v_adr points at
    auto read_v = [&](int kt, int ks2, X8 (&va)[DT]) PF_INLINE {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const lds_char *base = (const lds_char *)(size_t)v_adr[dt] + (32 * kt + 16 * ks2) * G::RB;
            const X4 lo = __builtin_bit_cast(X4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((pa_s16x4 __attribute__((address_space(3))) *)base));
            const X4 hi = __builtin_bit_cast(
                X4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((pa_s16x4 __attribute__((address_space(3))) *)(base + 8 * G::RB)));
#pragma unroll
            for (int e = 0; e < 4; ++e) { va[dt][e] = lo[e]; va[dt][4 + e] = hi[e]; }
        }
    };
    // causal / context-end mask of S^T
    auto mask_s = [&](f32x16 (&s)[NC], int key_base) PF_INLINE {
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int limit = min(ctx_len - 1, prefix + row0[c] + col) - key_base - 4 * half;  // last visible key
            if (bounded) {
                const int first = lo_row[c] - key_base - 4 * half;  // first visible key
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int idx = 8 * (i >> 2) + (i & 3);
                    s[c][i] = idx <= limit && idx >= first ? s[c][i] : -INFINITY;
                }
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) s[c][i] = 8 * (i >> 2) + (i & 3) <= limit ? s[c][i] : -INFINITY;
            }
        }
    };
    // Row maximum over a subtile's 32 keys, in two pieces (the empty asm statements pin each piece between the
    // scheduling fences around it): the first folds values 0..7, the second values 8..15 and the half of the
    // keys that the other half-wave holds.
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
    auto s_products = [&](const X8 (&ka)[KS], f32x16 (&s)[NC]) PF_INLINE {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int c = 0; c < NC; ++c) s[c] = M::mma(ka[ks], qreg[c][ks], ks == 0 ? ref[c] : s[c]);
    };

    // ---- fill the ring: tiles t0 .. t0 + kPfStages-2 ----
    bool counted[kPfStages - 1];  // loads of the tiles in flight, oldest first: issued as a full group of direct loads?
#pragma unroll
    for (int i = 0; i < kPfStages - 1; ++i) counted[i] = t0 + i < n_tiles ? issue(t0 + i) : false;
    if (counted[1] && counted[2]) pf_wait_loads<4 * NLW>(); else __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();  // tile t0 is visible

    // Software pipeline over the wave's 32-key subtiles g = 0 .. n_sub-1 (tile g/2).  While subtile g is
    // exponentiated and multiplied into O^T, the S^T products of subtile g+1 run on the matrix unit:
    //   (a) S^T products of subtile g+1, with the first half of subtile g's exponentials between them,
    //   (b) first k-step of subtile g's O^T products, with the second half of the exponentials,
    //   (c) second k-step of the O^T products, with subtile g+1's row maxima.
    // Every LDS operand is requested at least one stage before the product that consumes it.  Tile t+1 is
    // published (loads waited for, barrier) in the middle of tile t's first subtile, and the loads of tile
    // t+3 are issued behind that barrier into the stage tile t-1 occupied.
    X8 ka[KS], va0[DT], va1[DT];
    f32x16 sb[2][NC];  // S^T of the current and of the next subtile, swapping roles every subtile
    float mx[NC] = {kNegBig, kNegBig};
    const int g0 = t0 * kPfSub;  // first subtile
    if (n_sub > g0) {
        set_k_tile(t0);
        set_v_tile(t0);
        read_k(0, ka);
        read_v(0, 0, va0);
        PF_FENCE();
        s_products(ka, sb[0]);
        PF_FENCE();
        if (n_sub > g0 + 1) read_k(1, ka);
        PF_FENCE();
        if (32 * (g0 + 1) > mask_from || 32 * g0 < lo_mask_until) mask_s(sb[0], 32 * g0);
#pragma unroll
        for (int c = 0; c < NC; ++c) { max_piece(sb[0][c], 0, mx[c]); max_piece(sb[0][c], 1, mx[c]); }
        PF_FENCE();
    }

    // One tile.  STEADY: every subtile of the tile, the one after it and the operand reads for the one after
    // that exist for this wave, so the body is straight-line code (the compiler then places its LDS waits
    // exactly; with the run-time conditions below it has to assume the worst over all paths).
    auto do_tile = [&](int tile, auto steady_tag) PF_INLINE {
        constexpr bool STEADY = decltype(steady_tag)::value;
#pragma unroll
        for (int kt = 0; kt < kPfSub; ++kt) {
            const int g = tile * kPfSub + kt;
            const bool act = STEADY || g < n_sub;            // uniform per wave
            const bool has_next = STEADY || g + 1 < n_sub;
            // subtile g+1 reaches past the first causal limit, or starts below the last window bound
            const bool mask_next = 32 * (g + 2) > mask_from || 32 * (g + 1) < lo_mask_until;
            static_assert(kPfSub == 2, "the two S^T buffers swap roles once per subtile of a tile");
            f32x16(&s)[NC] = sb[kt & 1];
            f32x16(&s_nx)[NC] = sb[(kt + 1) & 1];
            uint32_t pp[NC][8];
            float sum[NC] = {0.f, 0.f};
            // exponentials of the pair of S^T values 2*j, 2*j+1 of column tile c, packed as a P^T operand word
            // (pinned like the maxima above: otherwise the compiler gathers all exponentials behind the products)
            auto exp_pair = [&](int c, int j) PF_INLINE {
                float x0 = s[c][2 * j], x1 = s[c][2 * j + 1];
                asm volatile("" : "+v"(x0), "+v"(x1));  // copies defined here: the arithmetic cannot start earlier
                const float p0 = __builtin_amdgcn_exp2f(x0);
                const float p1 = __builtin_amdgcn_exp2f(x1);
                sum[c] += p0 + p1;
                uint32_t w = M::pack(p0, p1);
                asm volatile("" : "+v"(w), "+v"(sum[c]));
                pp[c][j] = w;
            };
            // piece n of 16: pieces 0..7 make the operand words of the first k-step, 8..15 of the second
            auto exp_piece = [&](int n) PF_INLINE { exp_pair(n & 1, (n >> 1)); };
            if (act) {
                // ---- a row's maximum outgrew its reference by more than the slack (rare): rescale ----
                if (__builtin_expect(__builtin_amdgcn_ballot_w64(mx[0] > m_thr[0] || mx[1] > m_thr[1]) != 0, 0)) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        // the reference moves by delta: up to the new maximum, or - for a row that had seen no
                        // key so far (sums and accumulators still zero) - to its first maximum, whatever its sign
                        const bool unset = m_thr[c] == kNegBig;
                        const bool seen = mx[c] > kNegBig;
                        const float delta = unset ? (seen ? mx[c] : 0.f) : fmaxf(mx[c], 0.f);
                        const float alpha = unset ? 1.f : __builtin_amdgcn_exp2f(-delta);
                        l_run[c] *= alpha;
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                            for (int i = 0; i < 16; ++i) o[c][dt][i] *= alpha;
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            ref[c][i] -= delta;
                            s[c][i] -= delta;  // formed against the old reference
                        }
                        mx[c] -= delta;
                        if (seen) m_thr[c] = kPfSlack;
                    }
                }
                PF_FENCE();
                read_v(kt, 1, va1);  // second k-step's V^T: consumed in (c)
                PF_FENCE();
                // ---- (a) ----
                constexpr int PA = 8 / KS;  // pieces per k-step
                if (has_next) {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                        for (int c = 0; c < NC; ++c) s_nx[c] = M::mma(ka[ks], qreg[c][ks], ks == 0 ? ref[c] : s_nx[c]);
#pragma unroll
                        for (int n = 0; n < PA; ++n) exp_piece(ks * PA + n);
                        PF_FENCE();
                    }
                } else {
#pragma unroll
                    for (int n = 0; n < 8; ++n) exp_piece(n);
                    PF_FENCE();
                }
            }
            if (kt == 0) {
                // ---- publish tile+1; start the loads of tile+3 into the stage of tile-1 (all waves) ----
                if (STEADY || tile + 1 < n_tiles) {
                    // loads in flight, oldest first: tile+1, tile+2
                    if (counted[1]) pf_wait_loads<2 * NLW>(); else __builtin_amdgcn_s_waitcnt(0);
                    __syncthreads();
                }
                counted[0] = counted[1];
                counted[1] = counted[2];
                counted[2] = tile + 3 < n_tiles ? issue(tile + 3) : false;
                PF_FENCE();
            }
            // K operands of subtile g+2 (first subtile of the next tile when kt == 0): consumed in (a) of g+1
            if (STEADY || g + 2 < n_sub) {
                if (kt == 0) set_k_tile(tile + 1);
                read_k(kt == 0 ? 0 : 1, ka);
            }
            PF_FENCE();
            if (act) {
                // ---- (b) O^T += V^T . P^T, first k-step: result rows 0..7 of a lane, i.e. keys
                //      key_base + 8*(e/4) + 4*half + e%4 for operand element e ----
                constexpr int PB = 8 / (DT * NC);  // pieces per product
                {
                    X8 pb[NC];
#pragma unroll
                    for (int c = 0; c < NC; ++c) pb[c] = __builtin_bit_cast(X8, uint4{pp[c][0], pp[c][1], pp[c][2], pp[c][3]});
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int c = 0; c < NC; ++c) {
                            o[c][dt] = M::mma(va0[dt], pb[c], o[c][dt]);
#pragma unroll
                            for (int n = 0; n < PB; ++n) exp_piece(8 + (dt * NC + c) * PB + n);
                            PF_FENCE();
                        }
                }
                if (has_next) {  // first k-step's V^T of the next subtile
                    if (kt == kPfSub - 1) set_v_tile(tile + 1);
                    read_v(kt == kPfSub - 1 ? 0 : kt + 1, 0, va0);
                    if (mask_next) mask_s(s_nx, 32 * (g + 1));
                }
                PF_FENCE();
                // ---- (c) second k-step (keys +16), with the next subtile's row maxima ----
                {
                    X8 pb[NC];
#pragma unroll
                    for (int c = 0; c < NC; ++c) pb[c] = __builtin_bit_cast(X8, uint4{pp[c][4], pp[c][5], pp[c][6], pp[c][7]});
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int c = 0; c < NC; ++c) {
                            o[c][dt] = M::mma(va1[dt], pb[c], o[c][dt]);
                            const int i = dt * NC + c;  // products issued so far in this stage
                            if (has_next && i < 2 * NC) max_piece(s_nx[i / 2], i % 2, mx[i / 2]);
                            PF_FENCE();
                        }
                    if (has_next && DT * NC < 2 * NC) {  // head_dim 32: fewer products than pieces
#pragma unroll
                        for (int i = DT * NC; i < 2 * NC; ++i) max_piece(s_nx[i / 2], i % 2, mx[i / 2]);
                    }
                }
#pragma unroll
                for (int c = 0; c < NC; ++c) l_run[c] += sum[c];
                PF_FENCE();
            }
        }
    };
    const int steady_tiles = max(0, (n_sub - 2) / kPfSub);  // tiles whose subtiles g all have g + 2 < n_sub
    int tile = t0;
    for (; tile < steady_tiles; ++tile) do_tile(tile, PfBool<true>{});
    for (; tile < n_tiles; ++tile) do_tile(tile, PfBool<false>{});

    // ---- normalise and write: lane owns row (row0+col), d = 32*dt + 4*half + 8*g + j ----
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const float l_tot = l_run[c] + __shfl_xor(l_run[c], 32, 64);
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        const int row = row0[c] + col;
        if (!live[c] || row >= q_len) continue;
        T *orow = reinterpret_cast<T *>(a.out) + (((int64_t)a.q_starts[b] + row) * p.hq + qh[c]) * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                uint2 w;
                w.x = M::pack(o[c][dt][4 * g] * inv, o[c][dt][4 * g + 1] * inv);
                w.y = M::pack(o[c][dt][4 * g + 2] * inv, o[c][dt][4 * g + 3] * inv);
                *reinterpret_cast<uint2 *>(orow + 32 * dt + 4 * half + 8 * g) = w;
            }
    }
}

typedef void (*prefill_mfma_fn)(const RowwiseArgs);
// nullptr if the shape has no matrix-core kernel; `bs16` selects the variant for pools of 16-token blocks
prefill_mfma_fn pa_prefill_mfma_kernel(int dtype, int d, bool bs16);

}  // namespace pa_decode_detail
