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
//   workgroup = 8 waves (two per SIMD, so one wave's softmax arithmetic runs
//   under the other's matrix instructions); a wave owns 32 query rows (one MFMA
//   column tile) of ONE query head and keeps everything in ordinary VGPRs
//   (64 accumulators + 32 for Q + 16 for S); the 8 waves take 8 consecutive
//   (row block, query head of the kv head) tasks, so they share every K/V tile
//   (GQA packing: K/V are fetched once per kv head, not per query head).
//   grid.x = kv head (fastest): with 8 XCDs a kv head's K/V stays in one XCD's
//   L2 while all sequences and row blocks that share prefix blocks re-read it.
//   K/V tiles of 64 keys go global -> LDS directly (global_load_lds, 16 bytes per
//   lane, no staging registers) into one of two buffers, so the next tile's
//   loads are in flight while the current tile is multiplied and there is one
//   barrier per tile.  A direct load puts lane i's 16 bytes at base + 16*i, so
//   rows cannot be padded; instead each lane fetches the chunk that belongs at
//   its position under an XOR swizzle of the chunk index by the row, chosen so
//   that the 128-bit operand reads (16 rows, same chunk) and the transpose
//   reads (4 rows x 64 bytes) each touch all 64 banks once.
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

constexpr int kPfKeys = 128;  // keys per K/V tile
constexpr int kPfSub = kPfKeys / 32;  // 32-key subtiles per tile
constexpr int kPfRows = 32;   // query rows per task (one MFMA column tile)
constexpr int kPfCols = 2;    // tasks (column tiles) per wave
constexpr int kPfWaves = 4;
constexpr int kPfTasks = kPfWaves * kPfCols;  // tasks per workgroup
constexpr int kPfThreads = kPfWaves * 64;
constexpr float kPfSlack = 8.f;  // log2 of the factor by which a row's reference maximum may lag

// LDS tile geometry and swizzles for head_dim D (rows of D*2 bytes = CPR chunks of 16 bytes).
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

// Nothing may be moved across this point by the instruction scheduler: the order of the groups of matrix,
// vector and LDS instructions written below is the order they issue in.
#define PF_FENCE() __builtin_amdgcn_sched_barrier(0)

template <typename T, int D, bool BS16>
__global__ __launch_bounds__(kPfThreads) void prefill_mfma_kernel(const RowwiseArgs a) {
    using M = Mfma16<T>;
    using X8 = typename M::x8;
    using X4 = typename M::x4;
    using G = PfTile<D>;
    constexpr int KS = D / 16;  // k-steps of the first product
    constexpr int DT = D / 32;  // 32-wide d tiles of the second product
    constexpr int NC = kPfCols;
    // Two K/V tile buffers as four separate LDS objects: the compiler then knows that a direct load into one
    // buffer cannot alias the operand reads from the other and does not make the reads wait for the load.
    __shared__ __attribute__((aligned(1024))) char s_k0[G::BYTES];
    __shared__ __attribute__((aligned(1024))) char s_v0[G::BYTES];
    __shared__ __attribute__((aligned(1024))) char s_k1[G::BYTES];
    __shared__ __attribute__((aligned(1024))) char s_v1[G::BYTES];

    const PoolArgs &p = a.p;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;  // which 16 of the 32 keys / d values of a result tile
    const int col = lane & 31;   // query row inside a 32-row column tile

    const int kvh = blockIdx.x;
    const int b = blockIdx.z;
    const int q_len = a.q_lens[b];
    const int ctx_len = a.ctx_lens[b];
    const int prefix = ctx_len - q_len;
    const int n_rowblocks = (q_len + kPfRows - 1) / kPfRows;
    const int n_tasks = n_rowblocks * p.n_rep;
    const int task0 = blockIdx.y * kPfTasks;
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
    const int last_task = min(n_tasks, task0 + kPfTasks) - 1;
    const int wg_keys = min(ctx_len, prefix + min(q_len, (last_task / p.n_rep) * kPfRows + kPfRows));
    const int n_tiles = (wg_keys + kPfKeys - 1) / kPfKeys;

    // ---- Q^T operands: row = row0 + col, d = 16*ks + 8*half .. +8 ----
    X8 qreg[NC][KS];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const T *qbase = reinterpret_cast<const T *>(a.q) + ((int64_t)a.q_starts[b] * p.hq + qh[c]) * D;
        const int row = row0[c] + col;
        const bool ok = live[c] && row < q_len;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint4 raw = ok ? ld16(qbase + (int64_t)row * p.hq * D + 16 * ks + 8 * half) : uint4{0, 0, 0, 0};
            qreg[c][ks] = __builtin_bit_cast(X8, raw);
        }
    }

    f32x16 o[NC][DT];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[c][dt][i] = 0.f;
    // running maximum of the raw (unscaled) logits, the same times scale*log2e, and the running sum
    const float sc = p.scale_log2;
    // The reference maximum of a row is allowed to lag behind the true running maximum by up to 2^kPfSlack
    // (as a factor on the probabilities): sums and accumulators are rescaled only when a row's maximum grows
    // by more than that, which it rarely does, instead of on nearly every subtile.  The result is the same
    // quotient either way; probabilities stay below 2^kPfSlack, far inside the range of fp32 sums and of the
    // 16-bit operand types.
    const float slack_raw = kPfSlack / sc;
    float m_raw[NC], m_sc[NC], m_thr[NC], l_run[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) { m_raw[c] = kNegBig; m_thr[c] = kNegBig; m_sc[c] = kNegBig * sc; l_run[c] = 0.f; }

    // ---- tile loader: wave-wide direct load l covers rows l*RPL .. of the tile; wave w issues l = w, w+4, ... ----
    const int32_t *bt_row = p.bt + (int64_t)b * p.bt_stride;
    const int64_t tok_stride = (int64_t)p.hkv * D * 2;
    const char *pool_k = reinterpret_cast<const char *>(p.k) + (int64_t)kvh * D * 2;
    const char *pool_v = reinterpret_cast<const char *>(p.v) + (int64_t)kvh * D * 2;
    const int ld_row = lane / G::CPR, ld_slot = lane % G::CPR;
    constexpr int NLW = (G::LOADS + kPfWaves - 1) / kPfWaves;  // direct loads per wave, tile and tensor
    // Block ids are looked up one tile ahead of the loads that use them, so that the table read (and its
    // latency) never sits between the barrier and the products.
    //
    // Pools of 16-token blocks: a wave-wide load lies inside one pool block, and the position of a lane's
    // 16 bytes inside that block (token, swizzled chunk) is the same for every load the wave issues.  The
    // address is then a scalar block base plus one per-lane constant, and the block ids of a tile are one
    // vector register (lane i holds block i of the tile) read out with v_readlane.
    constexpr int BPT = kPfKeys / 16;  // pool blocks per tile
    int bid_vec = -1;
    const int64_t block_bytes = 16 * tok_stride;
    uint32_t lane_k = 0, lane_v = 0;
    if (BS16) {
        const int row = wave * G::RPL + ld_row;  // row of the tile for the wave's first load; +16 rows per further load
        const uint32_t tok_ofs = (uint32_t)((row % 16) * tok_stride);
        lane_k = tok_ofs + (uint32_t)((ld_slot ^ G::swz_k(row)) * 16);
        lane_v = tok_ofs + (uint32_t)((ld_slot ^ G::swz_v(row)) * 16);
    }
    // Other block sizes: per-lane block ids and addresses.
    int bid_next[BS16 ? 1 : NLW];  // kept as loaded: any arithmetic on it here would wait for the load
    auto lookup = [&](int tile) __attribute__((always_inline)) {
        if (BS16) {
            const int idx = tile * BPT + lane;
            bid_vec = -1;
            if (lane < BPT && idx < p.bt_stride && tile * kPfKeys < ctx_len) bid_vec = bt_row[idx];
            return;
        }
#pragma unroll
        for (int n = 0; n < NLW; ++n) {
            const int l = n * kPfWaves + wave;  // uniform
            bid_next[BS16 ? 0 : n] = -1;
            if (l >= G::LOADS) continue;
            const int key = tile * kPfKeys + l * G::RPL + ld_row;
            const int blk = key < ctx_len ? key / p.bs : -1;
            if (blk >= 0 && blk < p.bt_stride) bid_next[BS16 ? 0 : n] = bt_row[blk];
        }
    };
    auto load_rows = [&](const char *src_k, const char *src_v, char *dst_k, char *dst_v) __attribute__((always_inline)) {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src_k,
                                         (__attribute__((address_space(3))) void *)dst_k, 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src_v,
                                         (__attribute__((address_space(3))) void *)dst_v, 16, 0, 0);
    };
    auto zero_rows = [&](char *dst_k, char *dst_v) __attribute__((always_inline)) {
        // past the context end or a missing block: all-zero key and value rows
        *reinterpret_cast<uint4 *>(dst_k + lane * 16) = uint4{0, 0, 0, 0};
        *reinterpret_cast<uint4 *>(dst_v + lane * 16) = uint4{0, 0, 0, 0};
    };
    auto issue = [&](int tile, char *buf_k, char *buf_v) __attribute__((always_inline)) {
        if (BS16) {
            // whole tile inside the context and every block present (the common case): straight-line loads
            const bool in_pool = lane >= BPT || (bid_vec >= 0 && bid_vec < p.num_blocks);
            if ((tile + 1) * kPfKeys <= ctx_len && __builtin_amdgcn_ballot_w64(!in_pool) == 0) {
                uint32_t lk = lane_k, lv = lane_v;
                asm volatile("" : "+v"(lk), "+v"(lv));  // 32-bit lane offsets at the point of use: scalar base + offset loads
#pragma unroll
                for (int n = 0; n < NLW; ++n) {
                    const int l = n * kPfWaves + wave;  // uniform
                    if (G::LOADS % kPfWaves != 0 && l >= G::LOADS) break;
                    const uint32_t bid = (uint32_t)__builtin_amdgcn_readlane(bid_vec, (l * G::RPL) / 16);
                    const uint64_t ofs = (uint64_t)bid * (uint32_t)block_bytes;  // 32 x 32 -> 64 bits on the scalar unit
                    // (read back through the scalar unit so that the base stays apart from the lane offset)
                    const char *base_k = pf_scalar_ptr(pool_k + ofs);
                    const char *base_v = pf_scalar_ptr(pool_v + ofs);
                    load_rows(base_k + lk, base_v + lv, buf_k + l * G::RPL * G::RB, buf_v + l * G::RPL * G::RB);
                }
                return;
            }
        }
#pragma unroll
        for (int n = 0; n < NLW; ++n) {
            const int l = n * kPfWaves + wave;  // uniform
            if (l >= G::LOADS) break;
            char *dst_k = buf_k + l * G::RPL * G::RB;  // uniform; lane i lands at +16*i
            char *dst_v = buf_v + l * G::RPL * G::RB;
            const int row = l * G::RPL + ld_row;  // row of the tile this lane fills
            const int key = tile * kPfKeys + row;
            if (BS16) {
                const int64_t bid = __builtin_amdgcn_readlane(bid_vec, (l * G::RPL) / 16);  // uniform
                if (key < ctx_len && bid >= 0 && bid < p.num_blocks)
                    load_rows(pool_k + bid * block_bytes + lane_k, pool_v + bid * block_bytes + lane_v, dst_k, dst_v);
                else
                    zero_rows(dst_k, dst_v);
            } else {
                const int64_t bid = bid_next[BS16 ? 0 : n];  // sign-extended only now, one tile after it was loaded
                if (key < ctx_len && bid >= 0 && bid < p.num_blocks) {
                    const int64_t off = (bid * p.bs + key % p.bs) * tok_stride;
                    load_rows(pool_k + off + ((ld_slot ^ G::swz_k(row)) * 16), pool_v + off + ((ld_slot ^ G::swz_v(row)) * 16),
                              dst_k, dst_v);
                } else {
                    zero_rows(dst_k, dst_v);
                }
            }
        }
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

    // LDS addresses are handled as 32-bit integers: a tile's base is added to the per-lane offsets once per
    // tile, and every operand read of the tile is that register plus an immediate offset.
    typedef __attribute__((address_space(3))) char lds_char;
    auto lds_addr = [&](char *ptr) __attribute__((always_inline)) { return (uint32_t)(size_t)(lds_char *)ptr; };
    // K operands of the 32-key subtile `kt` (shared by the wave's column tiles)
    auto read_k = [&](const uint32_t (&k_adr)[KS], int kt, X8 (&ka)[KS]) __attribute__((always_inline)) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            ka[ks] = __builtin_bit_cast(X8, *reinterpret_cast<const __attribute__((address_space(3))) uint4 *>(
                                                (const lds_char *)(size_t)k_adr[ks] + kt * 32 * G::RB));
    };
    // V^T operands of k-step ks2 of subtile kt (keys 32*kt + 16*ks2 .. +16)
    auto read_v = [&](const uint32_t (&v_adr)[DT], int kt, int ks2, X8 (&va)[DT]) __attribute__((always_inline)) {
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
    auto mask_s = [&](f32x16 (&s)[NC], int key_base) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int limit = min(ctx_len - 1, prefix + row0[c] + col) - key_base - 4 * half;  // last visible key
#pragma unroll
            for (int i = 0; i < 16; ++i) s[c][i] = 8 * (i >> 2) + (i & 3) <= limit ? s[c][i] : -INFINITY;
        }
    };
    // Row maximum over a subtile's 32 keys, in two pieces (the empty asm statements pin each piece between the
    // scheduling fences around it): the first folds values 0..7, the second values 8..15 and the half of the
    // keys that the other half-wave holds.
    auto max_piece = [&](f32x16 &s, int h, float &mx) __attribute__((always_inline)) {
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

    // One K/V tile.  Per 32-key subtile the issue order is
    //   (a) S^T products of the NEXT subtile, with the first half of this subtile's exponentials between them,
    //   (b) first k-step of this subtile's O^T products, with the second half of the exponentials,
    //   (c) second k-step of the O^T products, with the next subtile's row maxima,
    // so that the matrix unit always has a product queued while the vector ALU does the softmax arithmetic,
    // and every LDS operand is requested at least one stage before the product that consumes it.
    auto do_tile = [&](int tile, char *cur_k, char *cur_v, char *nxt_k, char *nxt_v) __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(0);  // this wave's direct loads and zero fills of `tile` have landed
        __syncthreads();                // ... and everyone's; everyone is also done reading the other buffer
        if (tile + 1 < n_tiles) {
            issue(tile + 1, nxt_k, nxt_v);
            lookup(tile + 2);  // consumed by the next tile's issue()
        }
        const int key0 = tile * kPfKeys;
        if (key0 >= wave_keys) return;  // this wave's rows end before this tile (uniform per wave)
        // masking is needed only where the tile reaches past a first row's causal limit or the context end
        const bool need_mask = key0 + kPfKeys > prefix + min(row0[0], row0[1]) + 1 || key0 + kPfKeys > ctx_len;

        uint32_t k_adr[KS], v_adr[DT];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) { k_adr[ks] = lds_addr(cur_k) + k_ofs[ks]; asm volatile("" : "+v"(k_adr[ks])); }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) { v_adr[dt] = lds_addr(cur_v) + v_ofs[dt]; asm volatile("" : "+v"(v_adr[dt])); }

        X8 ka[KS], va0[DT], va1[DT];
        f32x16 s_nx[NC];
        float mx[NC];
        // prologue: S^T of the first subtile
        read_k(k_adr, 0, ka);
        read_v(v_adr, 0, 0, va0);
        PF_FENCE();
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int i = 0; i < 16; ++i) s_nx[c][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int c = 0; c < NC; ++c) s_nx[c] = M::mma(ka[ks], qreg[c][ks], s_nx[c]);
        PF_FENCE();
        read_k(k_adr, 1, ka);
        PF_FENCE();
        if (need_mask) mask_s(s_nx, key0);
#pragma unroll
        for (int c = 0; c < NC; ++c) { max_piece(s_nx[c], 0, mx[c]); max_piece(s_nx[c], 1, mx[c]); }
        PF_FENCE();

#pragma unroll
        for (int kt = 0; kt < kPfSub; ++kt) {
            const bool has_next = kt + 1 < kPfSub;
            f32x16 s[NC];
#pragma unroll
            for (int c = 0; c < NC; ++c) s[c] = s_nx[c];
            // ---- a row's maximum outgrew its reference by more than the slack (rare): rescale ----
            if (__builtin_expect(__builtin_amdgcn_ballot_w64(mx[0] > m_thr[0] || mx[1] > m_thr[1]) != 0, 0)) {
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const float m_new = fmaxf(m_raw[c], mx[c]);
                    const float alpha = __builtin_amdgcn_exp2f((m_raw[c] - m_new) * sc);
                    l_run[c] *= alpha;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int i = 0; i < 16; ++i) o[c][dt][i] *= alpha;
                    m_raw[c] = m_new;
                    m_thr[c] = m_new + slack_raw;
                    m_sc[c] = m_new * sc;
                }
            }
            PF_FENCE();
            read_v(v_adr, kt, 1, va1);  // second k-step's V^T: consumed in (c)
            PF_FENCE();
            uint32_t pp[NC][8];
            float sum[NC] = {0.f, 0.f};
            // exponentials of the pair of S^T values 2*j, 2*j+1 of column tile c, packed as a P^T operand word
            // (pinned like the maxima above: otherwise the compiler gathers all exponentials behind the products)
            auto exp_pair = [&](int c, int j) __attribute__((always_inline)) {
                float x0 = s[c][2 * j], x1 = s[c][2 * j + 1];
                asm volatile("" : "+v"(x0), "+v"(x1));
                const float p0 = __builtin_amdgcn_exp2f(fmaf(x0, sc, -m_sc[c]));
                const float p1 = __builtin_amdgcn_exp2f(fmaf(x1, sc, -m_sc[c]));
                sum[c] += p0 + p1;
                uint32_t w = M::pack(p0, p1);
                asm volatile("" : "+v"(w), "+v"(sum[c]));
                pp[c][j] = w;
            };
            // piece n of 16: pieces 0..7 make the operand words of the first k-step, 8..15 of the second
            auto exp_piece = [&](int n) __attribute__((always_inline)) { exp_pair(n & 1, (n >> 1)); };
            // ---- (a) ----
            constexpr int PA = 8 / KS;  // pieces per k-step
            if (has_next) {
#pragma unroll
                for (int c = 0; c < NC; ++c)
#pragma unroll
                    for (int i = 0; i < 16; ++i) s_nx[c][i] = 0.f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) s_nx[c] = M::mma(ka[ks], qreg[c][ks], s_nx[c]);
#pragma unroll
                    for (int n = 0; n < PA; ++n) exp_piece(ks * PA + n);
                    PF_FENCE();
                }
                if (kt + 2 < kPfSub) read_k(k_adr, kt + 2, ka);  // consumed in (a) of the next subtile
                PF_FENCE();
            } else {
#pragma unroll
                for (int n = 0; n < 8; ++n) exp_piece(n);
                PF_FENCE();
            }
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
            if (has_next) read_v(v_adr, kt + 1, 0, va0);  // first k-step's V^T of the next subtile
            if (has_next && need_mask) mask_s(s_nx, key0 + 32 * (kt + 1));
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
                        const int g = dt * NC + c;  // products issued so far in this stage
                        if (has_next && g < 2 * NC) max_piece(s_nx[g / 2], g % 2, mx[g / 2]);
                        PF_FENCE();
                    }
                if (has_next && DT * NC < 2 * NC) {  // head_dim 32: fewer products than pieces
#pragma unroll
                    for (int g = DT * NC; g < 2 * NC; ++g) max_piece(s_nx[g / 2], g % 2, mx[g / 2]);
                }
            }
#pragma unroll
            for (int c = 0; c < NC; ++c) l_run[c] += sum[c];
            PF_FENCE();
        }
    };
    lookup(0);
    issue(0, s_k0, s_v0);
    lookup(1);
    for (int tile = 0; tile < n_tiles; tile += 2) {
        do_tile(tile, s_k0, s_v0, s_k1, s_v1);
        if (tile + 1 < n_tiles) do_tile(tile + 1, s_k1, s_v1, s_k0, s_v0);
    }

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
