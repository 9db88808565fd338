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
constexpr int kPfRows = 32;   // query rows per wave
constexpr int kPfWaves = 8;
constexpr int kPfThreads = kPfWaves * 64;

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

template <typename T, int D, bool BS16>
__global__ __launch_bounds__(kPfThreads) void prefill_mfma_kernel(const RowwiseArgs a) {
    using M = Mfma16<T>;
    using X8 = typename M::x8;
    using X4 = typename M::x4;
    using G = PfTile<D>;
    constexpr int KS = D / 16;  // k-steps of the first product
    constexpr int DT = D / 32;  // 32-wide d tiles of the second product
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
    const int col = lane & 31;   // query row inside the wave's 32-row tile

    const int kvh = blockIdx.x;
    const int b = blockIdx.z;
    const int q_len = a.q_lens[b];
    const int ctx_len = a.ctx_lens[b];
    const int prefix = ctx_len - q_len;
    const int n_rowblocks = (q_len + kPfRows - 1) / kPfRows;
    const int n_tasks = n_rowblocks * p.n_rep;
    const int task0 = blockIdx.y * kPfWaves;
    if (task0 >= n_tasks || q_len <= 0) return;  // uniform over the workgroup

    // this wave's task and the last key any wave of the workgroup needs
    const int task = task0 + wave;
    const bool live = task < n_tasks;
    const int rb = live ? task / p.n_rep : 0;
    const int rep = live ? task - rb * p.n_rep : 0;
    const int row0 = rb * kPfRows;
    const int qh = kvh * p.n_rep + rep;
    const int my_keys = live ? min(ctx_len, prefix + min(q_len, row0 + kPfRows)) : 0;  // keys [0, my_keys)
    const int last_task = min(n_tasks, task0 + kPfWaves) - 1;
    const int wg_keys = min(ctx_len, prefix + min(q_len, (last_task / p.n_rep) * kPfRows + kPfRows));
    const int n_tiles = (wg_keys + kPfKeys - 1) / kPfKeys;

    // ---- Q^T operand: row = row0 + col, d = 16*ks + 8*half .. +8 ----
    const T *qbase = reinterpret_cast<const T *>(a.q) + ((int64_t)a.q_starts[b] * p.hq + qh) * D;
    X8 qreg[KS];
    {
        const int row = row0 + col;
        const bool ok = live && row < q_len;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint4 raw = ok ? ld16(qbase + (int64_t)row * p.hq * D + 16 * ks + 8 * half) : uint4{0, 0, 0, 0};
            qreg[ks] = __builtin_bit_cast(X8, raw);
        }
    }

    f32x16 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
    // running maximum of the raw (unscaled) logits, the same times scale*log2e, and the running sum
    const float c = p.scale_log2;
    float m_raw = kNegBig, m_sc = kNegBig * c, l_run = 0.f;

    // ---- tile loader: wave-wide direct load l covers rows l*RPL .. of the tile; wave w issues l = w, w+8, ... ----
    const int32_t *bt_row = p.bt + (int64_t)b * p.bt_stride;
    const int64_t tok_stride = (int64_t)p.hkv * D * 2;
    const char *pool_k = reinterpret_cast<const char *>(p.k) + (int64_t)kvh * D * 2;
    const char *pool_v = reinterpret_cast<const char *>(p.v) + (int64_t)kvh * D * 2;
    const int ld_row = lane / G::CPR, ld_slot = lane % G::CPR;
    constexpr int NLW = (G::LOADS + kPfWaves - 1) / kPfWaves;  // direct loads per wave, tile and tensor
    // Block ids are looked up one tile ahead of the loads that use them, so that the table read (and its
    // latency) never sits between the barrier and the products: bid_next[] holds the ids for the tile that
    // the next call of issue() will load.
    int bid_next[NLW];  // kept as loaded: any arithmetic on it here would wait for the load
    auto lookup = [&](int tile) {
#pragma unroll
        for (int n = 0; n < NLW; ++n) {
            const int l = n * kPfWaves + wave;  // uniform
            bid_next[n] = -1;
            if (l >= G::LOADS) continue;
            int blk;
            if (BS16) {
                blk = tile * (kPfKeys / 16) + (l * G::RPL) / 16;  // uniform: the load's rows lie in one pool block
            } else {
                const int key = tile * kPfKeys + l * G::RPL + ld_row;
                blk = key < ctx_len ? key / p.bs : -1;
            }
            // The index is laundered through a VGPR so that this becomes a vector load: a scalar load would
            // share its completion counter with the LDS operand reads and stall the first of them.
            asm volatile("" : "+v"(blk));
            if (blk >= 0 && blk < p.bt_stride && tile * kPfKeys < ctx_len) bid_next[n] = bt_row[blk];
        }
    };
    auto issue = [&](int tile, char *buf_k, char *buf_v) {
#pragma unroll
        for (int n = 0; n < NLW; ++n) {
            const int l = n * kPfWaves + wave;  // uniform
            if (l >= G::LOADS) break;
            const int row = l * G::RPL + ld_row;  // row of the tile this lane fills
            const int key = tile * kPfKeys + row;
            const int64_t bid = bid_next[n];  // sign-extended only now, one tile after the load was issued
            const int tok = BS16 ? (l * G::RPL) % 16 + ld_row : key % p.bs;
            const bool ok = key < ctx_len && bid >= 0 && bid < p.num_blocks;
            char *dst_k = buf_k + l * G::RPL * G::RB;  // uniform; lane i lands at +16*i
            char *dst_v = buf_v + l * G::RPL * G::RB;
            if (ok) {
                const int64_t off = (bid * p.bs + tok) * tok_stride;
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void *)(pool_k + off + ((ld_slot ^ G::swz_k(row)) * 16)),
                    (__attribute__((address_space(3))) void *)dst_k, 16, 0, 0);
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void *)(pool_v + off + ((ld_slot ^ G::swz_v(row)) * 16)),
                    (__attribute__((address_space(3))) void *)dst_v, 16, 0, 0);
            } else {
                // past the context end or a missing block: all-zero key and value rows
                *reinterpret_cast<uint4 *>(dst_k + lane * 16) = uint4{0, 0, 0, 0};
                *reinterpret_cast<uint4 *>(dst_v + lane * 16) = uint4{0, 0, 0, 0};
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

    // S^T = K . Q^T for one 32-key subtile (this wave's 32 rows)
    auto s_phase = [&](const char *tk) {
        f32x16 s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.f;
        constexpr int KG = KS < 4 ? KS : 4;  // operand reads are issued in groups of 4 k-steps
#pragma unroll
        for (int k0 = 0; k0 < KS; k0 += KG) {
            X8 ka[KG];
#pragma unroll
            for (int ks = 0; ks < KG; ++ks)
                ka[ks] = __builtin_bit_cast(X8, *reinterpret_cast<const uint4 *>(tk + k_ofs[k0 + ks]));
#pragma unroll
            for (int ks = 0; ks < KG; ++ks) s = M::mma(ka[ks], qreg[k0 + ks], s);
        }
        return s;
    };

    // Softmax and O^T update of one subtile whose S^T is `s`.  When there is a next subtile in the tile its
    // S^T products are issued here, between the running-maximum step and the exponentials, so that the matrix
    // unit works while this wave's vector ALU does the exp / sum / pack arithmetic.
    auto subtile = [&](f32x16 s, const char *tk_next, const char *tv, int key_base, bool need_mask, bool has_next) {
        // V^T operands of the first k-step are requested before the softmax arithmetic
        X4 vlo[DT], vhi[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            vlo[dt] = M::tr_read(tv + v_ofs[dt]);
            vhi[dt] = M::tr_read(tv + v_ofs[dt] + 8 * G::RB);
        }
        // ---- online softmax per row (= per lane); P^T is packed in place ----
        if (need_mask) {  // uniform
            const int limit = min(ctx_len - 1, prefix + row0 + col) - key_base - 4 * half;  // last visible key
#pragma unroll
            for (int i = 0; i < 16; ++i) s[i] = 8 * (i >> 2) + (i & 3) <= limit ? s[i] : -INFINITY;
        }
        float mx = fmaxf(s[0], s[1]);
#pragma unroll
        for (int i = 2; i < 16; ++i) mx = fmaxf(mx, s[i]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(mx > m_raw) != 0, 0)) {  // rare once the maxima settle
            const float m_new = fmaxf(m_raw, mx);
            const float alpha = __builtin_amdgcn_exp2f((m_raw - m_new) * c);
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
            m_raw = m_new;
            m_sc = m_new * c;
        }
        f32x16 s_next = s;
        if (has_next) s_next = s_phase(tk_next);
        uint32_t pp[8];
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
            const float p0 = __builtin_amdgcn_exp2f(fmaf(s[i], c, -m_sc));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(s[i + 1], c, -m_sc));
            sum += p0 + p1;
            pp[i >> 1] = M::pack(p0, p1);
        }
        l_run += sum;
        // ---- O^T += V^T . P^T.  k-step ks2 uses result rows 8*ks2..8*ks2+7 of the lane, i.e. keys
        //      key_base + 16*ks2 + 8*(e/4) + 4*half + e%4 for operand element e ----
#pragma unroll
        for (int ks2 = 0; ks2 < 2; ++ks2) {
            const X8 pb = __builtin_bit_cast(X8, uint4{pp[4 * ks2], pp[4 * ks2 + 1], pp[4 * ks2 + 2], pp[4 * ks2 + 3]});
            X8 va[DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int e = 0; e < 4; ++e) { va[dt][e] = vlo[dt][e]; va[dt][4 + e] = vhi[dt][e]; }
            if (ks2 == 0) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {  // operands of the second k-step, in flight during the first
                    vlo[dt] = M::tr_read(tv + 16 * G::RB + v_ofs[dt]);
                    vhi[dt] = M::tr_read(tv + 24 * G::RB + v_ofs[dt]);
                }
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) o[dt] = M::mma(va[dt], pb, o[dt]);
        }
        return s_next;
    };

    // one K/V tile: wait for it, start the next one into the other buffer, multiply
    auto do_tile = [&](int tile, char *cur_k, char *cur_v, char *nxt_k, char *nxt_v) {
        __builtin_amdgcn_s_waitcnt(0);  // this wave's direct loads and zero fills of `tile` have landed
        __syncthreads();                // ... and everyone's; everyone is also done reading the other buffer
        if (tile + 1 < n_tiles) {
            issue(tile + 1, nxt_k, nxt_v);
            lookup(tile + 2);  // consumed by the next tile's issue()
        }
        const int key0 = tile * kPfKeys;
        if (key0 < my_keys) {  // else this wave's rows end before this tile (uniform per wave)
            // masking is needed only where the tile reaches past the first row's causal limit or the context end
            const bool need_mask = key0 + kPfKeys > prefix + row0 + 1 || key0 + kPfKeys > ctx_len;
            f32x16 s = s_phase(cur_k);
#pragma unroll
            for (int kt = 0; kt < kPfSub; ++kt)
                s = subtile(s, cur_k + (kt + 1) * 32 * G::RB, cur_v + kt * 32 * G::RB, key0 + 32 * kt, need_mask,
                            kt + 1 < kPfSub);
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
    if (!live) return;
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int row = row0 + col;
    if (row >= q_len) return;
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

typedef void (*prefill_mfma_fn)(const RowwiseArgs);
// nullptr if the shape has no matrix-core kernel; `bs16` selects the variant for pools of 16-token blocks
prefill_mfma_fn pa_prefill_mfma_kernel(int dtype, int d, bool bs16);

}  // namespace pa_decode_detail
