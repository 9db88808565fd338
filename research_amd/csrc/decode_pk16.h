// Packed inner loop of single-query-row paged attention for gfx950: bf16 / fp16
// pools (head_dim 64, 128, 256) and fp8-e4m3 pools with bf16 / fp16 queries
// (head_dim 64, 128, 256).  An fp8 pool is widened two elements at a time to
// the query type (v_cvt_scalef32_pk_*_fp8, exact) and then runs the same
// 16-bit arithmetic; its per-(block, head) scales multiply the logit and p.
//
// The generic loop converts every K/V element to fp32 and spends most of its
// issue slots on conversions, per-head cross-lane sums and redundant softmax
// arithmetic.  This loop keeps the pool data packed:
//   * q.k: v_dot2 on the raw 16-bit pairs (fp32 accumulate), no conversion;
//   * the NREP per-head partial dots of a lane are combined over the LPR lanes
//     of a row with a reduce-scatter in DPP moves, so each lane ends up owning
//     the logit of ONE (token, head) (two for NREP = 8) and the exp2 / running
//     max / running sum are evaluated once, not once per lane;
//   * p.v: two tokens at a time, v_perm interleaves their V pairs and v_dot2
//     accumulates p(t0)*v(t0)+p(t1)*v(t1) with p rounded to the pool type; the
//     p pair of head h is broadcast inside the quad by a DPP move;
//   * loads are buffer loads against a per-block descriptor whose size is the
//     number of valid bytes in the block: rows past the sequence end read as
//     zero without a branch, and no index can leave the block.
#pragma once
#include "pa_common.h"

namespace pa_decode_detail {

typedef unsigned int pa_u4 __attribute__((ext_vector_type(4)));

// Cache policy of the K/V stream: every byte is used once, so the loads carry
// the non-temporal hint (bit 1 of the buffer-load policy operand = "nt").
// Measured on MI355X with a pure read of 3.4 GB in 32 KiB pages: 6.2 TB/s with
// default loads, 7.0 TB/s with nt loads.
constexpr int kStreamPolicy = 2;

template <typename KV> struct Pk16;
template <> struct Pk16<pa_bf16> {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), c, false);
    }
    // a.b with no addend: the three-operand encoding with the constant 0 (the compiler's choice for dot2 with a
    // zero addend is the accumulating encoding behind a v_mov of 0: one more instruction per chain)
    static __device__ __forceinline__ float dot2_first(uint32_t a, uint32_t b) {
        float d;
        asm("v_dot2_f32_bf16 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
        return d;
    }
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        v2 r = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, r);
    }
};
template <> struct Pk16<pa_f16> {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), c, false);
    }
    static __device__ __forceinline__ float dot2_first(uint32_t a, uint32_t b) {
        float d;
        asm("v_dot2_f32_f16 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
        return d;
    }
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        v2 r = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, r);
    }
};

// How the 16 bytes a lane loads turn into packed pairs of the arithmetic type AT.
template <typename KV, typename AT> struct PoolWords;
template <typename AT> struct PoolWords<AT, AT> {  // 16-bit pool: the raw dwords are the pairs
    static constexpr int NW = 4;
    static __device__ __forceinline__ void unpack(const pa_u4 &raw, uint32_t (&w)[NW]) {
        w[0] = raw[0]; w[1] = raw[1]; w[2] = raw[2]; w[3] = raw[3];
    }
    // The rows of two tokens as pairs across the tokens: lo[i] = (t0[2i], t1[2i]), hi[i] = (t0[2i+1], t1[2i+1]).
    static __device__ __forceinline__ void interleave(const pa_u4 &t0, const pa_u4 &t1, uint32_t (&lo)[NW], uint32_t (&hi)[NW]) {
#pragma unroll
        for (int i = 0; i < NW; ++i) {
            lo[i] = __builtin_amdgcn_perm(t1[i], t0[i], 0x05040100u);
            hi[i] = __builtin_amdgcn_perm(t1[i], t0[i], 0x07060302u);
        }
    }
};
template <> struct PoolWords<pa_fp8, pa_bf16> {
    static constexpr int NW = 8;
    static __device__ __forceinline__ void unpack(const pa_u4 &raw, uint32_t (&w)[NW]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            w[2 * i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw[i], 1.0f, false));
            w[2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw[i], 1.0f, true));
        }
    }
    // Pairs across two tokens: the bytes of the two rows are interleaved first (two byte permutes per dword of
    // four elements) and widened after, so every widening delivers a finished pair - 6 instructions per four
    // elements of both tokens instead of 4 widenings and 4 permutes of the widened words.
    static __device__ __forceinline__ void interleave(const pa_u4 &t0, const pa_u4 &t1, uint32_t (&lo)[NW], uint32_t (&hi)[NW]) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t a = __builtin_amdgcn_perm(t1[k], t0[k], 0x05010400u);  // t0.b0 t1.b0 t0.b1 t1.b1
            const uint32_t b = __builtin_amdgcn_perm(t1[k], t0[k], 0x07030602u);  // t0.b2 t1.b2 t0.b3 t1.b3
            lo[2 * k] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(a, 1.0f, false));
            hi[2 * k] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(a, 1.0f, true));
            lo[2 * k + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(b, 1.0f, false));
            hi[2 * k + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(b, 1.0f, true));
        }
    }
};
template <> struct PoolWords<pa_fp8, pa_f16> {
    static constexpr int NW = 8;
    static __device__ __forceinline__ void unpack(const pa_u4 &raw, uint32_t (&w)[NW]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            w[2 * i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[i], 1.0f, false));
            w[2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[i], 1.0f, true));
        }
    }
    // Pairs across two tokens: the bytes of the two rows are interleaved first (two byte permutes per dword of
    // four elements) and widened after, so every widening delivers a finished pair - 6 instructions per four
    // elements of both tokens instead of 4 widenings and 4 permutes of the widened words.
    static __device__ __forceinline__ void interleave(const pa_u4 &t0, const pa_u4 &t1, uint32_t (&lo)[NW], uint32_t (&hi)[NW]) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint32_t a = __builtin_amdgcn_perm(t1[k], t0[k], 0x05010400u);  // t0.b0 t1.b0 t0.b1 t1.b1
            const uint32_t b = __builtin_amdgcn_perm(t1[k], t0[k], 0x07030602u);  // t0.b2 t1.b2 t0.b3 t1.b3
            lo[2 * k] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(a, 1.0f, false));
            hi[2 * k] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(a, 1.0f, true));
            lo[2 * k + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(b, 1.0f, false));
            hi[2 * k + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(b, 1.0f, true));
        }
    }
};

template <int CTRL, int BANKS = 0xf> __device__ __forceinline__ float dpp_mov(float old, float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old),
                                                                 __builtin_bit_cast(int, x), CTRL, 0xf, BANKS, false));
}
template <int CTRL> __device__ __forceinline__ uint32_t dpp_mov_u(uint32_t x) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xf, 0xf, true);
}

// How NREP per-head values of a lane are combined over the LPR lanes of a row.
// After reduce(): a lane at quad position c = lane & 3 owns VPL totals, those
// of heads head_base(c) .. head_base(c)+VPL-1.
template <int NREP, int LPR> struct HeadScatter {
    static_assert(LPR == 4 || LPR == 8 || LPR == 16 || LPR == 32, "rows of 4, 8, 16 or 32 lanes");
    static constexpr int SC = NREP >= 4 ? 2 : (NREP == 2 ? 1 : 0);  // scatter steps (xor 1, xor 2)
    static constexpr int VPL = NREP >> SC;                            // values a lane keeps

    // The scatter steps exchange between lane pairs (xor 1, then xor 2): a lane keeps half of its values and adds
    // the partner's other half.  Which half a lane keeps would depend on its position in the quad - a select per
    // value - so instead the lanes hold their query heads in different orders: local index j of a lane stands for
    // head j ^ swizzle(lane).  Then every lane keeps its first half and receives the partner's second half, one
    // DPP add per value, and ends up owning local values 0 .. VPL-1 = heads head_of(0 .. VPL-1, lane).
    static __device__ __forceinline__ int swizzle(int lane) {
        return (SC >= 1 ? (lane & 1) * (NREP / 2) : 0) ^ (SC == 2 ? ((lane >> 1) & 1) * VPL : 0);
    }
    static __device__ __forceinline__ int head_of(int j, int lane) { return j ^ swizzle(lane); }

    // s[j]: this lane's partial dot product of head head_of(j, lane).
    static __device__ __forceinline__ void reduce(const float (&s)[NREP], float (&out)[VPL], int lane) {
        constexpr int H1 = SC >= 1 ? NREP / 2 : NREP;
        float t[H1];
        if (SC >= 1) {
#pragma unroll
            for (int i = 0; i < H1; ++i) t[i] = s[i] + dpp_mov<0xB1>(0.f, s[i + H1]);  // quad_perm [1,0,3,2]
        } else {
#pragma unroll
            for (int i = 0; i < H1; ++i) t[i] = s[i] + dpp_mov<0xB1>(0.f, s[i]);
        }
        if (SC == 2) {
#pragma unroll
            for (int i = 0; i < VPL; ++i) out[i] = t[i] + dpp_mov<0x4E>(0.f, t[i + VPL]);  // quad_perm [2,3,0,1]
        } else {
#pragma unroll
            for (int i = 0; i < VPL; ++i) out[i] = t[i] + dpp_mov<0x4E>(0.f, t[i]);
        }
        // remaining levels keep the quad position: every quad of the row gets the row total
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            if (LPR >= 16) {
                out[i] += dpp_mov<0x124>(0.f, out[i]);  // row_ror:4
                out[i] += dpp_mov<0x128>(0.f, out[i]);  // row_ror:8
                if (LPR == 32) {  // the row spans two groups of 16 lanes: add the partner group's total
                    const uint32_t u = __builtin_bit_cast(uint32_t, out[i]);
                    const auto sw = __builtin_amdgcn_permlane16_swap(u, u, false, false);
                    out[i] = __builtin_bit_cast(float, (uint32_t)sw[0]) + __builtin_bit_cast(float, (uint32_t)sw[1]);
                }
            } else if (LPR == 8) {
                // partner quad inside the row of 8: from 4 lanes below for banks 1,3, from 4 lanes above for banks 0,2
                float other = dpp_mov<0x114, 0xa>(0.f, out[i]);   // row_shr:4
                other = dpp_mov<0x104, 0x5>(other, out[i]);       // row_shl:4
                out[i] += other;
            }
        }
    }

    // quad position and slot that hold head h
    static constexpr int pos_of(int h) {
        return SC == 2 ? ((h / (NREP / 2)) | (((h / VPL) & 1) << 1)) : (SC == 1 ? h : 0);
    }
    static constexpr int slot_of(int h) { return SC == 2 ? h % VPL : 0; }

    template <int H> static __device__ __forceinline__ float bcast(const float (&x)[VPL]) {
        if (SC == 0) return x[0];
        return dpp_mov<pos_of(H) * 0x55>(0.f, x[slot_of(H)]);
    }
    template <int H> static __device__ __forceinline__ uint32_t bcast_u(const uint32_t (&x)[VPL]) {
        if (SC == 0) return x[0];
        return dpp_mov_u<pos_of(H) * 0x55>(x[slot_of(H)]);
    }
};

// A 64-bit value that is the same in every lane, as two scalar halves.
__device__ __forceinline__ int64_t uniform64(int64_t x) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)x), hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)x >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

template <int NREP, int VPL, int EPL> struct PkState {
    float m[VPL], l[VPL];
    float acc[NREP][EPL];
    int zero_keys;
    __device__ __forceinline__ void init() {
#pragma unroll
        for (int j = 0; j < VPL; ++j) { m[j] = -1.0e30f; l[j] = 0.f; }
#pragma unroll
        for (int r = 0; r < NREP; ++r)
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[r][e] = 0.f;
        zero_keys = 0;
    }
};

template <int N> struct StaticFor {
    template <typename F> static __device__ __forceinline__ void run(F &&f) {
        StaticFor<N - 1>::run(f);
        f(std::integral_constant<int, N - 1>{});
    }
};
template <> struct StaticFor<0> {
    template <typename F> static __device__ __forceinline__ void run(F &&) {}
};

// Attend keys [k_lo, L) of this wave's share of blocks [blk_first, blk_end), which the n_waves waves of the
// workgroup divide among themselves.  A chunk is the U token steps a wave keeps in flight (p.tpw * U tokens); a
// block holds cpb = ceil(block_size / chunk) of them.  The largest multiple of n_waves blocks is dealt out block by
// block (a wave streams whole blocks: one table entry and one descriptor per block) and the up to n_waves - 1
// blocks left over chunk by chunk, so the waves' shares differ by one chunk at most however short the run is
// (the waves meet at a barrier behind every run).  With `by_chunk` the whole run is dealt chunk by chunk: the
// chunks of a block are then requested by neighbouring waves at the same time instead of by one wave one after
// the other.  Measured on MI355X (32 query / 8 kv heads of 128): dealing everything by chunk takes about 2 us off
// a bf16 launch whatever its length (16 sequences of 4 096 to 65 536 keys; the 64-sequence ragged batch of
// 0.14 M keys: 99.4 -> 96.5 us) but costs the 256-sequence batch of 0.84 M keys 0.8 % (540 -> 545 us), so the
// split pass asks for it in launches of at most kChunkDealUnits blocks per workgroup; dealing only the left-over
// blocks by chunk took 3 us off the long-context fp8 launch (274 -> 271 us).
// qpk[r][i]: packed pairs of this lane's query elements of head r (raw bits of the query type AT).
// lane_kvh: the kv head this lane's row belongs to (selects the fp8 scales).
// SHORT: a chunk exceeds the block (cpb = 1), so whole token steps can lie past the block's end; they are skipped
// under uniform branches.  The straight-line form (SHORT = false) keeps the loop free of branches for the layouts
// where every step of a full chunk is live.
template <typename KV, typename AT, int D, int NREP, int U, bool SHORT>
__device__ __forceinline__ void attend_blocks_pk(
    PkState<NREP, HeadScatter<NREP, D * (int)sizeof(KV) / 16>::VPL, 2 * PoolWords<KV, AT>::NW> &st,
    const uint32_t (&qpk)[NREP][PoolWords<KV, AT>::NW], const PoolArgs &p, const int32_t *bt_row, int k_lo, int L,
    int blk_first, int blk_end, int wave, int n_waves, int cpb, bool by_chunk, int lane, int lane_voff, int lane_kvh,
    bool count_zero_keys) {
    static_assert(U % 2 == 0, "tokens are consumed in pairs");
    constexpr int LPR = D * (int)sizeof(KV) / 16;
    constexpr bool kFp8 = sizeof(KV) == 1;
    using HS = HeadScatter<NREP, LPR>;
    using PK = Pk16<AT>;
    using PW = PoolWords<KV, AT>;
    constexpr int NW = PW::NW;
    constexpr int VPL = HS::VPL;
    const int tok_stride = p.hkv * p.d * (int)sizeof(KV);  // bytes between tokens
    const int tok_local = (lane / LPR) / p.hpw;
    const int chunk = p.tpw * U;                          // tokens per chunk

    int voff[U];  // byte offset of this lane's 16 bytes in token step u of a chunk
#pragma unroll
    for (int u = 0; u < U; ++u) voff[u] = lane_voff + u * p.tpw * tok_stride;
    // chunk-by-chunk dealing indexes chunks with shifts, so it needs a power-of-two number of chunks per block
    const bool can_chunk = cpb > 1 && (cpb & (cpb - 1)) == 0;
    const int whole = !can_chunk ? blk_end - blk_first : by_chunk ? 0 : (blk_end - blk_first) / n_waves * n_waves;
    // phase 0: whole blocks, wave w takes blocks first+w, first+w+n_waves, ...; phase 1: the chunks of the blocks
    // not dealt out in phase 0, wave w takes chunks w, w+n_waves, ... of them.  One loop serves both: its index o
    // counts blocks (shift 0, a span of one block) or chunks (shift log2 cpb, a span of one chunk).
    for (int phase = 0; phase < 2; ++phase) {
    const int sh = phase == 0 ? 0 : __builtin_ctz(cpb);
    const int span = phase == 0 ? p.bs : chunk;
    const int o_begin = phase == 0 ? blk_first + wave : ((blk_first + whole) << sh) + wave;
    const int o_end = phase == 0 ? blk_first + whole : blk_end << sh;
    // the table entry of a step's block is requested one step ahead, so its latency is off the wave's critical path
    int64_t bid_next = o_begin < o_end && (o_begin >> sh) < p.bt_stride ? (int64_t)bt_row[o_begin >> sh] : -1;
    for (int o = o_begin; o < o_end; o += n_waves) {
        const int cur_blk = o >> sh;
        const int64_t bid = uniform64(bid_next);  // (a scalar from here on: the address arithmetic stays off the vector unit)
        {
            const int nb = (o + n_waves) >> sh;
            bid_next = o + n_waves < o_end && nb < p.bt_stride ? (int64_t)bt_row[nb] : -1;
        }
        const int ntok = min(p.bs, L - cur_blk * p.bs);
        const int tlo = max(0, k_lo - cur_blk * p.bs);  // tokens below it lie before the window (first block only)
        const int t_begin = (o - (cur_blk << sh)) * chunk, t_end = min(ntok, t_begin + span);  // this step's tokens
        if (bid < 0 || bid >= p.num_blocks) {
            if (count_zero_keys) st.zero_keys += max(0, t_end - max(tlo, t_begin));
            continue;
        }
        const int64_t block_off = bid * p.bs * (int64_t)tok_stride;
        float k_sc = p.scale_log2, v_sc = 1.f;  // logit scale (with the K scale folded in) and V scale of this block
        if (kFp8) {
            k_sc *= p.k_scale[bid * p.hkv + lane_kvh];
            v_sc = p.v_scale[bid * p.hkv + lane_kvh];
        }

        for (int t0 = t_begin; t0 < t_end; t0 += chunk) {
            if (t0 + chunk <= tlo) continue;  // the whole chunk lies before the window
            // descriptors of the valid rows of the block from t0 on: reads past them return 0.  The per-lane
            // offsets of the U token steps are loop invariants (voff), so a load costs no address arithmetic.
            const int64_t chunk_off = block_off + (int64_t)t0 * tok_stride;
            const int valid = (ntok - t0) * tok_stride;
            const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(reinterpret_cast<const char *>(p.k) + chunk_off), 0, valid, 0x00020000);
            const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(reinterpret_cast<const char *>(p.v) + chunk_off), 0, valid, 0x00020000);
            pa_u4 kraw[U], vraw[U];
#pragma unroll
            for (int u = 0; u < U; ++u) kraw[u] = __builtin_amdgcn_raw_buffer_load_b128(rk, voff[u], 0, kStreamPolicy);
#pragma unroll
            for (int u = 0; u < U; ++u) vraw[u] = __builtin_amdgcn_raw_buffer_load_b128(rv, voff[u], 0, kStreamPolicy);

            // ---- logits: one (token, head) per lane -----------------------
            float sv[U][VPL];
            const int rem = ntok - t0;                   // tokens of the block from t0 on (uniform)
            const bool partial = rem < chunk || t0 < tlo;  // uniform
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (SHORT && u * p.tpw >= rem) {  // uniform: the whole token step lies past the block
#pragma unroll
                    for (int j = 0; j < VPL; ++j) sv[u][j] = -INFINITY;
                    continue;
                }
                uint32_t kw[NW];
                PW::unpack(kraw[u], kw);
                float s[NREP];
#pragma unroll
                for (int r = 0; r < NREP; ++r) {
                    float d = PK::dot2_first(kw[0], qpk[r][0]);
#pragma unroll
                    for (int i = 1; i < NW; ++i) d = PK::dot2(kw[i], qpk[r][i], d);
                    s[r] = d;
                }
                HS::reduce(s, sv[u], lane);
#pragma unroll
                for (int j = 0; j < VPL; ++j) sv[u][j] *= k_sc;
            }
            if (partial) {
                // kept a branch (the empty statement stops the compiler from turning it into selects that every
                // step would execute): only the first and last block of a sequence have tokens to mask
                asm volatile("");
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int tt = t0 + u * p.tpw + tok_local;
                    const bool ok = tt < ntok && tt >= tlo;
#pragma unroll
                    for (int j = 0; j < VPL; ++j) sv[u][j] = ok ? sv[u][j] : -INFINITY;
                }
            }
            // ---- running maximum; rescale only when some lane's maximum grew ----
            float mx[VPL];
            bool grew = false;
#pragma unroll
            for (int j = 0; j < VPL; ++j) {
                mx[j] = st.m[j];
#pragma unroll
                for (int u = 0; u < U; ++u) mx[j] = fmaxf(mx[j], sv[u][j]);
                grew |= mx[j] > st.m[j];
            }
            if (__builtin_amdgcn_ballot_w64(grew) != 0) {
                float alpha[VPL];
#pragma unroll
                for (int j = 0; j < VPL; ++j) {
                    alpha[j] = __builtin_amdgcn_exp2f(st.m[j] - mx[j]);
                    st.m[j] = mx[j];
                    st.l[j] *= alpha[j];
                }
                StaticFor<NREP>::run([&](auto h) {
                    const float a = HS::template bcast<h.value>(alpha);
#pragma unroll
                    for (int e = 0; e < 2 * NW; ++e) st.acc[h.value][e] *= a;
                });
            }
            // ---- p.v, two tokens per step ----------------------------------
#pragma unroll
            for (int u = 0; u < U; u += 2) {
                if (SHORT && u * p.tpw >= rem) continue;  // uniform: both token steps lie past the block
                uint32_t ppk[VPL];
#pragma unroll
                for (int j = 0; j < VPL; ++j) {
                    const float p0 = __builtin_amdgcn_exp2f(sv[u][j] - st.m[j]);  // 0 for masked tokens
                    const float p1 = __builtin_amdgcn_exp2f(sv[u + 1][j] - st.m[j]);
                    st.l[j] += p0 + p1;
                    ppk[j] = kFp8 ? PK::pack(p0 * v_sc, p1 * v_sc) : PK::pack(p0, p1);
                }
                uint32_t lo[NW], hi[NW];  // (v_t0[2i], v_t1[2i]) and (v_t0[2i+1], v_t1[2i+1])
                PW::interleave(vraw[u], vraw[u + 1], lo, hi);
                StaticFor<NREP>::run([&](auto h) {
                    const uint32_t pb = HS::template bcast_u<h.value>(ppk);
#pragma unroll
                    for (int i = 0; i < NW; ++i) {
                        st.acc[h.value][2 * i] = PK::dot2(lo[i], pb, st.acc[h.value][2 * i]);
                        st.acc[h.value][2 * i + 1] = PK::dot2(hi[i], pb, st.acc[h.value][2 * i + 1]);
                    }
                });
            }
        }
    }
    }  // phase
}

// The same loop for layouts where a token step of the wave covers several tokens and a block holds only SPB
// steps (one kv head per load, 16-token blocks): the U steps in flight are taken from G = U / SPB consecutive
// blocks of the wave, each through its own descriptor, so the number of loads in flight and the work per loop
// entry stay what they are for wide layouts.  Requires p.bs == SPB * p.tpw.
template <typename KV, typename AT, int D, int NREP, int U, int SPB>
__device__ __forceinline__ void attend_blocks_pk_multi(
    PkState<NREP, HeadScatter<NREP, D * (int)sizeof(KV) / 16>::VPL, 2 * PoolWords<KV, AT>::NW> &st,
    const uint32_t (&qpk)[NREP][PoolWords<KV, AT>::NW], const PoolArgs &p, const int32_t *bt_row, int k_lo, int L,
    int blk_begin, int blk_end, int blk_step, int lane, int lane_voff, int lane_kvh, bool count_zero_keys) {
    static_assert(U % SPB == 0 && SPB % 2 == 0, "whole blocks per iteration, token pairs inside one block");
    constexpr int G = U / SPB;  // blocks per iteration
    constexpr int LPR = D * (int)sizeof(KV) / 16;
    constexpr bool kFp8 = sizeof(KV) == 1;
    using HS = HeadScatter<NREP, LPR>;
    using PK = Pk16<AT>;
    using PW = PoolWords<KV, AT>;
    constexpr int NW = PW::NW;
    constexpr int VPL = HS::VPL;
    const int tok_stride = p.hkv * p.d * (int)sizeof(KV);  // bytes between tokens
    const int tok_local = (lane / LPR) / p.hpw;

    for (int blk0 = blk_begin; blk0 < blk_end; blk0 += G * blk_step) {
        int ntok[G], tlo[G];
        float k_sc[G], v_sc[G];
        __amdgpu_buffer_rsrc_t rk[G], rv[G];
        bool partial = false;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int blk = blk0 + g * blk_step;
            const bool in_range = blk < blk_end;
            ntok[g] = in_range ? min(p.bs, L - blk * p.bs) : 0;
            tlo[g] = in_range ? max(0, k_lo - blk * p.bs) : 0;
            const int64_t bid = in_range && blk < p.bt_stride ? (int64_t)bt_row[blk] : -1;
            const bool ok = bid >= 0 && bid < p.num_blocks;
            if (!ok) {
                if (in_range && count_zero_keys) st.zero_keys += max(0, ntok[g] - tlo[g]);
                ntok[g] = 0;
            }
            // descriptor of the valid part of this block (empty for a missing block): reads past it return 0
            const int64_t block_off = (ok ? bid : 0) * p.bs * (int64_t)tok_stride;
            rk[g] = __builtin_amdgcn_make_buffer_rsrc((void *)(reinterpret_cast<const char *>(p.k) + block_off), 0,
                                                      ntok[g] * tok_stride, 0x00020000);
            rv[g] = __builtin_amdgcn_make_buffer_rsrc((void *)(reinterpret_cast<const char *>(p.v) + block_off), 0,
                                                      ntok[g] * tok_stride, 0x00020000);
            k_sc[g] = p.scale_log2;
            v_sc[g] = 1.f;
            if (kFp8 && ok) {
                k_sc[g] *= p.k_scale[bid * p.hkv + lane_kvh];
                v_sc[g] = p.v_scale[bid * p.hkv + lane_kvh];
            }
            partial |= ntok[g] < p.bs || tlo[g] > 0;
        }

        pa_u4 kraw[U], vraw[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
            kraw[u] = __builtin_amdgcn_raw_buffer_load_b128(rk[u / SPB], lane_voff + (u % SPB) * p.tpw * tok_stride, 0,
                                                            kStreamPolicy);
#pragma unroll
        for (int u = 0; u < U; ++u)
            vraw[u] = __builtin_amdgcn_raw_buffer_load_b128(rv[u / SPB], lane_voff + (u % SPB) * p.tpw * tok_stride, 0,
                                                            kStreamPolicy);

        // ---- logits: one (token, head) per lane -----------------------
        float sv[U][VPL];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int g = u / SPB, s0 = (u % SPB) * p.tpw;  // block of the step, its first token in the block
            if (partial && s0 >= ntok[g]) {  // uniform: the whole step lies past the block's end
#pragma unroll
                for (int j = 0; j < VPL; ++j) sv[u][j] = -INFINITY;
                continue;
            }
            uint32_t kw[NW];
            PW::unpack(kraw[u], kw);
            float s[NREP];
#pragma unroll
            for (int r = 0; r < NREP; ++r) {
                float d = PK::dot2_first(kw[0], qpk[r][0]);
#pragma unroll
                for (int i = 1; i < NW; ++i) d = PK::dot2(kw[i], qpk[r][i], d);
                s[r] = d;
            }
            HS::reduce(s, sv[u], lane);
#pragma unroll
            for (int j = 0; j < VPL; ++j) sv[u][j] *= k_sc[g];
            if (partial) {
                const int tt = s0 + tok_local;
                const bool ok = tt < ntok[g] && tt >= tlo[g];
#pragma unroll
                for (int j = 0; j < VPL; ++j) sv[u][j] = ok ? sv[u][j] : -INFINITY;
            }
        }
        // ---- running maximum; rescale only when some lane's maximum grew ----
        float mx[VPL];
        bool grew = false;
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            mx[j] = st.m[j];
#pragma unroll
            for (int u = 0; u < U; ++u) mx[j] = fmaxf(mx[j], sv[u][j]);
            grew |= mx[j] > st.m[j];
        }
        if (__builtin_amdgcn_ballot_w64(grew) != 0) {
            float alpha[VPL];
#pragma unroll
            for (int j = 0; j < VPL; ++j) {
                alpha[j] = __builtin_amdgcn_exp2f(st.m[j] - mx[j]);
                st.m[j] = mx[j];
                st.l[j] *= alpha[j];
            }
            StaticFor<NREP>::run([&](auto h) {
                const float a = HS::template bcast<h.value>(alpha);
#pragma unroll
                for (int e = 0; e < 2 * NW; ++e) st.acc[h.value][e] *= a;
            });
        }
        // ---- p.v, two tokens per step ----------------------------------
#pragma unroll
        for (int u = 0; u < U; u += 2) {
            const int g = u / SPB;
            if (partial && (u % SPB) * p.tpw >= ntok[g]) continue;  // uniform: both steps lie past the block's end
            uint32_t ppk[VPL];
#pragma unroll
            for (int j = 0; j < VPL; ++j) {
                const float p0 = __builtin_amdgcn_exp2f(sv[u][j] - st.m[j]);  // 0 for masked tokens
                const float p1 = __builtin_amdgcn_exp2f(sv[u + 1][j] - st.m[j]);
                st.l[j] += p0 + p1;
                ppk[j] = kFp8 ? PK::pack(p0 * v_sc[g], p1 * v_sc[g]) : PK::pack(p0, p1);
            }
            uint32_t lo[NW], hi[NW];  // (v_t0[2i], v_t1[2i]) and (v_t0[2i+1], v_t1[2i+1])
            PW::interleave(vraw[u], vraw[u + 1], lo, hi);
            StaticFor<NREP>::run([&](auto h) {
                const uint32_t pb = HS::template bcast_u<h.value>(ppk);
#pragma unroll
                for (int i = 0; i < NW; ++i) {
                    st.acc[h.value][2 * i] = PK::dot2(lo[i], pb, st.acc[h.value][2 * i]);
                    st.acc[h.value][2 * i + 1] = PK::dot2(hi[i], pb, st.acc[h.value][2 * i + 1]);
                }
            });
        }
    }
}

}  // namespace pa_decode_detail
