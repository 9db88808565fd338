// Paged attention of single query rows for gfx950: the split-K decode kernel,
// its reduction pass, and a row-per-workgroup kernel that evaluates causal
// prefill one query row at a time (the vector path for element types that
// have no matrix-core kernel).
//
// Work decomposition (decode)
//   plane = (group of <= NREP query heads per kv head, group of HPW kv heads).
//   The (plane, sequence, pool block) space is flattened and cut into equal
//   ranges, one per 256-thread workgroup of a grid sized to the machine, so
//   that every workgroup streams the same number of blocks however ragged the
//   batch is.  Each workgroup first builds the per-sequence block prefix sum in
//   LDS (seq_lens live on the device, the host never reads them) and finds the
//   sequences of its range by binary search in it.
//
// Lane layout (wave64)
//   A K or V row of one (token, kv head) is D elements = LPR lanes x 16 bytes,
//   so one 128-bit load instruction of a wave fetches RPW = 64/LPR rows.  The
//   pool is token-major ([slot][kv_head][d]); the RPW rows are mapped to HPW
//   neighbouring kv heads of TPW consecutive tokens (HPW*TPW = RPW) so that a
//   wave's load covers HPW*D contiguous elements per token.  The NREP query
//   heads that share a kv head are all evaluated from the same registers: each
//   K/V byte is loaded once.
//
// Softmax
//   base-2 online softmax in fp32 per row group, rescaled once per batch of U
//   token steps; the partial (m, l, acc) of the 4 waves x TPW token rows are
//   merged through LDS.  A sequence that one workgroup covers alone is written
//   out directly; where a sequence straddles workgroup ranges each piece leaves
//   a partial in the workspace and a second kernel merges them.
#pragma once
#include <type_traits>
#include <utility>

#include "decode_plan.h"
#include "pa_common.h"

namespace pa_decode_detail {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / PA_WAVE;
constexpr int kMaxBatch = kPlanMaxBatch;  // sequences per call (their block prefix sum lives in LDS)
constexpr float kNegBig = -1.0e30f;  // finite stand-in for -inf in running maxima
constexpr int kDeadLaneOffset = 0x40000000;  // byte offset past every buffer descriptor (a block is under 2 GiB / 4)

// What every kernel of this file needs to know about the pool and the heads.
struct PoolArgs {
    const void *k, *v;
    const int32_t *bt;
    int64_t bt_stride;
    const float *k_scale, *v_scale;
    int hq, hkv, n_rep, bs;
    int d;  // head_dim of the tensors in memory; the kernels' D is d rounded up to 32, 64, 128 or 256 and the lanes
            // (and d indices) at or past d hold zeros and store nothing
    int64_t num_blocks;
    float scale_log2;  // softmax scale * log2(e)
    int window;        // sliding window: a query at position i sees keys j with i - j < window (0 = all keys)
    int hpw, tpw, n_hgroups, n_rgroups;
};

struct DecodeArgs {
    PoolArgs p;
    const void *q;
    void *out;
    const int32_t *seq_lens;
    const int32_t *extra_zero;
    int batch;
    int split_grid;         // workgroups of the split pass (the reduction pass needs the same number)
    int64_t slot_cap;       // partial slots the workspace holds
    float *part_acc;        // [slot_cap][hpw*NREP][D]
    float *part_ml;         // [slot_cap][hpw*NREP][2]
    int32_t *block_prefix;  // [batch+1], written by the split pass for the reduction pass
    unsigned long long *tickets;        // [planes*batch]: arrivals per (plane, sequence); zero between launches
    unsigned long long *group_tickets;  // [2*split_grid]: arrivals per group of pieces of a many-piece sequence
    int merge_in_split;     // the workgroup that delivers a sequence's last piece merges the pieces (no second pass)
};

struct RowwiseArgs {
    PoolArgs p;
    const void *q;
    void *out;
    const int32_t *ctx_lens, *q_lens, *q_starts;
    const int32_t *row_lo;  // per query row: first key it sees (NULL = none); non-decreasing along a sequence
    int batch;
    int max_q_len;
    // Matrix-core kernels only: a workgroup's tiles cut into `splits` pieces, each run by a workgroup of its own
    // (grid.y = groups * splits) that leaves (m, l) and the unnormalised O rows of its piece in the workspace for
    // the merge kernel: part_o float [row][head][split][D], part_ml float [row][head][split][2].  1 = no split.
    int splits;
    float *part_o, *part_ml;
    // prefill_asm_kernel without lower bounds: groups of 8 tasks one workgroup runs in turn (grid.y = chunks of that
    // many groups); 1 everywhere else.
    int groups_per_wg;
};

__device__ __forceinline__ uint4 ld16(const void *p) { return *reinterpret_cast<const uint4 *>(p); }

// First key a query at position n_keys-1 sees under the sliding window (0 without one).
__device__ __forceinline__ int window_first_key(const PoolArgs &p, int n_keys) {
    return plan_first_key(n_keys, p.window);
}

// 16-byte load of pool data: used once, so it carries the non-temporal hint.
__device__ __forceinline__ uint4 ld16_stream(const void *p) {
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    const u4 v = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p));
    return uint4{v[0], v[1], v[2], v[3]};
}

template <typename KV, int D> struct RowShape {
    static constexpr int EPL = pa_vec16<KV>::N;  // elements per lane per 16-byte load
    static constexpr int LPR = D / EPL;          // lanes per row
    static constexpr int RPW = PA_WAVE / LPR;    // rows per wave load
    static_assert(D % EPL == 0 && LPR >= 1 && LPR <= 64 && (LPR & (LPR - 1)) == 0, "row shape");
};

// Fixed role of a lane within its wave.
struct LaneRole {
    int row, lir, head_local, tok_local, d0;
};
template <typename KV, int D> __device__ __forceinline__ LaneRole lane_role(int lane, const PoolArgs &p) {
    using S = RowShape<KV, D>;
    LaneRole r;
    r.row = lane / S::LPR;
    r.lir = lane - r.row * S::LPR;
    r.head_local = r.row % p.hpw;
    r.tok_local = r.row / p.hpw;
    r.d0 = r.lir * S::EPL;
    return r;
}

// Running softmax state of one row group for NREP query heads.
template <int NREP, int EPL> struct RowState {
    float m[NREP], l[NREP], acc[NREP][EPL];
    int zero_keys;  // keys of missing blocks (logit 0, value 0) seen by this row group
    __device__ __forceinline__ void init() {
#pragma unroll
        for (int r = 0; r < NREP; ++r) {
            m[r] = kNegBig;
            l[r] = 0.f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[r][e] = 0.f;
        }
        zero_keys = 0;
    }
    __device__ __forceinline__ void fold_zero_keys() {
        if (zero_keys <= 0) return;
#pragma unroll
        for (int r = 0; r < NREP; ++r) {
            const float mn = fmaxf(m[r], 0.f);
            const float alpha = __builtin_amdgcn_exp2f(m[r] - mn);
            l[r] = l[r] * alpha + (float)zero_keys * __builtin_amdgcn_exp2f(-mn);
#pragma unroll
            for (int e = 0; e < EPL; ++e) acc[r][e] *= alpha;
            m[r] = mn;
        }
        zero_keys = 0;
    }
};

// This lane's slice of the NREP query heads of kv head `kvh`, pre-multiplied by
// scale*log2(e).  `qrow` points at [num_q_heads][D] of the query row.
template <typename QT, int D, int NREP, int EPL>
__device__ __forceinline__ void load_q(float (&qf)[NREP][EPL], const QT *qrow, const PoolArgs &p, int kvh,
                                       int rep0, int d0) {
#pragma unroll
    for (int r = 0; r < NREP; ++r) {
        const bool live = rep0 + r < p.n_rep && d0 < p.d;
        const QT *qp = qrow + ((int64_t)kvh * p.n_rep + rep0 + (live ? r : 0)) * p.d + (live ? d0 : 0);
#pragma unroll
        for (int e = 0; e < EPL; ++e) qf[r][e] = live ? pa_scalar<QT>::load(qp + e) * p.scale_log2 : 0.f;
    }
}

// Attend keys [k_lo, L) restricted to blocks blk_begin, blk_begin+blk_step, ... < blk_end
// of the block-table row `bt_row`, for kv head `kvh`.
template <typename KV, int D, int NREP, int U>
__device__ __forceinline__ void attend_blocks(RowState<NREP, RowShape<KV, D>::EPL> &st,
                                              const float (&qf)[NREP][RowShape<KV, D>::EPL], const PoolArgs &p,
                                              const int32_t *bt_row, int k_lo, int L, int blk_begin, int blk_end,
                                              int blk_step, const LaneRole &role, int kvh) {
    using S = RowShape<KV, D>;
    constexpr int EPL = S::EPL;
    constexpr bool kFp8 = sizeof(KV) == 1;
    const int64_t tok_stride = (int64_t)p.hkv * p.d * sizeof(KV);  // bytes between tokens
    const bool lane_live = role.d0 < p.d;                          // (lanes past the row's end read nothing)

    for (int blk = blk_begin; blk < blk_end; blk += blk_step) {
        const int ntok = min(p.bs, L - blk * p.bs);
        const int tlo = max(0, k_lo - blk * p.bs);  // tokens below it lie before the window
        const int64_t bid = blk < p.bt_stride ? (int64_t)bt_row[blk] : -1;
        if (bid < 0 || bid >= p.num_blocks) {
            if (role.tok_local == 0) st.zero_keys += max(0, ntok - tlo);
            continue;
        }
        const int64_t base = ((bid * p.bs) * p.hkv + kvh) * (int64_t)(p.d * sizeof(KV)) + (int64_t)role.lir * 16;
        const char *kp = reinterpret_cast<const char *>(p.k) + base;
        const char *vp = reinterpret_cast<const char *>(p.v) + base;
        float ks = 1.f, vs = 1.f;
        if (kFp8) {
            ks = p.k_scale[bid * p.hkv + kvh];
            vs = p.v_scale[bid * p.hkv + kvh];
        }
        for (int t0 = 0; t0 < ntok; t0 += p.tpw * U) {
            uint4 kraw[U], vraw[U];
            bool ok[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int t = t0 + u * p.tpw + role.tok_local;
                ok[u] = t < ntok && t >= tlo;
                kraw[u] = ok[u] && lane_live ? ld16_stream(kp + t * tok_stride) : uint4{0, 0, 0, 0};
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int t = t0 + u * p.tpw + role.tok_local;
                vraw[u] = ok[u] && lane_live ? ld16_stream(vp + t * tok_stride) : uint4{0, 0, 0, 0};
            }
            float s[U][NREP];
            float mx[NREP];
#pragma unroll
            for (int r = 0; r < NREP; ++r) mx[r] = st.m[r];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float kf[EPL];
                pa_vec16<KV>::unpack(kraw[u], kf);
#pragma unroll
                for (int r = 0; r < NREP; ++r) {
                    float d = 0.f;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) d = fmaf(qf[r][e], kf[e], d);
                    d = pa_group_sum<S::LPR>(d);
                    if (kFp8) d *= ks;
                    s[u][r] = ok[u] ? d : -INFINITY;
                    mx[r] = fmaxf(mx[r], s[u][r]);
                }
            }
#pragma unroll
            for (int r = 0; r < NREP; ++r) {
                const float alpha = __builtin_amdgcn_exp2f(st.m[r] - mx[r]);
                st.m[r] = mx[r];
                st.l[r] *= alpha;
#pragma unroll
                for (int e = 0; e < EPL; ++e) st.acc[r][e] *= alpha;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float vf[EPL];
                pa_vec16<KV>::unpack(vraw[u], vf);
#pragma unroll
                for (int r = 0; r < NREP; ++r) {
                    float pr = __builtin_amdgcn_exp2f(s[u][r] - st.m[r]);  // 0 for masked steps
                    st.l[r] += pr;
                    if (kFp8) pr *= vs;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) st.acc[r][e] = fmaf(pr, vf[e], st.acc[r][e]);
                }
            }
        }
    }
}

}  // namespace pa_decode_detail

#include "decode_pk16.h"

namespace pa_decode_detail {

// One wave's pass over its blocks of one query row: picks the packed 16-bit
// loop where it applies (bf16/fp16 pool, head_dim 64, 128 or 256), else the generic
// fp32 loop.  Returns the row-group state in the generic form merge_rows takes.
template <typename KV, typename QT, int D, int NREP, int U> struct Attender {
    using S = RowShape<KV, D>;
    // packed loop: 16-bit pools and fp8 pools (16-bit queries) with head_dim 64/128/256
    static constexpr bool kPacked =
        (sizeof(KV) == 2 && std::is_same<KV, QT>::value && (D == 64 || D == 128 || D == 256)) ||
        (sizeof(KV) == 1 && sizeof(QT) == 2 && (D == 64 || D == 128 || D == 256));

    // Blocks [blk_first, blk_end) of the row are shared out among the `n_waves` waves of the workgroup; this is
    // wave `wave`'s share: alternate blocks in the generic and the several-blocks-per-iteration loops, alternate
    // chunks of a block (the U token steps of one iteration) in the packed loop when `by_chunk` asks for it.
    static __device__ __forceinline__ RowState<NREP, S::EPL> run(const PoolArgs &p, const QT *qrow,
                                                                  const int32_t *bt_row, int k_lo, int L,
                                                                  int blk_first, int blk_end, int wave, int n_waves,
                                                                  bool by_chunk, const LaneRole &role, int lane,
                                                                  int kvh, int rep0) {
        RowState<NREP, S::EPL> out;
        const int blk_begin = blk_first + wave, blk_step = n_waves;
        if constexpr (kPacked) {
            using HS = HeadScatter<NREP, S::LPR>;
            constexpr int NW = S::EPL / 2;  // packed pairs per lane
            uint32_t qpk[NREP][NW];
#pragma unroll
            for (int r = 0; r < NREP; ++r) {
                // local index r of this lane stands for head head_of(r, lane): the order that spares the
                // reduce-scatter of the logits its selects
                const int hr = HS::head_of(r, lane);
                const bool live = rep0 + hr < p.n_rep && role.d0 < p.d;
                const QT *qp = qrow + ((int64_t)kvh * p.n_rep + rep0 + hr) * p.d + role.d0;
#pragma unroll
                for (int i = 0; i < NW; i += 4) {
                    const uint4 raw = live ? ld16(qp + 2 * i) : uint4{0, 0, 0, 0};
                    qpk[r][i] = raw.x; qpk[r][i + 1] = raw.y; qpk[r][i + 2] = raw.z; qpk[r][i + 3] = raw.w;
                }
            }
            PkState<NREP, HS::VPL, S::EPL> st;
            st.init();
            // (a lane past the end of a head_dim that is not 32, 64, 128 or 256 gets an offset no descriptor covers:
            // its loads return zeros)
            const int lane_voff = role.d0 < p.d ? role.tok_local * (p.hkv * p.d * (int)sizeof(KV)) +
                                                      kvh * (p.d * (int)sizeof(KV)) + role.lir * 16
                                                : kDeadLaneOffset;
            // uniform choices: few kv heads per wave load and short blocks
            if (U % 4 == 0 && p.bs == 4 * p.tpw && U > 4)  // 4 steps per block: U/4 blocks per iteration
                attend_blocks_pk_multi<KV, QT, D, NREP, U, (U % 4 == 0 ? 4 : 2)>(
                    st, qpk, p, bt_row, k_lo, L, blk_begin, blk_end, blk_step, lane, lane_voff, kvh, role.tok_local == 0);
            else if (p.bs == 2 * p.tpw)  // 2 steps per block
                attend_blocks_pk_multi<KV, QT, D, NREP, U, 2>(st, qpk, p, bt_row, k_lo, L, blk_begin, blk_end, blk_step,
                                                              lane, lane_voff, kvh, role.tok_local == 0);
            else if (p.tpw * U > p.bs)
                attend_blocks_pk<KV, QT, D, NREP, U, true>(st, qpk, p, bt_row, k_lo, L, blk_first, blk_end, wave, n_waves,
                                                           1, false, lane, lane_voff, kvh, role.tok_local == 0);
            else
                attend_blocks_pk<KV, QT, D, NREP, U, false>(st, qpk, p, bt_row, k_lo, L, blk_first, blk_end, wave,
                                                            n_waves, (p.bs + p.tpw * U - 1) / (p.tpw * U), by_chunk,
                                                            lane, lane_voff, kvh, role.tok_local == 0);
            StaticFor<NREP>::run([&](auto h) {
                out.m[h.value] = HS::template bcast<h.value>(st.m);
                out.l[h.value] = HS::template bcast<h.value>(st.l);
#pragma unroll
                for (int e = 0; e < S::EPL; ++e) out.acc[h.value][e] = st.acc[h.value][e];
            });
            out.zero_keys = st.zero_keys;
        } else {
            float qf[NREP][S::EPL];
            load_q<QT, D, NREP, S::EPL>(qf, qrow, p, kvh, rep0, role.d0);
            out.init();
            attend_blocks<KV, D, NREP, U>(out, qf, p, bt_row, k_lo, L, blk_begin, blk_end, blk_step, role, kvh);
        }
        return out;
    }
};

// Merge the kWaves*TPW row-group partials of every (kv head of the group,
// query head r) through LDS and hand (qh, d, num[4], M, den) of the merged
// partial - four consecutive d at a time - to `emit`; out = num/den, M is the
// base-2 running maximum.
//
// The waves' lanes hold ROWS = kWaves*RPW partial rows per query head; rows
// with the same row % hpw belong to the same kv head and are merged.  HR query
// heads go through LDS per round (as many as the LDS budget allows): every
// lane writes its accumulators, then one thread per (head, row) computes the
// row's weight exp2(m_row - M) (and, for the first row of each kv head, M and
// the merged denominator), then one thread per (head, kv head, d) sums
// weight * accumulator over the rows.  The row loops are unrolled by 4 (the
// row count per kv head is kWaves*tpw, a multiple of 4) so that their LDS
// reads overlap.
template <typename KV, int D, int NREP> struct MergeShape {
    static constexpr int ROWS = kWaves * RowShape<KV, D>::RPW;
    static constexpr int ROWF = D + 2;  // floats of a partial row: D accumulators, m, l
    static constexpr int kBudget = 28 * 1024;
    static constexpr int per_head = ROWS * (ROWF + 3) * 4;  // bytes: rows + (weight, M, den) per row
    static constexpr int HR = NREP >= 8 && 8 * per_head <= kBudget   ? 8
                              : NREP >= 4 && 4 * per_head <= kBudget ? 4
                              : NREP >= 2 && 2 * per_head <= kBudget ? 2
                                                                     : 1;
    static constexpr int AUX = HR * ROWS * ROWF;   // float offset of the weights
    static constexpr int FLOATS = HR * ROWS * (ROWF + 3);
    // the host-visible statement of the same arithmetic (the launch checks the workgroup's LDS against it)
    static_assert(ROWS == plan_merge_rows(D, (int)sizeof(KV)) && HR == plan_merge_heads_per_round(D, (int)sizeof(KV), NREP) &&
                      FLOATS == plan_merge_floats(D, (int)sizeof(KV), NREP),
                  "decode_plan.h and MergeShape disagree");
};

template <typename KV, int D, int NREP, typename Emit>
__device__ __forceinline__ void merge_rows(RowState<NREP, RowShape<KV, D>::EPL> &st, float *s_part,
                                           const PoolArgs &p, const LaneRole &role, int wave, int tid, int hg,
                                           int rep0, Emit emit) {
    using S = RowShape<KV, D>;
    using MS = MergeShape<KV, D, NREP>;
    constexpr int ROWS = MS::ROWS, ROWF = MS::ROWF, HR = MS::HR;
    st.fold_zero_keys();
    const int prow = wave * S::RPW + role.row;  // = wave*RPW + tok_local*hpw + head_local
    float *s_wgt = s_part + MS::AUX, *s_M = s_wgt + HR * ROWS, *s_den = s_M + HR * ROWS;
    const int hpw = p.hpw;  // a power of two dividing RPW
    const int lg_hpw = __builtin_ctz(hpw);
#pragma unroll
    for (int round = 0; round < NREP / HR; ++round) {
        if (rep0 + round * HR >= p.n_rep) break;  // uniform over the workgroup
        __syncthreads();  // the readers of the previous round (or of the previous call) are done
#pragma unroll
        for (int h = 0; h < HR; ++h) {
            float *row = s_part + (h * ROWS + prow) * ROWF;
#pragma unroll
            for (int e = 0; e < S::EPL; ++e) row[role.d0 + e] = st.acc[round * HR + h][e];
            if (role.lir == 0) {
                row[D] = st.m[round * HR + h];
                row[D + 1] = st.l[round * HR + h];
            }
        }
        __syncthreads();
        for (int idx = tid; idx < HR * ROWS; idx += kThreads) {
            const int h = idx / ROWS, row = idx - h * ROWS;
            const int hl = row & (hpw - 1);
            const float *base = s_part + h * ROWS * ROWF;
            float M = kNegBig;
#pragma unroll 4
            for (int r2 = hl; r2 < ROWS; r2 += hpw) M = fmaxf(M, base[r2 * ROWF + D]);
            s_wgt[idx] = __builtin_amdgcn_exp2f(base[row * ROWF + D] - M);
            if (row < hpw) {  // first row of its kv head: the merged maximum and denominator
                float den = 0.f;
#pragma unroll 4
                for (int r2 = hl; r2 < ROWS; r2 += hpw)
                    den = fmaf(__builtin_amdgcn_exp2f(base[r2 * ROWF + D] - M), base[r2 * ROWF + D + 1], den);
                s_M[idx] = M;
                s_den[idx] = den;
            }
        }
        __syncthreads();
        // four consecutive d per thread: the results leave as one 16-byte store (a part's partial is 8 KB and
        // more; as single floats its stores were a measurable share of the pass)
        for (int o = tid; o < HR * hpw * (D / 4); o += kThreads) {
            const int d = (o & (D / 4 - 1)) * 4, hd = o / (D / 4);
            const int hl = hd & (hpw - 1), h = hd >> lg_hpw;
            const int r = round * HR + h;
            if (rep0 + r >= p.n_rep) continue;
            const float *base = s_part + h * ROWS * ROWF + d;
            const float *wgt = s_wgt + h * ROWS;
            float num[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
            for (int r2 = hl; r2 < ROWS; r2 += hpw) {
                const float w = wgt[r2];
#pragma unroll
                for (int j = 0; j < 4; ++j) num[j] = fmaf(w, base[r2 * ROWF + j], num[j]);
            }
            emit((hg * hpw + hl) * p.n_rep + rep0 + r, d, num, s_M[h * ROWS + hl], s_den[h * ROWS + hl]);
        }
    }
    __syncthreads();
}

// The partition arithmetic (which workgroup owns which blocks, where its partial goes) is in decode_plan.h.
__device__ __forceinline__ int64_t unit_begin(int64_t w, int64_t total, int64_t grid) { return plan_unit_begin(w, total, grid); }
__device__ __forceinline__ int owner_of(int64_t u, int64_t total, int64_t grid) { return plan_owner_of(u, total, grid); }
__device__ __forceinline__ int effective_grid(int64_t total, int grid) { return plan_effective_grid(total, grid); }

// Finish one (sequence, query head): fold `ez` extra all-zero keys into the
// merged (num, M, den) and normalise.
__device__ __forceinline__ float finish_row(float num, float M, float den, int ez) {
    if (ez > 0) {
        const float mn = fmaxf(M, 0.f);
        const float alpha = __builtin_amdgcn_exp2f(M - mn);
        num *= alpha;
        den = den * alpha + (float)ez * __builtin_amdgcn_exp2f(-mn);
    }
    return den > 0.f ? num / den : 0.f;
}

// Partials that another workgroup merges inside the same launch travel between compute dies (each XCD has its own
// L2): they are written and read as device-scope 8-byte accesses, which go through to the memory side.  Ordinary
// stores would need a write-back of the whole L2 before the ticket is counted (what a device-scope release fence
// does), which costs far more than the merge saves.
__device__ __forceinline__ void st_coherent(float *p, float a, float b) {
    const unsigned long long v = (unsigned long long)__builtin_bit_cast(uint32_t, a) |
                                 ((unsigned long long)__builtin_bit_cast(uint32_t, b) << 32);
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float2 ld_coherent(const float *p) {
    const unsigned long long v = __hip_atomic_load(reinterpret_cast<const unsigned long long *>(p), __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
    return float2{__builtin_bit_cast(float, (uint32_t)v), __builtin_bit_cast(float, (uint32_t)(v >> 32))};
}
// Every memory access this thread has issued is complete (a device-scope store has then reached the memory side),
// and the compiler moves no access across this point.
__device__ __forceinline__ void wait_all_memory() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void compiler_fence() { asm volatile("" ::: "memory"); }

// Arrival counting.  A ticket is a 64-bit counter in the zero-filled region at the start of the workspace.  One
// thread of a workgroup, after the workgroup's stores are complete, adds one; the arrival that brings the count to
// `expected` is the last one: it puts the counter back to zero (nobody else touches it any more in this launch),
// so every launch - also a replay of a captured graph - finds every ticket at zero.
__device__ __forceinline__ bool arrive_is_last(unsigned long long *ticket, int expected) {
    const unsigned long long old = __hip_atomic_fetch_add(ticket, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool last = old + 1 >= (unsigned long long)expected;
    if (last) __hip_atomic_store(ticket, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return last;
}

// How the pieces w0..w1 of one (plane, sequence) are merged inside the split pass.  Up to kInlinePieces pieces: the
// workgroup that delivers the last of them merges them all.  More (one sequence that dominates its batch is cut
// into hundreds): the pieces form groups of `group` consecutive workgroups, the last arrival of a group merges the
// group into the slot of the group's first piece, and the last group to finish merges the groups - two levels of
// at most 32 partials each instead of one workgroup reading hundreds.
constexpr int kInlinePieces = 8;
struct PieceTree {
    int pieces, group, n_groups;
};
__device__ __forceinline__ PieceTree piece_tree(int pieces) {
    PieceTree t;
    t.pieces = pieces;
    t.group = pieces <= kInlinePieces ? pieces : pieces <= 64 ? 8 : pieces <= 256 ? 16 : 32;
    t.n_groups = (pieces + t.group - 1) / t.group;
    return t;
}

// Merge `count` partials of (plane, sequence b) - the slots of workgroups w_first, w_first + stride, ... - one
// thread per (query head, four consecutive d), the loads of PIPE partials in flight at a time.  FINAL: normalise and
// write the plane's output rows; otherwise leave the merged partial in the slot of workgroup w_first (every thread
// overwrites exactly what it has itself read).
template <typename QT, int D, int NREP, bool FINAL>
__device__ __forceinline__ void merge_slots(const DecodeArgs &a, int plane, int b, int hg, int rep0, int w_first,
                                            int count, int stride, int tid) {
    constexpr int PIPE = 4;
    const PoolArgs &p = a.p;
    const int stride_acc = p.hpw * NREP * D, stride_ml = p.hpw * NREP * 2;
    const int64_t key = (int64_t)plane * a.batch + b;
    const int ez = FINAL && a.extra_zero ? max(0, a.extra_zero[b]) : 0;
    QT *orow = reinterpret_cast<QT *>(a.out) + (int64_t)b * p.hq * p.d;
    for (int item = tid; item < p.hpw * NREP * (D / 4); item += kThreads) {
        const int idx = item / (D / 4), d = (item - idx * (D / 4)) * 4;
        const int kv_local = idx / NREP, r = idx - kv_local * NREP;
        if (rep0 + r >= p.n_rep) continue;
        float M = kNegBig, den = 0.f, num[4] = {0.f, 0.f, 0.f, 0.f};
        for (int i = 0; i < count; i += PIPE) {
            float m[PIPE], l[PIPE];
            float4 x[PIPE];
#pragma unroll
            for (int j = 0; j < PIPE; ++j) {
                const int64_t want = (int64_t)w_first + (int64_t)(i + j) * stride + key;
                const bool have = i + j < count && want < a.slot_cap;
                const int64_t slot = have ? want : w_first + key;
                const float2 ml = ld_coherent(a.part_ml + slot * stride_ml + idx * 2);
                const float2 lo = ld_coherent(a.part_acc + slot * stride_acc + idx * D + d);
                const float2 hi = ld_coherent(a.part_acc + slot * stride_acc + idx * D + d + 2);
                x[j] = float4{lo.x, lo.y, hi.x, hi.y};
                m[j] = have ? ml.x : kNegBig;
                l[j] = have ? ml.y : 0.f;
                if (!have) x[j] = float4{0.f, 0.f, 0.f, 0.f};
            }
            float mn = M;
#pragma unroll
            for (int j = 0; j < PIPE; ++j) mn = fmaxf(mn, m[j]);
            const float so = __builtin_amdgcn_exp2f(M - mn);
            den *= so;
#pragma unroll
            for (int k = 0; k < 4; ++k) num[k] *= so;
#pragma unroll
            for (int j = 0; j < PIPE; ++j) {
                const float sn = __builtin_amdgcn_exp2f(m[j] - mn);
                den = fmaf(l[j], sn, den);
                num[0] = fmaf(x[j].x, sn, num[0]);
                num[1] = fmaf(x[j].y, sn, num[1]);
                num[2] = fmaf(x[j].z, sn, num[2]);
                num[3] = fmaf(x[j].w, sn, num[3]);
            }
            M = mn;
        }
        if (FINAL) {
            const int qh = (hg * p.hpw + kv_local) * p.n_rep + rep0 + r;
            if (d >= p.d) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                pa_scalar<QT>::store(orow + (int64_t)qh * p.d + d + j, finish_row(num[j], M, den, ez));
        } else if ((int64_t)w_first + key < a.slot_cap) {
            const int64_t slot = w_first + key;
            st_coherent(a.part_acc + slot * stride_acc + idx * D + d, num[0], num[1]);
            st_coherent(a.part_acc + slot * stride_acc + idx * D + d + 2, num[2], num[3]);
            if (d == 0) st_coherent(a.part_ml + slot * stride_ml + idx * 2, M, den);
        }
    }
}

// A piece of (plane, sequence b) that this workgroup has just stored; w0..w1 are the workgroups holding pieces of it.
struct PieceRef {
    int plane, b, hg, rep0, w0, w1;
};

// Count the piece and do whatever merging falls to this workgroup.  s_flag: one LDS word.
template <typename QT, int D, int NREP>
__device__ __forceinline__ void deliver_piece(const DecodeArgs &a, const PieceRef &pp, int *s_flag, int tid) {
    const PieceTree t = piece_tree(pp.w1 - pp.w0 + 1);
    const int me = (int)blockIdx.x - pp.w0;  // index of this workgroup's piece
    const int g = me / t.group;
    const int g_first = pp.w0 + g * t.group;                      // workgroup of the group's first piece
    const int g_count = min(t.group, t.pieces - g * t.group);     // pieces of this group
    unsigned long long *seq_ticket = a.tickets + ((int64_t)pp.plane * a.batch + pp.b);
    // a group's ticket is found by the workgroup of its first piece; a workgroup can be that for the sequence that
    // runs on into it (a later group of it) and for the sequence that starts in it (group 0 of it)
    unsigned long long *grp_ticket = a.group_tickets + (2 * (int64_t)g_first + (g == 0 ? 1 : 0));
    wait_all_memory();  // this thread's stores have reached the memory side
    __syncthreads();
    if (tid == 0) *s_flag = arrive_is_last(t.n_groups == 1 ? seq_ticket : grp_ticket, g_count);
    __syncthreads();
    compiler_fence();  // the pieces are read after the count, never before
    if (!*s_flag) return;  // uniform
    if (t.n_groups == 1) {
        merge_slots<QT, D, NREP, true>(a, pp.plane, pp.b, pp.hg, pp.rep0, pp.w0, t.pieces, 1, tid);
        return;
    }
    merge_slots<QT, D, NREP, false>(a, pp.plane, pp.b, pp.hg, pp.rep0, g_first, g_count, 1, tid);
    wait_all_memory();
    __syncthreads();
    if (tid == 0) *s_flag = arrive_is_last(seq_ticket, t.n_groups);
    __syncthreads();
    compiler_fence();
    if (!*s_flag) return;
    merge_slots<QT, D, NREP, true>(a, pp.plane, pp.b, pp.hg, pp.rep0, pp.w0, t.n_groups, t.group, tid);
}

// Launches with at most this many blocks per workgroup deal a run of blocks out to the waves chunk by chunk.
constexpr int kChunkDealUnits = 64;

// Batches up to this size get their block prefix sum from every wave on its own (no barrier); larger ones from the
// workgroup's scan through LDS.
constexpr int kWaveScanBatch = 512;

// Inclusive prefix sum of x over the 64 lanes of a wave: four shifted adds inside each row of 16 lanes (a lane
// with no source in its row adds 0), then the totals of the rows before a lane's own, read through scalars.
__device__ __forceinline__ int wave_inclusive_scan(int x, int lane) {
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false);  // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false);  // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false);  // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false);  // row_shr:8
    const int t0 = __builtin_amdgcn_readlane(x, 15), t1 = __builtin_amdgcn_readlane(x, 31),
              t2 = __builtin_amdgcn_readlane(x, 47);
    const int row = lane >> 4;
    return x + (row >= 1 ? t0 : 0) + (row >= 2 ? t1 : 0) + (row >= 3 ? t2 : 0);
}

// Split pass.  The (plane, sequence, block) space - plane = (rep group, head
// group) - is flattened in that order and cut into gridDim.x equal ranges, one
// per workgroup, so every workgroup streams the same number of pool blocks
// whatever the length distribution.  A range may cover the tail of one
// sequence, several whole sequences and the head of another.  A sequence that
// lies inside one range is finished in place; otherwise the workgroup leaves a
// partial in slot (workgroup index + plane*batch + sequence), unique because
// both terms only grow along the flattened order.
template <typename KV, typename QT, int D, int NREP, int U>
__global__ __launch_bounds__(kThreads) void decode_split_kernel(const DecodeArgs a) {
    using S = RowShape<KV, D>;
    extern __shared__ int s_prefix[];  // batch + 1 entries: blocks before each sequence
    __shared__ int s_scan[kThreads];
    __shared__ float s_part[MergeShape<KV, D, NREP>::FLOATS];
    __shared__ int s_last;  // this workgroup delivered the last piece of the sequence it just finished a part of

    const PoolArgs &p = a.p;
    const int tid = threadIdx.x;
    const int lane = tid & (PA_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / PA_WAVE);
    const int B = a.batch;

    // ---- block prefix sum over the batch --------------------------------
    // blocks of sequence b that hold visible keys: [first_key(b) / bs, ceil(L / bs))
    auto blocks_of = [&](int b) { return plan_blocks_of(a.seq_lens[b], p.bs, p.window); };
    if (B <= kWaveScanBatch) {
        // Every wave computes the whole prefix sum by itself: lane l of round c holds sequence 64 c + l, the lengths
        // of all rounds are requested at once, a round is scanned with data-parallel moves and the rounds are
        // chained through a scalar.  All four waves store the same values to the same LDS words and each reads
        // back what it has itself written, so no barrier stands between the lengths and the first table entry.
        int n[kWaveScanBatch / PA_WAVE];
#pragma unroll
        for (int c = 0; c < kWaveScanBatch / PA_WAVE; ++c) {
            const int b = c * PA_WAVE + lane;
            n[c] = c * PA_WAVE < B && b < B ? blocks_of(b) : 0;
        }
        int carry = 0;
#pragma unroll
        for (int c = 0; c < kWaveScanBatch / PA_WAVE; ++c) {
            if (c * PA_WAVE >= B) break;  // uniform
            const int x = wave_inclusive_scan(n[c], lane);
            if (c * PA_WAVE + lane < B) s_prefix[c * PA_WAVE + lane] = carry + x - n[c];
            carry += __builtin_amdgcn_readlane(x, PA_WAVE - 1);
        }
        if (lane == 0) s_prefix[B] = carry;
        if (blockIdx.x == 0 && wave == 0)
            for (int b = lane; b <= B; b += PA_WAVE) a.block_prefix[b] = s_prefix[b];
    } else {
        const int per = (B + kThreads - 1) / kThreads;
        const int lo = min(B, tid * per), hi = min(B, lo + per);
        int sum = 0;
        for (int b = lo; b < hi; ++b) sum += blocks_of(b);
        s_scan[tid] = sum;
        __syncthreads();
        for (int off = 1; off < kThreads; off <<= 1) {
            const int add = tid >= off ? s_scan[tid - off] : 0;
            __syncthreads();
            s_scan[tid] += add;
            __syncthreads();
        }
        int run = s_scan[tid] - sum;  // exclusive
        for (int b = lo; b < hi; ++b) {
            s_prefix[b] = run;
            run += blocks_of(b);
        }
        if (tid == kThreads - 1) s_prefix[B] = s_scan[tid];
        __syncthreads();
        if (blockIdx.x == 0)
            for (int b = tid; b <= B; b += kThreads) a.block_prefix[b] = s_prefix[b];
    }
    const int64_t per_plane = s_prefix[B];
    const int planes = p.n_hgroups * p.n_rgroups;
    const int64_t total = per_plane * planes;
    const LaneRole role = lane_role<KV, D>(lane, p);
    if (a.merge_in_split) {
        // no second pass: sequences without a visible key get their zero rows here, dealt out over the grid
        for (int b = blockIdx.x; b < B; b += gridDim.x) {
            if (s_prefix[b + 1] != s_prefix[b]) continue;
            QT *orow = reinterpret_cast<QT *>(a.out) + (int64_t)b * p.hq * p.d;
            for (int i = tid; i < p.hq * p.d; i += kThreads) pa_scalar<QT>::store(orow + i, 0.f);
        }
    }
    if (total == 0) return;
    const int grid = effective_grid(total, (int)gridDim.x);
    if ((int)blockIdx.x >= grid) return;  // uniform

    int64_t cur = unit_begin(blockIdx.x, total, grid);
    const int64_t end = unit_begin((int64_t)blockIdx.x + 1, total, grid);
    const bool by_chunk = total <= (int64_t)kChunkDealUnits * grid;  // short launches: see attend_blocks_pk
    while (cur < end) {
        const int plane = (int)(cur / per_plane);
        const int off = (int)(cur - plane * per_plane);
        int lo = 0, hi = B;  // last b with prefix[b] <= off
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (s_prefix[mid] <= off) lo = mid; else hi = mid;
        }
        const int b = lo;
        const int nblk = s_prefix[b + 1] - s_prefix[b];
        const int blk0 = off - s_prefix[b];
        const int blk1 = (int)min((int64_t)nblk, blk0 + (end - cur));
        const int hg = plane % p.n_hgroups;
        const int rg = plane / p.n_hgroups;
        const int kvh = hg * p.hpw + role.head_local;
        const int rep0 = rg * NREP;
        const int L = a.seq_lens[b];
        const int k_lo = window_first_key(p, L);  // the query sits at position L-1
        const int fb = k_lo / p.bs;               // first block with a visible key

        RowState<NREP, S::EPL> st = Attender<KV, QT, D, NREP, U>::run(
            p, reinterpret_cast<const QT *>(a.q) + (int64_t)b * p.hq * p.d, p.bt + (int64_t)b * p.bt_stride, k_lo, L,
            fb + blk0, fb + blk1, wave, kWaves, by_chunk, role, lane, kvh, rep0);
        if (blk0 == 0 && blk1 == nblk) {
            // the whole sequence is ours: write the output row
            const int ez = a.extra_zero ? max(0, a.extra_zero[b]) : 0;
            QT *orow = reinterpret_cast<QT *>(a.out) + (int64_t)b * p.hq * p.d;
            merge_rows<KV, D, NREP>(st, s_part, p, role, wave, tid, hg, rep0,
                                    [&](int qh, int d, const float (&num)[4], float M, float den) {
                                        if (d >= p.d) return;
#pragma unroll
                                        for (int j = 0; j < 4; ++j)
                                            pa_scalar<QT>::store(orow + (int64_t)qh * p.d + d + j,
                                                                 finish_row(num[j], M, den, ez));
                                    });
        } else {
            const int64_t slot = plan_slot((int)blockIdx.x, plane, B, b);
            if (slot < a.slot_cap) {  // never write outside the workspace
                float *acc = a.part_acc + slot * (p.hpw * NREP * D);
                float *ml = a.part_ml + slot * (p.hpw * NREP * 2);
                merge_rows<KV, D, NREP>(st, s_part, p, role, wave, tid, hg, rep0,
                                        [&](int qh, int d, const float (&num)[4], float M, float den) {
                                            const int kv = qh / p.n_rep;
                                            const int idx = (kv - hg * p.hpw) * NREP + (qh - kv * p.n_rep - rep0);
                                            if (a.merge_in_split) {  // uniform: read by another workgroup of this launch
                                                st_coherent(acc + idx * D + d, num[0], num[1]);
                                                st_coherent(acc + idx * D + d + 2, num[2], num[3]);
                                                if (d == 0) st_coherent(ml + idx * 2, M, den);
                                            } else {
                                                *reinterpret_cast<float4 *>(acc + idx * D + d) =
                                                    float4{num[0], num[1], num[2], num[3]};
                                                if (d == 0) {
                                                    ml[idx * 2] = M;
                                                    ml[idx * 2 + 1] = den;
                                                }
                                            }
                                        });
            }
            if (a.merge_in_split) {
                // Count the piece; if it completes its sequence (or its group of pieces), merge.  Done right away
                // and not behind the next run of blocks: a workgroup's first piece is the tail of a sequence whose
                // head the workgroup before it delivers at its very end, so delivering early leaves that merge to
                // the neighbour instead of stacking two merges at this workgroup's own end (measured: 0.7 % of
                // the 256-sequence launch).
                const int64_t u0 = plane * per_plane + s_prefix[b];
                const PieceRef piece = {plane, b, hg, rep0, owner_of(u0, total, grid),
                                        owner_of(u0 + nblk - 1, total, grid)};
                deliver_piece<QT, D, NREP>(a, piece, &s_last, tid);
            }
        }
        cur += blk1 - blk0;
    }
}

// Reduction pass: one workgroup per (sequence, query head).  A long sequence in a small batch has a piece in every
// workgroup of the split pass, hundreds of them, and all of this pass is waiting for small loads, so the
// workgroup spreads them wide: thread (p, v) takes pieces p, p + PL, ... and the four consecutive d of 16-byte
// vector v, keeps kPipe pieces in flight (PL * kPipe pieces of the row per round trip), merges its pieces online,
// and the PL partial merges are combined through LDS.  Rows the split pass finished in place are skipped; empty
// sequences get their zeros here.
template <typename QT, int D, int NREP>
__global__ __launch_bounds__(kThreads) void decode_reduce_kernel(const DecodeArgs a) {
    constexpr int V4 = D / 4;             // 16-byte vectors of a row
    constexpr int PL = kThreads / V4;     // pieces taken side by side
    constexpr int kPipe = 8;
    static_assert(D % 4 == 0 && kThreads % V4 == 0 && PL >= 1, "row shape");
    __shared__ float s_num[PL][D];
    __shared__ float s_m[PL], s_l[PL];
    const PoolArgs &p = a.p;
    const int hq = p.hq;
    const int b = blockIdx.x / hq;
    const int qh = blockIdx.x - b * hq;
    const int kv = qh / p.n_rep, rep = qh - kv * p.n_rep;
    const int hg = kv / p.hpw, rg = rep / NREP;
    const int plane = rg * p.n_hgroups + hg;
    const int idx = (kv - hg * p.hpw) * NREP + (rep - rg * NREP);
    const int64_t per_plane = a.block_prefix[a.batch];
    const int64_t total = per_plane * p.n_hgroups * p.n_rgroups;
    const int nblk = a.block_prefix[b + 1] - a.block_prefix[b];
    const int ez = a.extra_zero ? max(0, a.extra_zero[b]) : 0;
    const int tid = threadIdx.x;
    QT *orow = reinterpret_cast<QT *>(a.out) + ((int64_t)b * hq + qh) * p.d;
    if (nblk == 0) {
        for (int d = tid; d < p.d; d += kThreads) pa_scalar<QT>::store(orow + d, 0.f);
        return;
    }
    const int64_t u0 = plane * per_plane + a.block_prefix[b];
    const int grid = effective_grid(total, a.split_grid);
    const int w0 = owner_of(u0, total, grid), w1 = owner_of(u0 + nblk - 1, total, grid);
    if (w0 == w1) return;  // finished by the split pass
    const int64_t key = (int64_t)plane * a.batch + b;
    const int stride_acc = p.hpw * NREP * D, stride_ml = p.hpw * NREP * 2;
    // every taking-part workgroup has units (effective_grid never exceeds the number of units), so every index
    // in [w0, w1] left a partial unless its slot fell outside the workspace
    const int v = tid % V4, pl = tid / V4;
    float M = kNegBig, den = 0.f, num[4] = {0.f, 0.f, 0.f, 0.f};
    for (int w = w0 + pl; w <= w1; w += PL * kPipe) {
        float m[kPipe], l[kPipe];
        float4 x[kPipe];
#pragma unroll
        for (int j = 0; j < kPipe; ++j) {
            const int wj = w + j * PL;
            const bool have = wj <= w1 && wj + key < a.slot_cap;
            const int64_t slot = (have ? wj : w0) + key;
            const float2 ml = *reinterpret_cast<const float2 *>(a.part_ml + slot * stride_ml + idx * 2);
            x[j] = *reinterpret_cast<const float4 *>(a.part_acc + slot * stride_acc + idx * D + 4 * v);
            m[j] = have ? ml.x : kNegBig;
            l[j] = have ? ml.y : 0.f;
            if (!have) x[j] = float4{0.f, 0.f, 0.f, 0.f};
        }
        float mn = M;
#pragma unroll
        for (int j = 0; j < kPipe; ++j) mn = fmaxf(mn, m[j]);
        const float so = __builtin_amdgcn_exp2f(M - mn);
        den *= so;
#pragma unroll
        for (int k = 0; k < 4; ++k) num[k] *= so;
#pragma unroll
        for (int j = 0; j < kPipe; ++j) {
            const float sn = __builtin_amdgcn_exp2f(m[j] - mn);
            den = fmaf(l[j], sn, den);
            num[0] = fmaf(x[j].x, sn, num[0]);
            num[1] = fmaf(x[j].y, sn, num[1]);
            num[2] = fmaf(x[j].z, sn, num[2]);
            num[3] = fmaf(x[j].w, sn, num[3]);
        }
        M = mn;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) s_num[pl][4 * v + k] = num[k];
    if (v == 0) {
        s_m[pl] = M;
        s_l[pl] = den;
    }
    __syncthreads();
    for (int d = tid; d < p.d; d += kThreads) {
        float Mt = kNegBig;
#pragma unroll
        for (int q = 0; q < PL; ++q) Mt = fmaxf(Mt, s_m[q]);
        float n = 0.f, dn = 0.f;
#pragma unroll
        for (int q = 0; q < PL; ++q) {
            const float wgt = __builtin_amdgcn_exp2f(s_m[q] - Mt);
            n = fmaf(wgt, s_num[q][d], n);
            dn = fmaf(wgt, s_l[q], dn);
        }
        pa_scalar<QT>::store(orow + d, finish_row(n, Mt, dn, ez));
    }
}

// Reduction pass for large batches: one wave per (sequence, query head), four
// heads per workgroup.  With many sequences a sequence has few pieces, so one
// wave merges them all (loads of four pieces in flight at a time) and no LDS
// merge or barrier is needed; a quarter of the workgroups of the kernel above.
template <typename QT, int D, int NREP>
__global__ __launch_bounds__(kThreads) void decode_reduce_wave_kernel(const DecodeArgs a) {
    constexpr int DPL = (D + PA_WAVE - 1) / PA_WAVE;  // d values per lane
    constexpr int PIPE = 4;
    const PoolArgs &p = a.p;
    const int hq = p.hq;
    const int lane = threadIdx.x & (PA_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / PA_WAVE);
    const int row = blockIdx.x * kWaves + wave;
    if (row >= a.batch * hq) return;
    const int b = row / hq;
    const int qh = row - b * hq;
    const int kv = qh / p.n_rep, rep = qh - kv * p.n_rep;
    const int hg = kv / p.hpw, rg = rep / NREP;
    const int plane = rg * p.n_hgroups + hg;
    const int idx = (kv - hg * p.hpw) * NREP + (rep - rg * NREP);
    const int64_t per_plane = a.block_prefix[a.batch];
    const int64_t total = per_plane * p.n_hgroups * p.n_rgroups;
    const int nblk = a.block_prefix[b + 1] - a.block_prefix[b];
    const int ez = a.extra_zero ? max(0, a.extra_zero[b]) : 0;
    QT *orow = reinterpret_cast<QT *>(a.out) + ((int64_t)b * hq + qh) * p.d;
    if (nblk == 0) {
        for (int d = lane; d < p.d; d += PA_WAVE) pa_scalar<QT>::store(orow + d, 0.f);
        return;
    }
    const int64_t u0 = plane * per_plane + a.block_prefix[b];
    const int grid = effective_grid(total, a.split_grid);
    const int w0 = owner_of(u0, total, grid), w1 = owner_of(u0 + nblk - 1, total, grid);
    if (w0 == w1) return;  // finished by the split pass
    const int64_t key = (int64_t)plane * a.batch + b;
    const int stride_acc = p.hpw * NREP * D, stride_ml = p.hpw * NREP * 2;
    auto has_piece = [&](int w) { return w <= w1 && w + key < a.slot_cap; };  // every workgroup in range has units
    float M = kNegBig, den = 0.f, num[DPL];
#pragma unroll
    for (int k = 0; k < DPL; ++k) num[k] = 0.f;
    for (int w = w0; w <= w1; w += PIPE) {
        float m[PIPE], l[PIPE], x[PIPE][DPL];
#pragma unroll
        for (int j = 0; j < PIPE; ++j) {
            const bool have = has_piece(w + j);
            const int64_t slot = have ? w + j + key : w0 + key;
            m[j] = have ? a.part_ml[slot * stride_ml + idx * 2] : kNegBig;
            l[j] = have ? a.part_ml[slot * stride_ml + idx * 2 + 1] : 0.f;
#pragma unroll
            for (int k = 0; k < DPL; ++k) {
                const int d = lane + PA_WAVE * k;
                x[j][k] = have && d < D ? a.part_acc[slot * stride_acc + idx * D + d] : 0.f;
            }
        }
        float mn = M;
#pragma unroll
        for (int j = 0; j < PIPE; ++j) mn = fmaxf(mn, m[j]);
        const float so = __builtin_amdgcn_exp2f(M - mn);
        den *= so;
#pragma unroll
        for (int k = 0; k < DPL; ++k) num[k] *= so;
#pragma unroll
        for (int j = 0; j < PIPE; ++j) {
            const float sn = __builtin_amdgcn_exp2f(m[j] - mn);
            den = fmaf(l[j], sn, den);
#pragma unroll
            for (int k = 0; k < DPL; ++k) num[k] = fmaf(x[j][k], sn, num[k]);
        }
        M = mn;
    }
#pragma unroll
    for (int k = 0; k < DPL; ++k) {
        const int d = lane + PA_WAVE * k;
        if (d < p.d) pa_scalar<QT>::store(orow + d, finish_row(num[k], M, den, ez));
    }
}

// Causal prefill, one workgroup per (sequence, query row, head group, rep
// group): query row i of sequence b attends keys [0, ctx_len - q_len + i].
template <typename KV, typename QT, int D, int NREP, int U>
__global__ __launch_bounds__(kThreads) void prefill_rowwise_kernel(const RowwiseArgs a) {
    using S = RowShape<KV, D>;
    __shared__ float s_part[MergeShape<KV, D, NREP>::FLOATS];
    const PoolArgs &p = a.p;
    const int tid = threadIdx.x;
    const int lane = tid & (PA_WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / PA_WAVE);
    const int b = blockIdx.z;
    const int i = blockIdx.y;
    const int q_len = a.q_lens[b];
    if (i >= q_len) return;  // uniform over the workgroup
    const int hg = blockIdx.x % p.n_hgroups;
    const int rg = blockIdx.x / p.n_hgroups;
    const int L = min(a.ctx_lens[b], a.ctx_lens[b] - q_len + i + 1);
    const LaneRole role = lane_role<KV, D>(lane, p);
    const int kvh = hg * p.hpw + role.head_local;
    const int rep0 = rg * NREP;
    const int64_t qrow = (int64_t)a.q_starts[b] + i;

    const int nblk = L > 0 ? (L + p.bs - 1) / p.bs : 0;
    int k_lo = window_first_key(p, max(L, 0));  // the row sits at position L-1
    if (a.row_lo) k_lo = max(k_lo, min(a.row_lo[qrow], L - 1));
    k_lo = max(k_lo, 0);
    RowState<NREP, S::EPL> st = Attender<KV, QT, D, NREP, U>::run(
        p, reinterpret_cast<const QT *>(a.q) + qrow * p.hq * p.d, p.bt + (int64_t)b * p.bt_stride, k_lo, L,
        k_lo / p.bs, nblk, wave, kWaves, false, role, lane, kvh, rep0);
    QT *orow = reinterpret_cast<QT *>(a.out) + qrow * p.hq * p.d;
    merge_rows<KV, D, NREP>(st, s_part, p, role, wave, tid, hg, rep0,
                            [&](int qh, int d, const float (&num)[4], float M, float den) {
                                if (d >= p.d) return;
#pragma unroll
                                for (int j = 0; j < 4; ++j)
                                    pa_scalar<QT>::store(orow + (int64_t)qh * p.d + d + j, den > 0.f ? num[j] / den : 0.f);
                            });
}

typedef void (*split_fn)(const DecodeArgs);
typedef void (*reduce_fn)(const DecodeArgs);
typedef void (*rowwise_fn)(const RowwiseArgs);

struct KernelSet {
    split_fn split = nullptr;
    reduce_fn reduce = nullptr;
    reduce_fn reduce_wave = nullptr;  // for batches with few pieces per sequence
    rowwise_fn rowwise = nullptr;
};

template <typename KV, typename QT, int D> KernelSet kernels_for_d(int nrep_t) {
    constexpr int U = sizeof(KV) == 1 && D == 32 ? 4 : 8;  // token steps in flight per wave (the fp8 pools' generic loop at head_dim 32 would spill with 8)
    KernelSet k;
    switch (nrep_t) {
    case 1: k.reduce = decode_reduce_kernel<QT, D, 1>; k.reduce_wave = decode_reduce_wave_kernel<QT, D, 1>; k.split = decode_split_kernel<KV, QT, D, 1, U>; k.rowwise = prefill_rowwise_kernel<KV, QT, D, 1, U>; break;
    case 2: k.reduce = decode_reduce_kernel<QT, D, 2>; k.reduce_wave = decode_reduce_wave_kernel<QT, D, 2>; k.split = decode_split_kernel<KV, QT, D, 2, U>; k.rowwise = prefill_rowwise_kernel<KV, QT, D, 2, U>; break;
    case 4: k.reduce = decode_reduce_kernel<QT, D, 4>; k.reduce_wave = decode_reduce_wave_kernel<QT, D, 4>; k.split = decode_split_kernel<KV, QT, D, 4, U>; k.rowwise = prefill_rowwise_kernel<KV, QT, D, 4, U>; break;
    case 8: k.reduce = decode_reduce_kernel<QT, D, 8>; k.reduce_wave = decode_reduce_wave_kernel<QT, D, 8>; k.split = decode_split_kernel<KV, QT, D, 8, U>; k.rowwise = prefill_rowwise_kernel<KV, QT, D, 8, U>; break;
    }
    return k;
}

template <typename KV, typename QT> KernelSet kernels_for(int d, int nrep_t) {
    switch (d) {
    case 32: return kernels_for_d<KV, QT, 32>(nrep_t);
    case 64: return kernels_for_d<KV, QT, 64>(nrep_t);
    case 128: return kernels_for_d<KV, QT, 128>(nrep_t);
    case 256: return kernels_for_d<KV, QT, 256>(nrep_t);
    }
    return KernelSet{};
}

// one definition each, in decode_inst_<type>.hip
KernelSet pa_kernels_bf16(int d, int nrep_t);
KernelSet pa_kernels_f16(int d, int nrep_t);
KernelSet pa_kernels_f32(int d, int nrep_t);
KernelSet pa_kernels_fp8(int q_dtype, int d, int nrep_t);

// Kernel set for (q dtype, KV dtype, head_dim, padded group size), empty if none.
KernelSet pa_pick_kernels(int q_dtype, int kv_dtype, int d, int nrep_t);

// Head-mapping fields of PoolArgs derived from the shapes; returns the padded
// group size (template NREP) or 0 when head_dim / dtype has no kernel.
int pa_fill_head_mapping(PoolArgs &p, int num_q_heads, int num_kv_heads, int head_dim, int kv_dtype);

}  // namespace pa_decode_detail
