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
//   workgroup = 4 waves; a wave owns 64 query rows (two 32-row MFMA column
//   tiles) of ONE query head; the 4 waves of a workgroup take 4 consecutive
//   (row block, query head of the kv head) tasks, so they share every K/V tile
//   (GQA packing: K/V are fetched once per kv head, not per query head).
//   grid.x = kv head (fastest): with 8 XCDs a kv head's K/V stays in one XCD's
//   L2 while all sequences and row blocks that share prefix blocks re-read it.
//   K/V tiles of 64 keys go global -> registers -> LDS (next tile's loads are
//   in flight while the current tile is multiplied); rows are padded in LDS
//   so the 128-bit operand reads and the transpose reads are conflict free.
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
constexpr int kPfRows = 64;   // query rows per wave
constexpr int kPfWaves = 4;

template <int D> struct PfLds {
    static constexpr int kRowBytesK = D * 2 + 16;               // +16 B: 16 keys x 16 B hit 64 distinct banks
    static constexpr int kRowBytesV = D * 2 + (D >= 64 ? 64 : 0);  // 4 keys x 64 B hit 64 distinct banks
    static constexpr int kBytesK = kPfKeys * kRowBytesK;
    static constexpr int kBytesV = kPfKeys * kRowBytesV;
};

template <typename T, int D>
__global__ __launch_bounds__(256) void prefill_mfma_kernel(const RowwiseArgs a) {
    using M = Mfma16<T>;
    using X8 = typename M::x8;
    using X4 = typename M::x4;
    using L = PfLds<D>;
    constexpr int KS = D / 16;            // k-steps of the first product
    constexpr int DT = D / 32;            // 32-wide d tiles of the second product
    constexpr int CPR = D / 8;            // 16-byte chunks per K/V row
    constexpr int LD = (kPfKeys * CPR) / 256;  // chunks a thread loads per tile and tensor
    static_assert(LD >= 1, "tile smaller than the workgroup");
    __shared__ __attribute__((aligned(16))) char s_k[L::kBytesK];
    __shared__ __attribute__((aligned(16))) char s_v[L::kBytesV];

    const PoolArgs &p = a.p;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;   // which 16 of the 32 keys / d values of a result tile
    const int col = lane & 31;    // query row inside a 32-row tile

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

    // ---- Q^T operand: row = row0 + 32*nt + col, d = 16*ks + 8*half .. +8 ----
    const T *qbase = reinterpret_cast<const T *>(a.q) + ((int64_t)a.q_starts[b] * p.hq + qh) * D;
    X8 qreg[2][KS];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
        const int row = row0 + 32 * nt + col;
        const bool ok = live && row < q_len;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            uint4 raw = ok ? ld16(qbase + (int64_t)row * p.hq * D + 16 * ks + 8 * half) : uint4{0, 0, 0, 0};
            qreg[nt][ks] = __builtin_bit_cast(X8, raw);
        }
    }

    f32x16 o[2][DT];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[nt][dt][i] = 0.f;
    float m_run[2] = {kNegBig, kNegBig}, l_run[2] = {0.f, 0.f};

    // ---- cooperative tile loader: thread -> (key, 16-byte chunk) ------------
    const int32_t *bt_row = p.bt + (int64_t)b * p.bt_stride;
    const int64_t tok_stride = (int64_t)p.hkv * D * 2;
    uint4 kst[LD], vst[LD];
    auto fetch = [&](int tile) {
#pragma unroll
        for (int i = 0; i < LD; ++i) {
            const int idx = tid + 256 * i;
            const int kk = idx / CPR, c = idx - kk * CPR;
            const int key = tile * kPfKeys + kk;
            kst[i] = vst[i] = uint4{0, 0, 0, 0};
            if (key < ctx_len) {
                const int blk = key / p.bs;
                const int64_t bid = blk < p.bt_stride ? (int64_t)bt_row[blk] : -1;
                if (bid >= 0 && bid < p.num_blocks) {
                    const int64_t off = (bid * p.bs + (key - blk * p.bs)) * tok_stride + (int64_t)kvh * D * 2 + c * 16;
                    kst[i] = ld16(reinterpret_cast<const char *>(p.k) + off);
                    vst[i] = ld16(reinterpret_cast<const char *>(p.v) + off);
                }
            }
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int i = 0; i < LD; ++i) {
            const int idx = tid + 256 * i;
            const int kk = idx / CPR, c = idx - kk * CPR;
            *reinterpret_cast<uint4 *>(s_k + kk * L::kRowBytesK + c * 16) = kst[i];
            *reinterpret_cast<uint4 *>(s_v + kk * L::kRowBytesV + c * 16) = vst[i];
        }
    };

    // per-lane byte offsets of the operand reads inside a tile
    const int k_rd = col * L::kRowBytesK + half * 16;  // + 32-key subtile, + 32*ks
    // V^T transpose read: 16-lane group g = lane/16 covers d = 16*(g%2).., keys 4*(g/2)..; source lane s of the
    // group reads the 8 bytes at key +s/4, d +4*(s%4)
    const int g16 = lane >> 4, s16 = lane & 15;
    const int v_rd = (4 * (g16 >> 1) + (s16 >> 2)) * L::kRowBytesV + (16 * (g16 & 1) + 4 * (s16 & 3)) * 2;

    fetch(0);
    for (int tile = 0; tile < n_tiles; ++tile) {
        __syncthreads();  // everyone is done reading the previous tile
        stash();
        __syncthreads();
        if (tile + 1 < n_tiles) fetch(tile + 1);  // in flight during the products below
        const int key0 = tile * kPfKeys;
        if (key0 >= my_keys) continue;  // this wave's rows end before this tile (uniform per wave)
        // masking is needed only where the tile reaches past the first row's causal limit or the context end
        const bool need_mask = key0 + kPfKeys > prefix + row0 + 1 || key0 + kPfKeys > ctx_len;

#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            // ---- S^T = K . Q^T for 32 keys x 64 rows ---------------------
            f32x16 s[2];
#pragma unroll
            for (int nt = 0; nt < 2; ++nt)
#pragma unroll
                for (int i = 0; i < 16; ++i) s[nt][i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const uint4 raw = *reinterpret_cast<const uint4 *>(s_k + kt * 32 * L::kRowBytesK + k_rd + ks * 32);
                const X8 ka = __builtin_bit_cast(X8, raw);
                s[0] = M::mma(ka, qreg[0][ks], s[0]);
                s[1] = M::mma(ka, qreg[1][ks], s[1]);
            }
            // ---- online softmax per row (= per lane), P^T packed in place ----
            uint32_t pp[2][8];
#pragma unroll
            for (int nt = 0; nt < 2; ++nt) {
                float v[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) v[i] = s[nt][i] * p.scale_log2;
                if (need_mask) {
                    const int limit = min(ctx_len - 1, prefix + row0 + 32 * nt + col);  // last visible key
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int key = key0 + 32 * kt + 4 * half + 8 * (i >> 2) + (i & 3);
                        v[i] = key <= limit ? v[i] : -INFINITY;
                    }
                }
                float mx = v[0];
#pragma unroll
                for (int i = 1; i < 16; ++i) mx = fmaxf(mx, v[i]);
                mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                const float m_new = fmaxf(m_run[nt], mx);
                if (__builtin_amdgcn_ballot_w64(m_new > m_run[nt]) != 0) {
                    const float alpha = __builtin_amdgcn_exp2f(m_run[nt] - m_new);
                    l_run[nt] *= alpha;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int i = 0; i < 16; ++i) o[nt][dt][i] *= alpha;
                    m_run[nt] = m_new;
                }
                float sum = 0.f;
#pragma unroll
                for (int i = 0; i < 16; i += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(v[i] - m_run[nt]);
                    const float p1 = __builtin_amdgcn_exp2f(v[i + 1] - m_run[nt]);
                    sum += p0 + p1;
                    pp[nt][i >> 1] = M::pack(p0, p1);
                }
                l_run[nt] += sum;
            }
            // ---- O^T += V^T . P^T: k-step ks2 uses result rows 8*ks2..8*ks2+7 of the lane, i.e. keys
            //      32*kt + 8*(2*ks2 + e/4) + 4*half + e%4 for operand element e ----
#pragma unroll
            for (int ks2 = 0; ks2 < 2; ++ks2) {
                X8 pb[2];
#pragma unroll
                for (int nt = 0; nt < 2; ++nt) {
                    const uint4 raw = uint4{pp[nt][4 * ks2], pp[nt][4 * ks2 + 1], pp[nt][4 * ks2 + 2], pp[nt][4 * ks2 + 3]};
                    pb[nt] = __builtin_bit_cast(X8, raw);
                }
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const char *vp = s_v + (32 * kt + 16 * ks2) * L::kRowBytesV + v_rd + dt * 64;
                    const X4 lo = M::tr_read(vp);                        // keys +0..3 (+4 for the upper half-wave)
                    const X4 hi = M::tr_read(vp + 8 * L::kRowBytesV);   // keys +8..11
                    X8 va;
#pragma unroll
                    for (int e = 0; e < 4; ++e) { va[e] = lo[e]; va[4 + e] = hi[e]; }
                    o[0][dt] = M::mma(va, pb[0], o[0][dt]);
                    o[1][dt] = M::mma(va, pb[1], o[1][dt]);
                }
            }
        }
    }

    // ---- normalise and write: lane owns row (row0+32*nt+col), d = 32*dt + 4*half + 8*g + j ----
    if (!live) return;
    T *obase = reinterpret_cast<T *>(a.out) + ((int64_t)a.q_starts[b] * p.hq + qh) * D;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
        const float l_tot = l_run[nt] + __shfl_xor(l_run[nt], 32, 64);
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        const int row = row0 + 32 * nt + col;
        if (row >= q_len) continue;
        T *orow = obase + (int64_t)row * p.hq * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                uint2 w;
                w.x = M::pack(o[nt][dt][4 * g] * inv, o[nt][dt][4 * g + 1] * inv);
                w.y = M::pack(o[nt][dt][4 * g + 2] * inv, o[nt][dt][4 * g + 3] * inv);
                *reinterpret_cast<uint2 *>(orow + 32 * dt + 4 * half + 8 * g) = w;
            }
    }
}

typedef void (*prefill_mfma_fn)(const RowwiseArgs);
prefill_mfma_fn pa_prefill_mfma_kernel(int dtype, int d);  // nullptr if the shape has no matrix-core kernel

}  // namespace pa_decode_detail
