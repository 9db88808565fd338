// fp8-e4m3 pool construction: one workgroup per (block, kv head) finds the
// absolute maximum of the block_size x head_dim tile, stores scale = max/448
// and writes the tile as OCP e4m3fn bytes of x/scale (round to nearest even).
#include "pa_common.h"

namespace {

constexpr int kQThreads = 256;

template <typename T>
__global__ __launch_bounds__(kQThreads) void quantize_e4m3_kernel(const T *__restrict__ src,
                                                                   uint8_t *__restrict__ dst,
                                                                   float *__restrict__ scale, int block_size,
                                                                   int hkv, int d) {
    __shared__ float s_max[kQThreads / PA_WAVE];
    const int64_t blk = blockIdx.x / hkv;
    const int h = blockIdx.x - (int)(blk * hkv);
    const int n = block_size * d;  // elements of the tile
    const int64_t tile0 = (blk * block_size * hkv + h) * (int64_t)d;
    const int64_t tok_stride = (int64_t)hkv * d;

    float amax = 0.f;
    for (int i = threadIdx.x; i < n; i += kQThreads) {
        const int t = i / d, e = i - t * d;
        amax = fmaxf(amax, fabsf(pa_scalar<T>::load(src + tile0 + t * tok_stride + e)));
    }
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
    const float sc = amax > 0.f ? amax / 448.0f : 1.0f;
    if (threadIdx.x == 0) scale[blk * hkv + h] = sc;

    for (int i = threadIdx.x; i < n; i += kQThreads) {
        const int t = i / d, e = i - t * d;
        const float x = pa_scalar<T>::load(src + tile0 + t * tok_stride + e) / sc;
        // gfx950 encodes OCP e4m3fn here; the low byte of the packed pair is x
        const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(x, 0.f, 0, false);
        dst[tile0 + t * tok_stride + e] = (uint8_t)(packed & 0xff);
    }
}

// Append to an fp8 pool ("re-round on growth"): one workgroup per (touched block, kv head) tile.
//   rows of the tile below the lowest offset this call writes are the tile's content so far; rows from there
//   on are new or not yet written (a recycled block starts over when its offset 0 is written);
//   a_old = scale * max|byte value| over the content, a_new = max|x| over the rows this call writes;
//   a_new <= a_old: the scale stays and only the new rows are encoded;
//   otherwise scale' = a_new / 448 and the content is re-rounded: byte' = e4m3(float(byte) * (scale / scale')).
constexpr int kMaxBlockTokens = 256;

// Rotary tables of a fused append: the rows are rotated as they are read, x' = (x*cos) + (rotate_half(x)*sin)
// with every product and the sum rounded to the rows' type T (the rounding of that statement evaluated in T).
struct RopeTables {
    const void *cos, *sin;     // [rope_rows][d] of T
    const int32_t *positions;  // row per token, or NULL: the token's own index
    int64_t rope_rows;
};

template <typename T> __device__ __forceinline__ float round_to(float x) {
    T t;
    pa_scalar<T>::store(&t, x);
    return pa_scalar<T>::load(&t);
}

template <typename T, bool ROPE>
__device__ __forceinline__ float load_src_elem(const T *src, const RopeTables &rt, int tok, int hkv, int h, int d, int e) {
#pragma clang fp contract(off)
    const T *row = src + ((int64_t)tok * hkv + h) * d;
    const float x = pa_scalar<T>::load(row + e);
    if (!ROPE) return x;
    int64_t r = rt.positions ? (int64_t)rt.positions[tok] : tok;
    r = r < 0 ? 0 : (r >= rt.rope_rows ? rt.rope_rows - 1 : r);
    const int half = d / 2;
    const float other = e < half ? -pa_scalar<T>::load(row + e + half) : pa_scalar<T>::load(row + e - half);
    const float c = pa_scalar<T>::load((const T *)rt.cos + r * d + e);
    const float sn = pa_scalar<T>::load((const T *)rt.sin + r * d + e);
    const float a = round_to<T>(x * c);
    const float b = round_to<T>(other * sn);
    return round_to<T>(a + b);
}

// ---- eight elements at a time (head_dim a multiple of 8, 16 with the rotation) ----
template <typename T> __device__ __forceinline__ float round_hw(float x);  // one rounding to T, hardware conversions
template <> __device__ __forceinline__ float round_hw<float>(float x) { return x; }
template <> __device__ __forceinline__ float round_hw<pa_bf16>(float x) { return (float)(__bf16)x; }
template <> __device__ __forceinline__ float round_hw<pa_f16>(float x) { return (float)(_Float16)x; }

template <typename T> __device__ __forceinline__ void load8(const T *p, float (&f)[8]) {
    if constexpr (sizeof(T) == 4) {
        const uint4 a = reinterpret_cast<const uint4 *>(p)[0], b = reinterpret_cast<const uint4 *>(p)[1];
        pa_vec16<float>::unpack(a, f);
        pa_vec16<float>::unpack(b, f + 4);
    } else {
        pa_vec16<T>::unpack(*reinterpret_cast<const uint4 *>(p), f);
    }
}

__device__ __forceinline__ void load8_fp8(const uint8_t *p, float (&f)[8]) {
    const uint2 raw = *reinterpret_cast<const uint2 *>(p);
    const uint32_t w[2] = {raw.x, raw.y};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], false);
        const auto hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], true);
        f[4 * i] = lo[0]; f[4 * i + 1] = lo[1]; f[4 * i + 2] = hi[0]; f[4 * i + 3] = hi[1];
    }
}

__device__ __forceinline__ void store8_fp8(uint8_t *p, const float (&f)[8]) {
    uint32_t w[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        int packed = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * i], f[4 * i + 1], 0, false);
        packed = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * i + 2], f[4 * i + 3], packed, true);
        w[i] = (uint32_t)packed;
    }
    *reinterpret_cast<uint2 *>(p) = make_uint2(w[0], w[1]);
}

// elements e .. e+7 of head h of token tok, rotated when ROPE (same arithmetic and rounding as load_src_elem)
template <typename T, bool ROPE>
__device__ __forceinline__ void load_src8(const T *src, const RopeTables &rt, int tok, int hkv, int h, int d, int e,
                                          float (&x)[8]) {
#pragma clang fp contract(off)
    const T *row = src + ((int64_t)tok * hkv + h) * d;
    load8<T>(row + e, x);
    if (!ROPE) return;
    int64_t r = rt.positions ? (int64_t)rt.positions[tok] : tok;
    r = r < 0 ? 0 : (r >= rt.rope_rows ? rt.rope_rows - 1 : r);
    const int half = d / 2;
    float other[8], c[8], sn[8];
    load8<T>(row + (e < half ? e + half : e - half), other);
    load8<T>((const T *)rt.cos + r * d + e, c);
    load8<T>((const T *)rt.sin + r * d + e, sn);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float a = round_hw<T>(x[k] * c[k]);
        const float b = round_hw<T>(other[k] * sn[k]);
        x[k] = round_hw<T>(e < half ? a - b : a + b);  // rotate_half negates the second half's partner
    }
}

// Optional index of a call's rows by touched block: rows order[start[i]] .. order[start[i+1]-1] are the tokens
// whose slots fall in touched block i.  Without it (order == nullptr) every workgroup scans the whole slot list.
struct RowIndex {
    const int32_t *order, *start;
};

// s_token[offset] = the token of this call that writes that offset of the block (the highest index wins)
__device__ __forceinline__ void find_rows(int *s_token, const int64_t *__restrict__ slots, int64_t n_tokens,
                                          int64_t slot0, int block_size, const RowIndex rows, int touched_idx) {
    if (rows.order) {
        const int64_t lo = max(0, rows.start[touched_idx]);
        const int64_t hi = min(n_tokens, (int64_t)rows.start[touched_idx + 1]);
        for (int64_t i = lo + threadIdx.x; i < hi; i += kQThreads) {
            const int64_t t = rows.order[i];
            if (t < 0 || t >= n_tokens) continue;  // (a bad index entry names no row)
            const int64_t off = slots[t] - slot0;
            if (off >= 0 && off < block_size) atomicMax(&s_token[off], (int)t);
        }
        return;
    }
    for (int64_t t0 = threadIdx.x; t0 < n_tokens; t0 += 8 * kQThreads) {  // eight loads in flight per thread
        int64_t off[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int64_t t = t0 + (int64_t)k * kQThreads;
            off[k] = t < n_tokens ? slots[t] - slot0 : -1;
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
            if (off[k] >= 0 && off[k] < block_size) atomicMax(&s_token[off[k]], (int)(t0 + (int64_t)k * kQThreads));
    }
}

template <typename T, bool ROPE, bool VEC>
__global__ __launch_bounds__(kQThreads) void append_e4m3_kernel(const T *__restrict__ src, uint8_t *__restrict__ dst,
                                                                 float *__restrict__ scale,
                                                                 const int64_t *__restrict__ slots, int64_t n_tokens,
                                                                 const int32_t *__restrict__ touched, const RowIndex rows,
                                                                 int64_t num_blocks, int block_size, int hkv, int d,
                                                                 const RopeTables rt) {
    __shared__ int s_token[kMaxBlockTokens];  // token of this call that writes offset i (-1: none); highest index wins
    __shared__ float s_max[2][kQThreads / PA_WAVE];
    const int64_t blk = touched[blockIdx.x];
    const int h = blockIdx.y;
    if (blk < 0 || blk >= num_blocks) return;  // uniform
    for (int i = threadIdx.x; i < block_size; i += kQThreads) s_token[i] = -1;
    __syncthreads();
    const int64_t slot0 = blk * block_size;
    find_rows(s_token, slots, n_tokens, slot0, block_size, rows, blockIdx.x);
    __syncthreads();
    int first = block_size;  // lowest offset written
    for (int i = 0; i < block_size; ++i)
        if (s_token[i] >= 0) { first = i; break; }
    if (first == block_size) return;  // uniform: the block is not touched after all

    const int64_t tok_stride = (int64_t)hkv * d;
    const int64_t tile0 = (slot0 * hkv + h) * (int64_t)d;
    const float s_old = scale[blk * hkv + h];
    // content so far: rows [0, first)
    float q_max = 0.f, a_new = 0.f;
    const int vpr = d / 8;  // vectors of eight elements per row (VEC)
    if (VEC) {
        for (int i = threadIdx.x; i < first * vpr; i += kQThreads) {
            const int t = i / vpr, e = (i - t * vpr) * 8;
            float f[8];
            load8_fp8(dst + tile0 + t * tok_stride + e, f);
#pragma unroll
            for (int k = 0; k < 8; ++k) q_max = fmaxf(q_max, fabsf(f[k]));
        }
        for (int i = threadIdx.x; i < (block_size - first) * vpr; i += kQThreads) {
            const int t = first + i / vpr, e = (i % vpr) * 8;
            const int tok = s_token[t];
            if (tok < 0) continue;
            float x[8];
            load_src8<T, ROPE>(src, rt, tok, hkv, h, d, e, x);
#pragma unroll
            for (int k = 0; k < 8; ++k) a_new = fmaxf(a_new, fabsf(x[k]));
        }
    } else {
        for (int i = threadIdx.x; i < first * d; i += kQThreads) {
            const int t = i / d, e = i - t * d;
            q_max = fmaxf(q_max, fabsf(__builtin_amdgcn_cvt_f32_fp8((int)dst[tile0 + t * tok_stride + e], 0)));
        }
        for (int i = threadIdx.x; i < (block_size - first) * d; i += kQThreads) {
            const int t = first + i / d, e = i % d;
            const int tok = s_token[t];
            if (tok >= 0) a_new = fmaxf(a_new, fabsf(load_src_elem<T, ROPE>(src, rt, tok, hkv, h, d, e)));
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        q_max = fmaxf(q_max, __shfl_xor(q_max, off, 64));
        a_new = fmaxf(a_new, __shfl_xor(a_new, off, 64));
    }
    if ((threadIdx.x & 63) == 0) { s_max[0][threadIdx.x >> 6] = q_max; s_max[1][threadIdx.x >> 6] = a_new; }
    __syncthreads();
    q_max = fmaxf(fmaxf(s_max[0][0], s_max[0][1]), fmaxf(s_max[0][2], s_max[0][3]));
    a_new = fmaxf(fmaxf(s_max[1][0], s_max[1][1]), fmaxf(s_max[1][2], s_max[1][3]));
    const float a_old = first > 0 ? s_old * q_max : 0.f;
    float s_new = s_old;
    if (first == 0 || a_new > a_old) s_new = a_new > 0.f ? a_new / 448.0f : 1.0f;
    if (first > 0 && s_new != s_old) {  // uniform: re-round the content to the new scale
        const float ratio = s_old / s_new;
        if (VEC) {
            for (int i = threadIdx.x; i < first * vpr; i += kQThreads) {
                const int t = i / vpr, e = (i - t * vpr) * 8;
                float f[8];
                load8_fp8(dst + tile0 + t * tok_stride + e, f);
#pragma unroll
                for (int k = 0; k < 8; ++k) f[k] *= ratio;
                store8_fp8(dst + tile0 + t * tok_stride + e, f);
            }
        } else {
            for (int i = threadIdx.x; i < first * d; i += kQThreads) {
                const int t = i / d, e = i - t * d;
                const float x = __builtin_amdgcn_cvt_f32_fp8((int)dst[tile0 + t * tok_stride + e], 0) * ratio;
                dst[tile0 + t * tok_stride + e] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(x, 0.f, 0, false) & 0xff);
            }
        }
    }
    if (VEC) {
        for (int i = threadIdx.x; i < (block_size - first) * vpr; i += kQThreads) {
            const int t = first + i / vpr, e = (i % vpr) * 8;
            const int tok = s_token[t];
            if (tok < 0) continue;
            float x[8];
            load_src8<T, ROPE>(src, rt, tok, hkv, h, d, e, x);
#pragma unroll
            for (int k = 0; k < 8; ++k) x[k] = x[k] / s_new;
            store8_fp8(dst + tile0 + t * tok_stride + e, x);
        }
    } else {
        for (int i = threadIdx.x; i < (block_size - first) * d; i += kQThreads) {
            const int t = first + i / d, e = i % d;
            const int tok = s_token[t];
            if (tok < 0) continue;
            const float x = load_src_elem<T, ROPE>(src, rt, tok, hkv, h, d, e) / s_new;
            dst[tile0 + t * tok_stride + e] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(x, 0.f, 0, false) & 0xff);
        }
    }
    if (threadIdx.x == 0) scale[blk * hkv + h] = s_new;
}

template <typename T> __device__ __forceinline__ uint32_t pack_pair(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack_pair<pa_bf16>(float lo, float hi) {
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    const v2 r = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, r);
}
template <> __device__ __forceinline__ uint32_t pack_pair<pa_f16>(float lo, float hi) {
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    const v2 r = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, r);
}

// Dequantise listed blocks of an fp8 pool into a compact 16-bit pool: block j of dst = block ids[j] of src times
// its scales.  One workgroup per (listed block, kv head) tile; a lane widens 16 bytes to 16 values (two 16-byte
// stores).  Ids outside the pool give zero blocks.
template <typename T>
__global__ __launch_bounds__(kQThreads) void dequantize_blocks_kernel(const uint8_t *__restrict__ src,
                                                                       const float *__restrict__ scale,
                                                                       const int32_t *__restrict__ ids,
                                                                       T *__restrict__ dst, int64_t num_blocks,
                                                                       int block_size, int hkv, int d) {
    const int j = blockIdx.x, h = blockIdx.y;
    const int64_t bid = ids[j];
    const bool ok = bid >= 0 && bid < num_blocks;
    const float sc = ok ? scale[bid * hkv + h] : 0.f;
    const int vecs_per_row = d / 16;
    const int64_t tok_stride = (int64_t)hkv * d;
    for (int i = threadIdx.x; i < block_size * vecs_per_row; i += kQThreads) {
        const int t = i / vecs_per_row, e = (i - t * vecs_per_row) * 16;
        float f[16];
        if (ok) {
            const uint4 raw = *reinterpret_cast<const uint4 *>(src + ((bid * block_size + t) * hkv + h) * (int64_t)d + e);
            pa_vec16<pa_fp8>::unpack(raw, f);
        } else {
#pragma unroll
            for (int k = 0; k < 16; ++k) f[k] = 0.f;
        }
        T *out = dst + (((int64_t)j * block_size + t) * tok_stride + (int64_t)h * d + e);
        uint32_t w[8];  // 16 values of T, rounded to nearest even by the hardware conversions
#pragma unroll
        for (int k = 0; k < 8; ++k) w[k] = pack_pair<T>(f[2 * k] * sc, f[2 * k + 1] * sc);
        reinterpret_cast<uint4 *>(out)[0] = make_uint4(w[0], w[1], w[2], w[3]);
        reinterpret_cast<uint4 *>(out)[1] = make_uint4(w[4], w[5], w[6], w[7]);
    }
}

// The same append, one workgroup per touched block for all its kv heads: the slot list is scanned once per
// block instead of once per (block, head), 32 lanes own a head's tile (eight elements per lane and step) and
// reduce its maxima among themselves, so there is no barrier after the scan.  Rows must allow 16-byte loads
// and 8-byte stores (head_dim a multiple of 8, 16 with the rotation).
template <typename T, bool ROPE>
__global__ __launch_bounds__(kQThreads) void append_e4m3_block_kernel(const T *__restrict__ src, uint8_t *__restrict__ dst,
                                                                       float *__restrict__ scale,
                                                                       const int64_t *__restrict__ slots, int64_t n_tokens,
                                                                       const int32_t *__restrict__ touched, const RowIndex rows,
                                                                       int64_t num_blocks, int block_size, int hkv, int d,
                                                                       const RopeTables rt) {
    __shared__ int s_token[kMaxBlockTokens];
    const int64_t blk = touched[blockIdx.x];
    if (blk < 0 || blk >= num_blocks) return;  // uniform
    for (int i = threadIdx.x; i < block_size; i += kQThreads) s_token[i] = -1;
    __syncthreads();
    const int64_t slot0 = blk * block_size;
    find_rows(s_token, slots, n_tokens, slot0, block_size, rows, blockIdx.x);
    __syncthreads();
    int first = block_size;  // lowest offset written
    for (int i = 0; i < block_size; ++i)
        if (s_token[i] >= 0) { first = i; break; }
    if (first == block_size) return;  // uniform: the block is not touched after all

    constexpr int kHeadLanes = 32, kHeadsPerPass = kQThreads / kHeadLanes;
    const int sub = threadIdx.x & (kHeadLanes - 1);
    const int64_t tok_stride = (int64_t)hkv * d;
    const int vpr = d / 8;
    for (int h0 = 0; h0 < hkv; h0 += kHeadsPerPass) {
        const int h = h0 + threadIdx.x / kHeadLanes;
        if (h >= hkv) continue;  // whole groups of 32 lanes
        const int64_t tile0 = (slot0 * hkv + h) * (int64_t)d;
        const float s_old = scale[blk * hkv + h];
        float q_max = 0.f, a_new = 0.f;
        for (int i = sub; i < first * vpr; i += kHeadLanes) {
            const int t = i / vpr, e = (i - t * vpr) * 8;
            float f[8];
            load8_fp8(dst + tile0 + t * tok_stride + e, f);
#pragma unroll
            for (int k = 0; k < 8; ++k) q_max = fmaxf(q_max, fabsf(f[k]));
        }
        // The first kKeep vectors of a lane stay in registers for the encoding pass (a 16 x 128 tile is exactly
        // 8 per lane): their loads are issued together and the rows are read (and rotated) once.
        constexpr int kKeep = 8;
        const int n_new = (block_size - first) * vpr;
        float keep[kKeep][8];
        bool live[kKeep];
#pragma unroll
        for (int it = 0; it < kKeep; ++it) {
            const int i = sub + it * kHeadLanes;
            const int t = first + i / vpr, e = (i % vpr) * 8;
            const int tok = i < n_new ? s_token[t] : -1;
            live[it] = tok >= 0;
            if (live[it]) load_src8<T, ROPE>(src, rt, tok, hkv, h, d, e, keep[it]);
        }
#pragma unroll
        for (int it = 0; it < kKeep; ++it)
            if (live[it])
#pragma unroll
                for (int k = 0; k < 8; ++k) a_new = fmaxf(a_new, fabsf(keep[it][k]));
        for (int i = sub + kKeep * kHeadLanes; i < n_new; i += kHeadLanes) {
            const int t = first + i / vpr, e = (i % vpr) * 8;
            const int tok = s_token[t];
            if (tok < 0) continue;
            float x[8];
            load_src8<T, ROPE>(src, rt, tok, hkv, h, d, e, x);
#pragma unroll
            for (int k = 0; k < 8; ++k) a_new = fmaxf(a_new, fabsf(x[k]));
        }
        for (int off = kHeadLanes / 2; off > 0; off >>= 1) {  // among the 32 lanes of the head
            q_max = fmaxf(q_max, __shfl_xor(q_max, off, 64));
            a_new = fmaxf(a_new, __shfl_xor(a_new, off, 64));
        }
        const float a_old = first > 0 ? s_old * q_max : 0.f;
        float s_new = s_old;
        if (first == 0 || a_new > a_old) s_new = a_new > 0.f ? a_new / 448.0f : 1.0f;
        if (first > 0 && s_new != s_old) {  // re-round the content to the new scale
            const float ratio = s_old / s_new;
            for (int i = sub; i < first * vpr; i += kHeadLanes) {
                const int t = i / vpr, e = (i - t * vpr) * 8;
                float f[8];
                load8_fp8(dst + tile0 + t * tok_stride + e, f);
#pragma unroll
                for (int k = 0; k < 8; ++k) f[k] *= ratio;
                store8_fp8(dst + tile0 + t * tok_stride + e, f);
            }
        }
#pragma unroll
        for (int it = 0; it < kKeep; ++it) {
            if (!live[it]) continue;
            const int i = sub + it * kHeadLanes;
            const int t = first + i / vpr, e = (i % vpr) * 8;
#pragma unroll
            for (int k = 0; k < 8; ++k) keep[it][k] = keep[it][k] / s_new;
            store8_fp8(dst + tile0 + t * tok_stride + e, keep[it]);
        }
        for (int i = sub + kKeep * kHeadLanes; i < n_new; i += kHeadLanes) {
            const int t = first + i / vpr, e = (i % vpr) * 8;
            const int tok = s_token[t];
            if (tok < 0) continue;
            float x[8];
            load_src8<T, ROPE>(src, rt, tok, hkv, h, d, e, x);
#pragma unroll
            for (int k = 0; k < 8; ++k) x[k] = x[k] / s_new;
            store8_fp8(dst + tile0 + t * tok_stride + e, x);
        }
        if (sub == 0) scale[blk * hkv + h] = s_new;
    }
}

template <bool ROPE, bool VEC>
void launch_append_v(const void *src, uint8_t *dst, float *sc, const int64_t *slots, int64_t n_tokens,
                     const int32_t *touched, int n_touched, const RowIndex rows, int64_t num_blocks, int block_size, int hkv, int d,
                     int src_dtype, const RopeTables &rt, hipStream_t s) {
    const dim3 block(kQThreads);
    if constexpr (VEC) {
        const dim3 grid((unsigned)n_touched);
        if (src_dtype == PA_F32)
            append_e4m3_block_kernel<float, ROPE><<<grid, block, 0, s>>>((const float *)src, dst, sc, slots, n_tokens,
                                                                         touched, rows, num_blocks, block_size, hkv, d, rt);
        else if (src_dtype == PA_BF16)
            append_e4m3_block_kernel<pa_bf16, ROPE><<<grid, block, 0, s>>>((const pa_bf16 *)src, dst, sc, slots, n_tokens,
                                                                           touched, rows, num_blocks, block_size, hkv, d, rt);
        else
            append_e4m3_block_kernel<pa_f16, ROPE><<<grid, block, 0, s>>>((const pa_f16 *)src, dst, sc, slots, n_tokens,
                                                                          touched, rows, num_blocks, block_size, hkv, d, rt);
    } else {
        const dim3 grid((unsigned)n_touched, (unsigned)hkv);
        if (src_dtype == PA_F32)
            append_e4m3_kernel<float, ROPE, false><<<grid, block, 0, s>>>((const float *)src, dst, sc, slots, n_tokens,
                                                                          touched, rows, num_blocks, block_size, hkv, d, rt);
        else if (src_dtype == PA_BF16)
            append_e4m3_kernel<pa_bf16, ROPE, false><<<grid, block, 0, s>>>((const pa_bf16 *)src, dst, sc, slots, n_tokens,
                                                                            touched, rows, num_blocks, block_size, hkv, d, rt);
        else
            append_e4m3_kernel<pa_f16, ROPE, false><<<grid, block, 0, s>>>((const pa_f16 *)src, dst, sc, slots, n_tokens,
                                                                           touched, rows, num_blocks, block_size, hkv, d, rt);
    }
}

// Appends one of K / V; ROPE rotates the rows on the way (K of a fused rotary append).  Eight elements per
// thread and step when the rows allow 16-byte loads and 8-byte stores, one element otherwise.
template <bool ROPE>
void launch_append(const void *src, uint8_t *dst, float *sc, const int64_t *slots, int64_t n_tokens,
                   const int32_t *touched, int n_touched, const RowIndex rows, int64_t num_blocks, int block_size, int hkv, int d,
                   int src_dtype, const RopeTables &rt, hipStream_t s) {
    const bool vec = d % (ROPE ? 16 : 8) == 0 && pa_aligned16(src) && ((uintptr_t)dst & 7u) == 0 &&
                     (!ROPE || (pa_aligned16(rt.cos) && pa_aligned16(rt.sin)));
    if (vec)
        launch_append_v<ROPE, true>(src, dst, sc, slots, n_tokens, touched, n_touched, rows, num_blocks, block_size, hkv, d,
                                    src_dtype, rt, s);
    else
        launch_append_v<ROPE, false>(src, dst, sc, slots, n_tokens, touched, n_touched, rows, num_blocks, block_size, hkv, d,
                                     src_dtype, rt, s);
}

int check_append(int64_t n_tokens, int n_touched, int block_size, int num_kv_heads, int head_dim, int src_dtype) {
    PA_REQUIRE(n_tokens >= 0 && n_touched >= 0, "n_tokens=%lld / n_touched=%d is negative", (long long)n_tokens, n_touched);
    PA_REQUIRE(block_size > 0 && block_size <= kMaxBlockTokens, "block_size=%d outside 1..%d", block_size, kMaxBlockTokens);
    PA_REQUIRE(num_kv_heads > 0 && num_kv_heads <= 65535 && head_dim > 0, "num_kv_heads / head_dim out of range");
    PA_REQUIRE(src_dtype == PA_F32 || src_dtype == PA_BF16 || src_dtype == PA_F16, "src_dtype=%d is not F32, BF16 or F16",
               src_dtype);
    PA_REQUIRE(n_tokens <= 0x7fffffffll, "n_tokens above 2^31-1");
    return PA_OK;
}

}  // namespace

extern "C" int pa_kv_append_e4m3(void *k_cache, void *v_cache, float *k_scale, float *v_scale, const void *k_src,
                                 const void *v_src, const int64_t *slots, int64_t n_tokens,
                                 const int32_t *touched_blocks, int n_touched, const int32_t *row_order,
                                 const int32_t *block_start, int64_t num_blocks, int block_size, int num_kv_heads,
                                 int head_dim, int src_dtype, void *stream) {
    pa_clear_error();
    if (int rc = check_append(n_tokens, n_touched, block_size, num_kv_heads, head_dim, src_dtype)) return rc;
    if (n_tokens == 0 || n_touched == 0) return PA_OK;
    PA_REQUIRE(k_cache && v_cache && k_scale && v_scale && k_src && v_src && slots && touched_blocks, "NULL pointer argument");
    PA_REQUIRE((row_order == nullptr) == (block_start == nullptr), "row_order and block_start go together (both or neither)");
    const RowIndex rows{row_order, block_start};
    hipStream_t s = (hipStream_t)stream;
    const RopeTables none{};
    launch_append<false>(k_src, (uint8_t *)k_cache, k_scale, slots, n_tokens, touched_blocks, n_touched, rows, num_blocks,
                         block_size, num_kv_heads, head_dim, src_dtype, none, s);
    PA_CHECK_LAUNCH("pa_kv_append_e4m3");
    launch_append<false>(v_src, (uint8_t *)v_cache, v_scale, slots, n_tokens, touched_blocks, n_touched, rows, num_blocks,
                         block_size, num_kv_heads, head_dim, src_dtype, none, s);
    PA_CHECK_LAUNCH("pa_kv_append_e4m3");
    return PA_OK;
}

extern "C" int pa_rope_kv_append_e4m3(const void *q, void *q_out, const void *k_src, const void *v_src, void *k_cache,
                                      void *v_cache, float *k_scale, float *v_scale, const void *cos, const void *sin,
                                      const int32_t *positions, int64_t rope_rows, const int64_t *slots,
                                      int64_t n_tokens, const int32_t *touched_blocks, int n_touched,
                                      const int32_t *row_order, const int32_t *block_start, int64_t num_blocks,
                                      int block_size, int num_q_heads, int num_kv_heads, int head_dim, int src_dtype,
                                      void *stream) {
    pa_clear_error();
    if (int rc = check_append(n_tokens, n_touched, block_size, num_kv_heads, head_dim, src_dtype)) return rc;
    if (int rc = pa_rope_check("pa_rope_kv_append_e4m3", n_tokens, rope_rows, positions, num_q_heads, num_kv_heads,
                               head_dim, src_dtype))
        return rc;
    if (n_tokens == 0) return PA_OK;
    PA_REQUIRE(q && q_out && cos && sin, "NULL q / q_out / cos / sin");
    PA_REQUIRE(pa_aligned16(q) && pa_aligned16(q_out) && pa_aligned16(cos) && pa_aligned16(sin),
               "q, q_out, cos and sin must be 16-byte aligned");
    if (int rc = pa_rope_q_only(q, q_out, cos, sin, positions, rope_rows, n_tokens, num_q_heads, head_dim, src_dtype, stream))
        return rc;
    if (n_touched == 0) return PA_OK;
    PA_REQUIRE(k_cache && v_cache && k_scale && v_scale && k_src && v_src && slots && touched_blocks, "NULL pointer argument");
    PA_REQUIRE((row_order == nullptr) == (block_start == nullptr), "row_order and block_start go together (both or neither)");
    const RowIndex rows{row_order, block_start};
    hipStream_t s = (hipStream_t)stream;
    const RopeTables rt{cos, sin, positions, rope_rows};
    launch_append<true>(k_src, (uint8_t *)k_cache, k_scale, slots, n_tokens, touched_blocks, n_touched, rows, num_blocks,
                        block_size, num_kv_heads, head_dim, src_dtype, rt, s);
    PA_CHECK_LAUNCH("pa_rope_kv_append_e4m3");
    launch_append<false>(v_src, (uint8_t *)v_cache, v_scale, slots, n_tokens, touched_blocks, n_touched, rows, num_blocks,
                         block_size, num_kv_heads, head_dim, src_dtype, RopeTables{}, s);
    PA_CHECK_LAUNCH("pa_rope_kv_append_e4m3");
    return PA_OK;
}

extern "C" int pa_quantize_kv_e4m3(const void *src, void *dst, float *scale, int64_t num_blocks,
                                   int block_size, int num_kv_heads, int head_dim, int src_dtype,
                                   void *stream) {
    pa_clear_error();
    PA_REQUIRE(num_blocks >= 0, "num_blocks=%lld is negative", (long long)num_blocks);
    PA_REQUIRE(block_size > 0 && num_kv_heads > 0 && head_dim > 0, "block_size / num_kv_heads / head_dim must be positive");
    PA_REQUIRE(src_dtype == PA_F32 || src_dtype == PA_BF16 || src_dtype == PA_F16, "src_dtype=%d is not F32, BF16 or F16",
               src_dtype);
    PA_REQUIRE(num_blocks * num_kv_heads <= 0x7fffffffll, "num_blocks*num_kv_heads above 2^31-1");
    PA_REQUIRE((int64_t)block_size * head_dim <= (1 << 24), "tile of %d x %d elements is too large", block_size, head_dim);
    if (num_blocks == 0) return PA_OK;
    PA_REQUIRE(src && dst && scale, "NULL src / dst / scale");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)(num_blocks * num_kv_heads)), block(kQThreads);
    if (src_dtype == PA_F32)
        quantize_e4m3_kernel<float><<<grid, block, 0, s>>>((const float *)src, (uint8_t *)dst, scale, block_size,
                                                           num_kv_heads, head_dim);
    else if (src_dtype == PA_BF16)
        quantize_e4m3_kernel<pa_bf16><<<grid, block, 0, s>>>((const pa_bf16 *)src, (uint8_t *)dst, scale, block_size,
                                                             num_kv_heads, head_dim);
    else
        quantize_e4m3_kernel<pa_f16><<<grid, block, 0, s>>>((const pa_f16 *)src, (uint8_t *)dst, scale, block_size,
                                                            num_kv_heads, head_dim);
    PA_CHECK_LAUNCH("pa_quantize_kv_e4m3");
    return PA_OK;
}

extern "C" int pa_dequantize_blocks_e4m3(const void *cache, const float *scale, const int32_t *block_ids, int n_ids,
                                         void *dst, int64_t num_blocks, int block_size, int num_kv_heads, int head_dim,
                                         int dst_dtype, void *stream) {
    pa_clear_error();
    PA_REQUIRE(n_ids >= 0 && num_blocks >= 0, "n_ids=%d / num_blocks=%lld is negative", n_ids, (long long)num_blocks);
    PA_REQUIRE(block_size > 0 && num_kv_heads > 0 && num_kv_heads <= 65535 && head_dim > 0,
               "block_size / num_kv_heads / head_dim out of range");
    PA_REQUIRE(head_dim % 16 == 0, "head_dim=%d is not a multiple of 16", head_dim);
    PA_REQUIRE(dst_dtype == PA_BF16 || dst_dtype == PA_F16, "dst_dtype=%d is not BF16 or F16", dst_dtype);
    if (n_ids == 0) return PA_OK;
    PA_REQUIRE(cache && scale && block_ids && dst, "NULL pointer argument");
    PA_REQUIRE(pa_aligned16(cache) && pa_aligned16(dst), "cache and dst must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)n_ids, (unsigned)num_kv_heads), block(kQThreads);
    if (dst_dtype == PA_BF16)
        dequantize_blocks_kernel<pa_bf16><<<grid, block, 0, s>>>((const uint8_t *)cache, scale, block_ids, (pa_bf16 *)dst,
                                                                 num_blocks, block_size, num_kv_heads, head_dim);
    else
        dequantize_blocks_kernel<pa_f16><<<grid, block, 0, s>>>((const uint8_t *)cache, scale, block_ids, (pa_f16 *)dst,
                                                                num_blocks, block_size, num_kv_heads, head_dim);
    PA_CHECK_LAUNCH("pa_dequantize_blocks_e4m3");
    return PA_OK;
}
