// Rotary position embedding fused with the KV append: one pass over a step's
// new Q/K/V rows rotates Q (to q_out) and K, writes the rotated K and the V row
// to their cache slots (and the rotated K to a dense buffer when asked).
// HBM-bound.  The arithmetic keeps the rounding of the elementwise statement
//     x_embed = (x * cos) + (rotate_half(x) * sin)
// evaluated in the tensors' own type: each product and the sum are rounded to
// that type, so results match that statement bit for bit.
#include "pa_common.h"

namespace {

constexpr int kRopeThreads = 256;

// One rounding step to the element type T, value kept as float.
template <typename T> __device__ __forceinline__ float rope_round(float x);
template <> __device__ __forceinline__ float rope_round<float>(float x) { return x; }
// (gfx950 rounds float -> bf16 to nearest even in hardware: v_cvt_pk_bf16_f32)
template <> __device__ __forceinline__ float rope_round<pa_bf16>(float x) { return (float)(__bf16)x; }
template <> __device__ __forceinline__ float rope_round<pa_f16>(float x) { return (float)(_Float16)x; }

template <typename T> __device__ __forceinline__ uint4 rope_pack(const float *f);
template <> __device__ __forceinline__ uint4 rope_pack<float>(const float *f) {
    return make_uint4(__builtin_bit_cast(uint32_t, f[0]), __builtin_bit_cast(uint32_t, f[1]),
                      __builtin_bit_cast(uint32_t, f[2]), __builtin_bit_cast(uint32_t, f[3]));
}
template <> __device__ __forceinline__ uint4 rope_pack<pa_bf16>(const float *f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
        const bf2 pair = {(__bf16)f[2 * i], (__bf16)f[2 * i + 1]};
        w[i] = __builtin_bit_cast(uint32_t, pair);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}
template <> __device__ __forceinline__ uint4 rope_pack<pa_f16>(const float *f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint16_t lo = __builtin_bit_cast(uint16_t, (_Float16)f[2 * i]);
        const uint16_t hi = __builtin_bit_cast(uint16_t, (_Float16)f[2 * i + 1]);
        w[i] = (uint32_t)lo | ((uint32_t)hi << 16);
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// (x1, x2) = the matching vectors of the first and the second half of one head; on return the rotated ones.
//   out1 = x1*cos1 + (-x2)*sin1,  out2 = x2*cos2 + x1*sin2   (rotate_half(x) = cat(-x2, x1))
template <typename T>
__device__ __forceinline__ void rope_rotate(uint4 &v1, uint4 &v2, const uint4 &c1, const uint4 &c2, const uint4 &s1,
                                            const uint4 &s2) {
#pragma clang fp contract(off)
    constexpr int N = pa_vec16<T>::N;
    float x1[N], x2[N], fc1[N], fc2[N], fs1[N], fs2[N], o1[N], o2[N];
    pa_vec16<T>::unpack(v1, x1);
    pa_vec16<T>::unpack(v2, x2);
    pa_vec16<T>::unpack(c1, fc1);
    pa_vec16<T>::unpack(c2, fc2);
    pa_vec16<T>::unpack(s1, fs1);
    pa_vec16<T>::unpack(s2, fs2);
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const float a1 = rope_round<T>(x1[i] * fc1[i]);
        const float b1 = rope_round<T>(x2[i] * fs1[i]);  // -(x2*sin) = (-x2)*sin exactly, rounding included
        o1[i] = a1 - b1;                                  // rounded by the pack
        const float a2 = rope_round<T>(x2[i] * fc2[i]);
        const float b2 = rope_round<T>(x1[i] * fs2[i]);
        o2[i] = a2 + b2;
    }
    v1 = rope_pack<T>(o1);
    v2 = rope_pack<T>(o2);
}

struct RopeArgs {
    const uint4 *q;
    uint4 *q_out;
    const uint4 *k_src, *v_src;
    uint4 *k_out;              // dense rotated K rows, or NULL
    uint4 *k_cache, *v_cache;  // or NULL with slots == NULL
    const uint4 *cos, *sin;
    const int32_t *positions;  // row of cos/sin per token, or NULL: the token's own index
    const int64_t *slots;
    int64_t n_tokens, total_slots, rope_rows;
    int hq, hkv;
    int half_vecs;  // 16-byte vectors in half a head
};

// One thread per (token, group of HG heads, vector of the first half) for the rotated heads: it loads its four
// cos/sin vectors once and rotates that vector (and its partner in the second half) of HG heads, so the table
// rows are fetched HG times less often than the data they multiply.  The heads of a group are hq/HG apart
// (group g holds heads g, g + hq/HG, ...), so that consecutive lanes touch consecutive heads in every load and
// store.  One thread per (token, vector) for V.
template <typename T, int HG> __global__ __launch_bounds__(kRopeThreads) void rope_kv_append_kernel(const RopeArgs a) {
    const int hv = a.half_vecs;
    const int qg = a.hq / HG, kg = a.hkv / HG;  // head groups (hq and hkv are multiples of HG)
    const int units = (qg + kg + 2 * a.hkv) * hv;  // per token: hv per head group, 2*hv per v head
    const int64_t gid = (int64_t)blockIdx.x * kRopeThreads + threadIdx.x;
    const int64_t tok = gid / units;
    if (tok >= a.n_tokens) return;
    const int u = (int)(gid - tok * units);
    const int64_t slot = a.slots ? a.slots[tok] : -1;
    const bool cached = slot >= 0 && slot < a.total_slots;
    const int rot_units = (qg + kg) * hv;
    if (u >= rot_units) {  // V: plain copy, one vector per thread (a V row holds 2*hkv*hv vectors)
        if (!cached) return;
        const int j = u - rot_units;
        const int64_t vrow = 2 * (int64_t)a.hkv * hv;
        a.v_cache[slot * vrow + j] = a.v_src[tok * vrow + j];
        return;
    }
    int64_t r = a.positions ? (int64_t)a.positions[tok] : tok;
    r = r < 0 ? 0 : (r >= a.rope_rows ? a.rope_rows - 1 : r);  // never read outside the tables
    const int group = u / hv, j = u - group * hv;
    const uint4 c1 = a.cos[r * 2 * hv + j], c2 = a.cos[r * 2 * hv + hv + j];
    const uint4 s1 = a.sin[r * 2 * hv + j], s2 = a.sin[r * 2 * hv + hv + j];
    if (group < qg) {
        uint4 v1[HG], v2[HG];
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            const int64_t at = (tok * a.hq + h * qg + group) * 2 * hv + j;
            v1[h] = a.q[at];
            v2[h] = a.q[at + hv];
        }
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            const int64_t at = (tok * a.hq + h * qg + group) * 2 * hv + j;
            rope_rotate<T>(v1[h], v2[h], c1, c2, s1, s2);
            a.q_out[at] = v1[h];
            a.q_out[at + hv] = v2[h];
        }
    } else {
        const int kgi = group - qg;  // this thread's kv heads: kgi, kgi + kg, kgi + 2 kg, ...
        uint4 v1[HG], v2[HG];
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            const int64_t at = (tok * a.hkv + h * kg + kgi) * 2 * hv + j;
            v1[h] = a.k_src[at];
            v2[h] = a.k_src[at + hv];
        }
#pragma unroll
        for (int h = 0; h < HG; ++h) {
            const int64_t at = (tok * a.hkv + h * kg + kgi) * 2 * hv + j;
            rope_rotate<T>(v1[h], v2[h], c1, c2, s1, s2);
            if (a.k_out) {
                a.k_out[at] = v1[h];
                a.k_out[at + hv] = v2[h];
            }
            if (cached) {
                const int64_t dst = (slot * a.hkv + h * kg + kgi) * 2 * hv + j;
                a.k_cache[dst] = v1[h];
                a.k_cache[dst + hv] = v2[h];
            }
        }
    }
}

template <typename T> void launch_rope_typed(const RopeArgs &a, int hg, int64_t grid, hipStream_t s) {
    if (hg == 4)
        rope_kv_append_kernel<T, 4><<<dim3((unsigned)grid), dim3(kRopeThreads), 0, s>>>(a);
    else if (hg == 2)
        rope_kv_append_kernel<T, 2><<<dim3((unsigned)grid), dim3(kRopeThreads), 0, s>>>(a);
    else
        rope_kv_append_kernel<T, 1><<<dim3((unsigned)grid), dim3(kRopeThreads), 0, s>>>(a);
}

int launch_rope(const RopeArgs &a, int dtype, hipStream_t s, const char *what) {
    // heads per thread: the largest of 4, 2, 1 that divides both head counts (hkv = 0: q only)
    int hg = 4;
    while (hg > 1 && (a.hq % hg != 0 || a.hkv % hg != 0)) hg >>= 1;
    const int64_t units = (int64_t)(a.hq / hg + a.hkv / hg + 2 * a.hkv) * a.half_vecs;
    PA_REQUIRE(units <= 0x7fffffff, "row of %lld vectors is too large", (long long)units);
    const int64_t grid = (a.n_tokens * units + kRopeThreads - 1) / kRopeThreads;
    PA_REQUIRE(grid <= 0x7fffffff, "n_tokens=%lld is too large for one launch", (long long)a.n_tokens);
    if (dtype == PA_F32)
        launch_rope_typed<float>(a, hg, grid, s);
    else if (dtype == PA_BF16)
        launch_rope_typed<pa_bf16>(a, hg, grid, s);
    else
        launch_rope_typed<pa_f16>(a, hg, grid, s);
    PA_CHECK_LAUNCH(what);
    return PA_OK;
}

}  // namespace

int pa_rope_check(const char *what, int64_t n_tokens, int64_t rope_rows, const int32_t *positions, int num_q_heads,
                  int num_kv_heads, int head_dim, int dtype) {
    PA_REQUIRE(n_tokens >= 0 && rope_rows >= 0, "n_tokens / rope_rows must be non-negative");
    PA_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && head_dim > 0, "head counts / head_dim must be positive");
    PA_REQUIRE(dtype == PA_F32 || dtype == PA_BF16 || dtype == PA_F16, "dtype=%d is not F32, BF16 or F16", dtype);
    if ((head_dim / 2 * pa_dtype_bytes(dtype)) % 16 != 0 || head_dim % 2 != 0)
        return pa_fail(PA_ERR_UNSUPPORTED, "%s: half a head of %d elements is not a multiple of 16 bytes", what,
                       head_dim / 2);
    if (n_tokens == 0) return PA_OK;
    PA_REQUIRE(rope_rows > 0, "empty cos / sin tables");
    PA_REQUIRE(positions || rope_rows >= n_tokens, "cos / sin hold %lld rows for %lld tokens and no positions",
               (long long)rope_rows, (long long)n_tokens);
    return PA_OK;
}

int pa_rope_q_only(const void *q, void *q_out, const void *cos, const void *sin, const int32_t *positions,
                   int64_t rope_rows, int64_t n_tokens, int num_q_heads, int head_dim, int dtype, void *stream) {
    RopeArgs a{};
    a.q = (const uint4 *)q; a.q_out = (uint4 *)q_out;
    a.cos = (const uint4 *)cos; a.sin = (const uint4 *)sin; a.positions = positions;
    a.n_tokens = n_tokens; a.rope_rows = rope_rows;
    a.hq = num_q_heads; a.hkv = 0;
    a.half_vecs = head_dim / 2 * pa_dtype_bytes(dtype) / 16;
    return launch_rope(a, dtype, (hipStream_t)stream, "rotary embedding of q");
}

extern "C" int pa_rope_kv_append(const void *q, void *q_out, const void *k_src, const void *v_src, void *k_out,
                                 void *k_cache, void *v_cache, const void *cos, const void *sin,
                                 const int32_t *positions, int64_t rope_rows, const int64_t *slots, int64_t n_tokens,
                                 int64_t total_slots, int num_q_heads, int num_kv_heads, int head_dim, int dtype,
                                 void *stream) {
    pa_clear_error();
    PA_REQUIRE(total_slots >= 0, "total_slots=%lld is negative", (long long)total_slots);
    if (int rc = pa_rope_check("pa_rope_kv_append", n_tokens, rope_rows, positions, num_q_heads, num_kv_heads, head_dim,
                               dtype))
        return rc;
    if (n_tokens == 0) return PA_OK;
    PA_REQUIRE(q && q_out && k_src && v_src && cos && sin, "NULL q / q_out / k_src / v_src / cos / sin");
    PA_REQUIRE(!slots || (k_cache && v_cache), "slots given without cache pointers");
    PA_REQUIRE(slots || k_out, "neither slots nor k_out: the rotated keys would go nowhere");
    PA_REQUIRE(pa_aligned16(q) && pa_aligned16(q_out) && pa_aligned16(k_src) && pa_aligned16(v_src) && pa_aligned16(cos) &&
                   pa_aligned16(sin) && pa_aligned16(k_out) && pa_aligned16(k_cache) && pa_aligned16(v_cache),
               "pointers must be 16-byte aligned");
    RopeArgs a{};
    a.q = (const uint4 *)q; a.q_out = (uint4 *)q_out; a.k_src = (const uint4 *)k_src; a.v_src = (const uint4 *)v_src;
    a.k_out = (uint4 *)k_out; a.k_cache = (uint4 *)k_cache; a.v_cache = (uint4 *)v_cache;
    a.cos = (const uint4 *)cos; a.sin = (const uint4 *)sin; a.positions = positions; a.slots = slots;
    a.n_tokens = n_tokens; a.total_slots = total_slots; a.rope_rows = rope_rows;
    a.hq = num_q_heads; a.hkv = num_kv_heads;
    a.half_vecs = head_dim / 2 * pa_dtype_bytes(dtype) / 16;
    return launch_rope(a, dtype, (hipStream_t)stream, "pa_rope_kv_append");
}
