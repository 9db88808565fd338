// Shared host/device helpers for libpaged_attn (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/paged_attn.h"

// ---------------------------------------------------------------- host side
// Records printf-style text as the calling thread's last error and returns
// `code`, so that entry points can `return pa_fail(PA_ERR_..., "...")`.
int pa_fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
void pa_clear_error();

#define PA_REQUIRE(cond, ...)                                  \
    do {                                                       \
        if (!(cond)) return pa_fail(PA_ERR_INVALID_ARG, __VA_ARGS__); \
    } while (0)

// Launch-error check: hipGetLastError after a kernel launch.
#define PA_CHECK_LAUNCH(what)                                                      \
    do {                                                                           \
        hipError_t e_ = hipGetLastError();                                         \
        if (e_ != hipSuccess)                                                      \
            return pa_fail(PA_ERR_HIP, "%s: %s", what, hipGetErrorString(e_));     \
    } while (0)

// Shared by the rotary entry points (rope.hip): argument checks, and the rotation of q alone (no K/V work).
int pa_rope_check(const char *what, int64_t n_tokens, int64_t rope_rows, const int32_t *positions, int num_q_heads,
                  int num_kv_heads, int head_dim, int dtype);
int pa_rope_q_only(const void *q, void *q_out, const void *cos, const void *sin, const int32_t *positions,
                   int64_t rope_rows, int64_t n_tokens, int num_q_heads, int head_dim, int dtype, void *stream);

static inline bool pa_aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// -------------------------------------------------------------- device side
#define PA_WAVE 64

struct pa_bf16 { uint16_t bits; };
struct pa_f16 { _Float16 v; };
struct pa_fp8 { uint8_t bits; };

__device__ __forceinline__ float pa_bf16_to_f32(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }

// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ uint16_t pa_f32_to_bf16(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <typename T> struct pa_scalar;  // load/store one element as float
template <> struct pa_scalar<float> {
    static __device__ __forceinline__ float load(const float *p) { return *p; }
    static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
};
template <> struct pa_scalar<pa_bf16> {
    static __device__ __forceinline__ float load(const pa_bf16 *p) { return pa_bf16_to_f32(p->bits); }
    static __device__ __forceinline__ void store(pa_bf16 *p, float v) { p->bits = pa_f32_to_bf16(v); }
};
template <> struct pa_scalar<pa_f16> {
    static __device__ __forceinline__ float load(const pa_f16 *p) { return (float)p->v; }
    static __device__ __forceinline__ void store(pa_f16 *p, float v) { p->v = (_Float16)v; }
};

// Unpack one 16-byte vector of pool elements into floats.
template <typename T> struct pa_vec16;
template <> struct pa_vec16<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ void unpack(const uint4 &r, float *f) {
        f[0] = __builtin_bit_cast(float, r.x); f[1] = __builtin_bit_cast(float, r.y);
        f[2] = __builtin_bit_cast(float, r.z); f[3] = __builtin_bit_cast(float, r.w);
    }
};
template <> struct pa_vec16<pa_bf16> {
    static constexpr int N = 8;
    static __device__ __forceinline__ void unpack(const uint4 &r, float *f) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __builtin_bit_cast(float, w[i] << 16);
            f[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
        }
    }
};
template <> struct pa_vec16<pa_f16> {
    static constexpr int N = 8;
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ void unpack(const uint4 &r, float *f) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            h2 h = __builtin_bit_cast(h2, w[i]);
            f[2 * i] = (float)h[0];
            f[2 * i + 1] = (float)h[1];
        }
    }
};
template <> struct pa_vec16<pa_fp8> {
    static constexpr int N = 16;
    static __device__ __forceinline__ void unpack(const uint4 &r, float *f) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // gfx950 decodes OCP e4m3fn here (gfx942 decoded the fnuz variant)
            auto lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], false);
            auto hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], true);
            f[4 * i] = lo[0]; f[4 * i + 1] = lo[1];
            f[4 * i + 2] = hi[0]; f[4 * i + 3] = hi[1];
        }
    }
};

// x + (x moved across lanes by a DPP pattern); the compiler folds the move
// into v_add_f32_dpp.
template <int CTRL> __device__ __forceinline__ float pa_dpp(float x) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}

// Sum over aligned groups of W consecutive lanes (W a power of two <= 64);
// every lane of the group receives the total.
template <int W> __device__ __forceinline__ float pa_group_sum(float x) {
    if (W >= 2) x += pa_dpp<0xB1>(x);   // quad_perm [1,0,3,2]
    if (W >= 4) x += pa_dpp<0x4E>(x);   // quad_perm [2,3,0,1]
    if (W >= 8) x += pa_dpp<0x141>(x);  // row_half_mirror
    if (W >= 16) x += pa_dpp<0x140>(x); // row_mirror
    if (W >= 32) x += __shfl_xor(x, 16, 64);
    if (W >= 64) x += __shfl_xor(x, 32, 64);
    return x;
}
