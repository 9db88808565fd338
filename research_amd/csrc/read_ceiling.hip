// Stand-alone measurement of what the memory system delivers to a kernel that only reads, in the access
// pattern of the paged decode kernel: two pools (K and V) of 32 KiB pages in random order, 512 workgroups of
// 4 waves, 16 loads of 16 bytes in flight per wave.  Not part of the library; built by `make read_ceiling`.
//
//   pattern 0: a wave reads its pages contiguously (64 lanes x 16 B per instruction).
//   pattern 1: a wave reads one half (1 KiB) of every 2 KiB token row of its pages, K and V pages alternating;
//              the first half of the grid takes the first half of the rows (the decode kernel's two head groups).
//   kind    0: global loads; 1: buffer loads through a descriptor per page with the given cache-policy bits
//              (1 = sc0, 2 = nt, 16 = sc1).
//   work     : independent multiply-adds executed per 16-byte load.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <numeric>
#include <random>
#include <vector>

#define CK(x)                                                                         \
    do {                                                                              \
        hipError_t e_ = (x);                                                          \
        if (e_ != hipSuccess) {                                                       \
            std::printf("%s failed: %s (line %d)\n", #x, hipGetErrorString(e_), __LINE__); \
            return 1;                                                                 \
        }                                                                             \
    } while (0)

typedef unsigned int u4 __attribute__((ext_vector_type(4)));
constexpr int kPageVecs = 2048;  // 32 KiB page = 16 token rows of 128 vectors
constexpr int kInFlight = 16;

template <int PATTERN, int KIND, int POLICY, int WORK>
__global__ __launch_bounds__(256) void read_kernel(const u4 *__restrict__ pool_k, const u4 *__restrict__ pool_v,
                                                   const int *__restrict__ pages, int npages, float *out) {
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int halves = PATTERN == 1 ? 2 : 1;
    const int nwg = gridDim.x / halves;
    const int half = blockIdx.x / nwg, wg = blockIdx.x % nwg;
    auto consume = [&](const u4 &v) {
        const float x = __builtin_bit_cast(float, v.x), y = __builtin_bit_cast(float, v.y),
                    z = __builtin_bit_cast(float, v.z), w = __builtin_bit_cast(float, v.w);
        if (WORK == 0) { a0 += x; a1 += y; a2 += z; a3 += w; }
#pragma unroll
        for (int k = 0; k < WORK / 4; ++k) {
            a0 = __builtin_fmaf(a0, x, y); a1 = __builtin_fmaf(a1, y, z);
            a2 = __builtin_fmaf(a2, z, w); a3 = __builtin_fmaf(a3, w, x);
        }
    };
    // pattern 0 walks both pools as one list of 2*npages pages; pattern 1 reads page p of both pools together
    const int n_items = PATTERN == 0 ? 2 * npages : npages;
    for (int item = wg * 4 + wave; item < n_items; item += nwg * 4) {
        const int page = __builtin_amdgcn_readfirstlane(pages[item % npages]);
        const u4 *pk = (PATTERN == 0 && item >= npages ? pool_v : pool_k) + (size_t)page * kPageVecs;
        const u4 *pv = pool_v + (size_t)page * kPageVecs;
        u4 v[kInFlight];
        if (PATTERN == 0) {
            for (int j = 0; j < kPageVecs; j += 64 * kInFlight) {
#pragma unroll
                for (int i = 0; i < kInFlight; ++i) {
                    if (KIND == 0) {
                        v[i] = POLICY & 2 ? __builtin_nontemporal_load(pk + j + i * 64 + lane) : pk[j + i * 64 + lane];
                    } else {
                        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void *)pk, 0, 32768, 0x00020000);
                        v[i] = __builtin_amdgcn_raw_buffer_load_b128(r, (j + i * 64 + lane) * 16, 0, POLICY);
                    }
                }
#pragma unroll
                for (int i = 0; i < kInFlight; ++i) consume(v[i]);
            }
        } else {
            constexpr int H = kInFlight / 2;
            const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc((void *)pk, 0, 32768, 0x00020000);
            const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc((void *)pv, 0, 32768, 0x00020000);
            const int off = half * 64 + lane;  // vector inside a token row
            for (int t = 0; t < 16; t += H) {
#pragma unroll
                for (int i = 0; i < H; ++i) {
                    if (KIND == 0) {
                        v[i] = __builtin_nontemporal_load(pk + (t + i) * 128 + off);
                        v[H + i] = __builtin_nontemporal_load(pv + (t + i) * 128 + off);
                    } else {
                        v[i] = __builtin_amdgcn_raw_buffer_load_b128(rk, ((t + i) * 128 + off) * 16, 0, POLICY);
                        v[H + i] = __builtin_amdgcn_raw_buffer_load_b128(rv, ((t + i) * 128 + off) * 16, 0, POLICY);
                    }
                }
#pragma unroll
                for (int i = 0; i < kInFlight; ++i) consume(v[i]);
            }
        }
    }
    if (a0 + a1 + a2 + a3 == 1.2345f) out[0] = a0;  // keeps the loads alive
}

template <int PATTERN, int KIND, int POLICY, int WORK>
int measure(const char *what, const u4 *k, const u4 *v, const int *pages, int npages, float *out) {
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    for (int it = 0; it < 10; ++it) read_kernel<PATTERN, KIND, POLICY, WORK><<<512, 256>>>(k, v, pages, npages, out);
    CK(hipEventRecord(e0));
    for (int it = 0; it < 20; ++it) read_kernel<PATTERN, KIND, POLICY, WORK><<<512, 256>>>(k, v, pages, npages, out);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms = 0.f;
    CK(hipEventElapsedTime(&ms, e0, e1));
    ms /= 20;
    std::printf("%-86s %7.1f us  %6.0f GB/s\n", what, ms * 1e3, 2.0 * npages * 32768 / ms / 1e6);
    return 0;
}

int main() {
    const int npages = 52656;  // per pool: the 52 656 blocks of 16 tokens of workload c4 (Hkv=8, D=128, bf16)
    const size_t bytes = (size_t)npages * 32768;
    char *k = nullptr, *v = nullptr;
    float *out = nullptr;
    int *pages = nullptr;
    CK(hipMalloc(&k, bytes));
    CK(hipMalloc(&v, bytes));
    CK(hipMalloc(&out, 4));
    CK(hipMalloc(&pages, npages * sizeof(int)));
    CK(hipMemset(k, 1, bytes));
    CK(hipMemset(v, 1, bytes));
    std::vector<int> order(npages);
    std::iota(order.begin(), order.end(), 0);
    std::mt19937 gen(1);
    std::shuffle(order.begin(), order.end(), gen);
    CK(hipMemcpy(pages, order.data(), npages * sizeof(int), hipMemcpyHostToDevice));
    const u4 *pk = (const u4 *)k, *pv = (const u4 *)v;
    int rc = 0;
    rc |= measure<0, 0, 0, 0>("contiguous pages, global loads, default policy", pk, pv, pages, npages, out);
    rc |= measure<0, 0, 2, 0>("contiguous pages, global loads, nt", pk, pv, pages, npages, out);
    rc |= measure<1, 0, 2, 0>("half token rows, K and V alternating, global loads, nt", pk, pv, pages, npages, out);
    rc |= measure<1, 1, 2, 0>("half token rows, K and V alternating, buffer loads, nt", pk, pv, pages, npages, out);
    rc |= measure<1, 1, 19, 0>("half token rows, K and V alternating, buffer loads, sc0 sc1 nt", pk, pv, pages, npages, out);
    rc |= measure<1, 1, 1, 0>("half token rows, K and V alternating, buffer loads, sc0 (no nt)", pk, pv, pages, npages, out);
    rc |= measure<1, 1, 0, 0>("half token rows, K and V alternating, buffer loads, default policy", pk, pv, pages, npages, out);
    rc |= measure<1, 1, 2, 32>("half token rows, buffer loads, nt, 32 multiply-adds per load", pk, pv, pages, npages, out);
    rc |= measure<1, 1, 2, 48>("half token rows, buffer loads, nt, 48 multiply-adds per load", pk, pv, pages, npages, out);
    rc |= measure<1, 1, 2, 64>("half token rows, buffer loads, nt, 64 multiply-adds per load", pk, pv, pages, npages, out);
    return rc;
}
