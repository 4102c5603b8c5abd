// Shared by every kernel file of the library: element types, conversions,
// wave/block reductions, the error convention of the C entry points.
//
// Target: gfx950 (CDNA4), 64-wide wavefronts.  Every extern "C" entry point
// returns nullptr on success or a message (valid until the thread's next call)
// that names what was refused; it checks its arguments on the host before any
// launch, so a refused call has launched nothing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define CPMCU_WAVE 64

// element type codes of the C ABI
enum { CPMCU_F32 = 0, CPMCU_BF16 = 1 };

struct bf16_t {
    uint16_t v;
};

__host__ __device__ inline float to_f32(float x) { return x; }
__host__ __device__ inline float to_f32(bf16_t x) {
    union { uint32_t u; float f; } c;
    c.u = ((uint32_t)x.v) << 16;
    return c.f;
}
// round to nearest even; NaN stays NaN
__host__ __device__ inline bf16_t f32_to_bf16(float f) {
    union { uint32_t u; float f; } c;
    c.f = f;
    uint32_t u = c.u;
    bf16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        r.v = (uint16_t)((u >> 16) | 0x40);
    } else {
        u += 0x7fffu + ((u >> 16) & 1u);
        r.v = (uint16_t)(u >> 16);
    }
    return r;
}
template <typename T> __host__ __device__ inline T from_f32(float f);
template <> __host__ __device__ inline float from_f32<float>(float f) { return f; }
template <> __host__ __device__ inline bf16_t from_f32<bf16_t>(float f) { return f32_to_bf16(f); }

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int o = CPMCU_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, CPMCU_WAVE);
    return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int o = CPMCU_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, CPMCU_WAVE));
    return v;
}
// Sum over a block of up to 1024 threads; every thread gets the result.
// `red` is LDS for 17 floats.  The order of the additions is fixed, so the
// result does not depend on timing.
__device__ inline float block_sum(float v, float* red) {
    const int lane = threadIdx.x & (CPMCU_WAVE - 1), w = threadIdx.x / CPMCU_WAVE;
    const int nw = (blockDim.x + CPMCU_WAVE - 1) / CPMCU_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    // every thread adds the wave sums in the same order
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}
__device__ inline float block_max(float v, float* red) {
    const int lane = threadIdx.x & (CPMCU_WAVE - 1), w = threadIdx.x / CPMCU_WAVE;
    const int nw = (blockDim.x + CPMCU_WAVE - 1) / CPMCU_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
    return t;
}

// ---- error convention ----
inline char* cpmcu_errbuf() {
    static thread_local char buf[512];
    return buf;
}
#define CPMCU_FAIL(...)                                        \
    do {                                                       \
        snprintf(cpmcu_errbuf(), 512, __VA_ARGS__);            \
        return cpmcu_errbuf();                                 \
    } while (0)
#define CPMCU_REQUIRE(cond, ...)                               \
    do {                                                       \
        if (!(cond)) CPMCU_FAIL(__VA_ARGS__);                  \
    } while (0)
#define CPMCU_LAUNCH_CHECK(name)                                                          \
    do {                                                                                  \
        hipError_t e_ = hipGetLastError();                                                \
        if (e_ != hipSuccess) CPMCU_FAIL("%s: launch failed: %s", name, hipGetErrorString(e_)); \
    } while (0)

// Where a token's row lies in a paged stream: the page table of its slot maps
// page number -> physical page; a stream holds `rows_per_page` rows a page.
struct PagedView {
    const int* page_table;   // [slots, table_width]
    int table_width;
    int page_size;           // tokens a page
};
__device__ inline long paged_row(const PagedView& pv, int slot, int pos) {
    const int page = pv.page_table[(long)slot * pv.table_width + pos / pv.page_size];
    return (long)page * pv.page_size + pos % pv.page_size;
}

// Values are kept transposed in tiles of value_tile() tokens inside a page,
// [page][kv head][tile][d][token of the tile], so that attention reads, for one d, the values of consecutive
// keys as one vector and a chunk of 32 keys is one contiguous piece of memory.
__host__ __device__ inline int value_tile(int page_size) { return page_size % 32 == 0 ? 32 : page_size; }
__device__ inline long value_index(long page, int in_page, int kvh, int d, int nkv, int hd, int page_size) {
    const int vt = value_tile(page_size);
    return (((page * nkv + kvh) * (page_size / vt) + in_page / vt) * hd + d) * vt + in_page % vt;
}
