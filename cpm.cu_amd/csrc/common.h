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

// Max / sum over the four rows of 16 lanes of a wavefront (lanes that differ in bits 4 and 5 only); every
// lane gets the result.  gfx950's row swaps exchange rows between two registers inside the vector unit:
// swapping a value with itself leaves (row 0, row 0, row 2, row 2) and (row 1, row 1, row 3, row 3).
typedef unsigned cpmcu_u32x2_t __attribute__((ext_vector_type(2)));
__device__ inline float rows_max(float v) {
    cpmcu_u32x2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ inline float rows_sum(float v) {
    cpmcu_u32x2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// Sum / max over the 64 lanes of a wavefront, the result in every lane, inside the vector unit: four steps
// over a row of 16 lanes with the data-parallel lane patterns (neighbours, pairs, mirrored halves of 8,
// mirrored halves of 16), then the four rows.  The order of the operations is fixed.
// (a lane whose partner is switched off reads `idle`: 0 for sums, its own value for maxima)
#define CPMCU_DPP(v, ctrl) __uint_as_float(__builtin_amdgcn_update_dpp(0, __float_as_uint(v), ctrl, 0xf, 0xf, false))
#define CPMCU_DPP_SELF(v, ctrl) \
    __uint_as_float(__builtin_amdgcn_update_dpp(__float_as_uint(v), __float_as_uint(v), ctrl, 0xf, 0xf, false))
__device__ inline float row16_sum(float v) {
    v += CPMCU_DPP(v, 0xB1);      // quad_perm [1,0,3,2]
    v += CPMCU_DPP(v, 0x4E);      // quad_perm [2,3,0,1]
    v += CPMCU_DPP(v, 0x141);     // row_half_mirror
    v += CPMCU_DPP(v, 0x140);     // row_mirror
    return v;
}
__device__ inline float row16_max(float v) {
    v = fmaxf(v, CPMCU_DPP_SELF(v, 0xB1));
    v = fmaxf(v, CPMCU_DPP_SELF(v, 0x4E));
    v = fmaxf(v, CPMCU_DPP_SELF(v, 0x141));
    v = fmaxf(v, CPMCU_DPP_SELF(v, 0x140));
    return v;
}
__device__ inline float wave_sum(float v) { return rows_sum(row16_sum(v)); }
__device__ inline float wave_max(float v) { return rows_max(row16_max(v)); }
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

// ---- the norm's row factor, for products that apply it at their end ----
// add_norm_columns leaves x * w and, for every row, the sums of x^2 over slices of NORM_SLICE columns;
// r = rsqrt(sum of the slices / width + eps).  A workgroup of NT threads forms r for its ROWS rows at its
// start: NT / ROWS neighbouring lanes share a row, each adds a contiguous run of the slices (16-byte loads,
// four in flight, when the rows are aligned: a loop of dependent 4-byte loads cost 9 us in a 64-row product),
// the lanes' shares meet inside the vector unit and the first lane writes r to rs_out[row] (LDS; the caller's
// next barrier makes it visible).
#define NORM_SLICE 64
template <int TPR>
__device__ inline float lanes_sum(float v) {
    static_assert(TPR == 1 || TPR == 2 || TPR == 4 || TPR == 8 || TPR == 16, "lanes a row");
    if (TPR >= 2) v += CPMCU_DPP(v, 0xB1);      // quad_perm [1,0,3,2]
    if (TPR >= 4) v += CPMCU_DPP(v, 0x4E);      // quad_perm [2,3,0,1]
    if (TPR >= 8) v += CPMCU_DPP(v, 0x141);     // row_half_mirror
    if (TPR >= 16) v += CPMCU_DPP(v, 0x140);    // row_mirror
    return v;
}
template <int NT, int ROWS>
__device__ inline void row_scales(const float* __restrict__ row_ss, int n_slices, int n_rows, float inv_width,
                                  float eps, float* rs_out) {
    constexpr int TPR = NT / ROWS;
    const int row = threadIdx.x / TPR, part = threadIdx.x % TPR;
    const float* src = row_ss + (long)min(row, n_rows - 1) * n_slices;
    const int per = ((n_slices + TPR - 1) / TPR + 3) & ~3;
    const int i0 = part * per, i1 = min(i0 + per, n_slices);
    float s = 0.f;
    if ((n_slices & 3) == 0) {
#pragma unroll 4
        for (int i = i0; i < i1; i += 4) {
            const float4 v = *(const float4*)(src + i);
            s += (v.x + v.y) + (v.z + v.w);
        }
    } else {
        for (int i = i0; i < i1; ++i) s += src[i];
    }
    s = lanes_sum<TPR>(s);
    if (part == 0) rs_out[row] = 1.0f / sqrtf(s * inv_width + eps);
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

// Keys and values of a page lie in the order in which the matrix cores take them, so that a wavefront's
// operand load is one contiguous KiB (loads of 16 bytes a lane that are scattered over rows keep the
// address unit busy four times as long).  A page holds a multiple of 32 tokens; per chunk of 32 tokens
// and kv head (the chunk comes first: physical chunk number = physical token row / 32):
//   keys:   two tiles of 16 key slots (token 8a + 4u + i of the chunk is slot 4a + i of tile u; a lane's 8
//           scores of a chunk are then 8 consecutive keys), a tile is [d / 8][slot][d % 8]
//   values: [d / 16][token / 8][d % 16][token % 8], the transposed operand of P.V
// key_index / value_index give the element of (token row, d = 0); *_d_offset adds d.
__host__ __device__ inline long chunk_base(long row, int kvh, int nkv, int hd) {
    return ((row >> 5) * nkv + kvh) * (32L * hd);
}
__host__ __device__ inline long key_index(long row, int kvh, int nkv, int hd) {
    const int t32 = (int)(row & 31);
    const int u = (t32 >> 2) & 1, slot = ((t32 >> 3) << 2) | (t32 & 3);
    return chunk_base(row, kvh, nkv, hd) + (u * (hd >> 3) * 16 + slot) * 8;
}
__host__ __device__ inline int key_d_offset(int d) { return (d >> 3) * 128 + (d & 7); }
__host__ __device__ inline long value_index(long row, int kvh, int nkv, int hd) {
    const int t32 = (int)(row & 31);
    return chunk_base(row, kvh, nkv, hd) + (t32 >> 3) * 128 + (t32 & 7);
}
__host__ __device__ inline int value_d_offset(int d) { return (d >> 4) * 512 + (d & 15) * 8; }

// Compressed keys (one row for every `stride` tokens, rows_per_page rows a page) lie per kv head as
// [d / 8][row of the page][d % 8]: neighbouring lanes of a matrix-core operand load, which hold neighbouring
// rows, then read neighbouring 16 bytes.
__host__ __device__ inline long ck_index(long page, int row_in_page, int kvh, int nkv, int hd, int rows_per_page) {
    return ((page * nkv + kvh) * (hd >> 3) * rows_per_page + row_in_page) * 8;
}
__host__ __device__ inline int ck_d_offset(int d, int rows_per_page) { return (d >> 3) * rows_per_page * 8 + (d & 7); }
