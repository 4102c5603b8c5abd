// Row-wise kernels around the matrix products: token embedding, residual add
// fused with RMSNorm, SiLU gating, rotary position encoding fused with the
// write of keys and values into the paged cache.
//
// The residual stream is always float; `T` is the activation/weight element
// type of the engine (float in the 32-bit engine, bf16 in the serving one).
// All statistics (sum of squares, rsqrt, angles, sin/cos, sigmoid) are float.
#include "common.h"

// ---------------------------------------------------------------------------
// embedding:  out[r,:] = float(table[ids[r],:]) * scale
// (reference: src/model/embedding.cuh:7-20 gathers, elementwise.cuh:34-41 scales)
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids, float* __restrict__ out,
                             int H, float scale) {
    const long r = blockIdx.x;
    const T* src = table + (long)ids[r] * H;
    float* dst = out + r * H;
    for (int c = threadIdx.x; c < H; c += blockDim.x) dst[c] = to_f32(src[c]) * scale;
}

extern "C" const char* cpmcu_embed(const void* table, int dtype, const int* ids, float* out, int n, int H, int V,
                                   float scale, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && V > 0, "embed: empty shape n=%d H=%d V=%d", n, H, V);
    CPMCU_REQUIRE(dtype == CPMCU_F32 || dtype == CPMCU_BF16, "embed: unknown dtype %d", dtype);
    const int block = H >= 1024 ? 256 : 64;
    if (dtype == CPMCU_F32)
        embed_kernel<float><<<n, block, 0, stream>>>((const float*)table, ids, out, H, scale);
    else
        embed_kernel<bf16_t><<<n, block, 0, stream>>>((const bf16_t*)table, ids, out, H, scale);
    CPMCU_LAUNCH_CHECK("embed");
    return nullptr;
}

// ---------------------------------------------------------------------------
// x += bscale * sum_p branch[p]   (written back unless `rows` selects rows)
// out = x * rsqrt(mean(x^2) + eps) * w
// (reference: src/model/norm.cuh:53-99; eps inside the root, weight after)
// `branch` may be null (plain norm), and may come as `nparts` partial sums of
// a split matrix product, `part_stride` elements apart.
// ---------------------------------------------------------------------------
// The sum of nparts partial results `stride` elements apart, added in the order of the parts, up to 4 (8)
// loads asked for together (see add_parts4 below for why).
template <int W, typename BT>
__device__ inline float add_parts(float acc, const BT* p, int first, int nparts, long stride) {
    float t[W];
#pragma unroll
    for (int j = 0; j < W; ++j) t[j] = to_f32(p[(long)min(first + j, nparts - 1) * stride]);
#pragma unroll
    for (int j = 0; j < W; ++j)
        if (first + j < nparts) acc += t[j];
    return acc;
}
template <typename BT>
__device__ inline float sum_parts(const BT* p, int nparts, long stride) {
    if (nparts <= 4) return add_parts<4>(0.f, p, 0, nparts, stride);
    float b = 0.f;
    for (int f = 0; f < nparts; f += 8) b = add_parts<8>(b, p, f, nparts, stride);
    return b;
}

template <typename BT, typename OT>
__global__ void add_rms_norm_kernel(float* __restrict__ x, const BT* __restrict__ branch, int nparts,
                                    long part_stride, float bscale, const float* __restrict__ w, float eps,
                                    OT* __restrict__ out, const int* __restrict__ rows, int H) {
    __shared__ float red[17];
    const long r_out = blockIdx.x;
    const long r = rows ? rows[r_out] : r_out;
    float* xr = x + r * H;
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float v = xr[c];
        if (branch) {
            const float b = sum_parts(branch + r * H + c, nparts, part_stride);
            v += bscale * b;
            if (!rows) xr[c] = v;
        }
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)H + eps);
    OT* o = out + r_out * H;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float v = xr[c];
        if (branch && rows) {
            const float b = sum_parts(branch + r * H + c, nparts, part_stride);
            v += bscale * b;
        }
        o[c] = from_f32<OT>(v * rs * w[c]);
    }
}

// The same with 4 columns a thread and 16-byte accesses (H a multiple of 4, float branch or none):
// the decode steps' norms have few rows and up to 16 partial sums to add, so the row's work
// is spread over up to 1024 threads.
__device__ inline void store4(float* p, float a, float b, float c, float d) { *(float4*)p = make_float4(a, b, c, d); }
__device__ inline void store4(bf16_t* p, float a, float b, float c, float d) {
    const bf16_t o0 = f32_to_bf16(a), o1 = f32_to_bf16(b), o2 = f32_to_bf16(c), o3 = f32_to_bf16(d);
    *(uint2*)p = make_uint2((uint32_t)o0.v | ((uint32_t)o1.v << 16), (uint32_t)o2.v | ((uint32_t)o3.v << 16));
}
__device__ inline float4 load4(const float* p) { return *(const float4*)p; }
__device__ inline float4 load4(const bf16_t* p) {
    const uint2 u = *(const uint2*)p;
    float4 r;
    r.x = __uint_as_float(u.x << 16);
    r.y = __uint_as_float(u.x & 0xffff0000u);
    r.z = __uint_as_float(u.y << 16);
    r.w = __uint_as_float(u.y & 0xffff0000u);
    return r;
}
// acc + the partial results first .. first + W - 1 (of nparts, `stride` elements apart), added in the order of
// the parts.  The W loads are asked for together: a loop of single loads whose trip count the compiler does not
// know waits for each load before it asks for the next, a trip to memory a part.  A part beyond the last repeats
// the last one and is not added.
template <int W, typename BT>
__device__ inline float4 add_parts4(float4 acc, const BT* p, int first, int nparts, long stride) {
    float4 t[W];
#pragma unroll
    for (int j = 0; j < W; ++j) t[j] = load4(p + (long)min(first + j, nparts - 1) * stride);
#pragma unroll
    for (int j = 0; j < W; ++j)
        if (first + j < nparts) {
            acc.x += t[j].x; acc.y += t[j].y; acc.z += t[j].z; acc.w += t[j].w;
        }
    return acc;
}
template <typename BT>
__device__ inline float4 sum_parts4(const BT* p, int nparts, long stride) {
    float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
    if (nparts <= 4) return add_parts4<4>(b, p, 0, nparts, stride);
    for (int f = 0; f < nparts; f += 8) b = add_parts4<8>(b, p, f, nparts, stride);
    return b;
}

template <typename BT, typename OT>
__global__ __launch_bounds__(1024) void add_rms_norm_vec4_kernel(float* __restrict__ x, const BT* __restrict__ branch,
                                                                 int nparts, long part_stride, float bscale,
                                                                 const float* __restrict__ w, float eps,
                                                                 OT* __restrict__ out, const int* __restrict__ rows, int H) {
    __shared__ float red[17];
    const long r_out = blockIdx.x;
    const long r = rows ? rows[r_out] : r_out;
    float* xr = x + r * H;
    const int H4 = H / 4;
    OT* o = out + r_out * H;
    auto summed = [&](int c) {
        float4 v = *(const float4*)(xr + 4 * c);
        if (branch) {
            const float4 b = sum_parts4(branch + r * H + 4 * c, nparts, part_stride);
            v.x += bscale * b.x; v.y += bscale * b.y; v.z += bscale * b.z; v.w += bscale * b.w;
        }
        return v;
    };
    auto emit = [&](int c, float4 v, float rs) {
        const float4 wv = *(const float4*)(w + 4 * c);
        store4(o + 4 * c, v.x * rs * wv.x, v.y * rs * wv.y, v.z * rs * wv.z, v.w * rs * wv.w);   // one store of 16 or 8 bytes
    };
    if (H4 <= (int)blockDim.x) {
        // the whole row fits the block: each thread keeps its 4 columns in registers between the two phases
        const int c = threadIdx.x;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c < H4) {
            v = summed(c);
            if (branch && !rows) *(float4*)(xr + 4 * c) = v;
        }
        const float ss = block_sum(v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w, red);
        if (c < H4) emit(c, v, 1.0f / sqrtf(ss / (float)H + eps));
        return;
    }
    if (H4 <= 4 * (int)blockDim.x) {
        // up to 4 vectors a thread stay in registers as well (many rows: blocks of 256 threads, rows of 4,096)
        float4 v[4];
        float ss = 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int c = threadIdx.x + k * blockDim.x;
            v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (c < H4) {
                v[k] = summed(c);
                if (branch && !rows) *(float4*)(xr + 4 * c) = v[k];
            }
            ss += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
        }
        const float rs = 1.0f / sqrtf(block_sum(ss, red) / (float)H + eps);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int c = threadIdx.x + k * blockDim.x;
            if (c < H4) emit(c, v[k], rs);
        }
        return;
    }
    float ss = 0.f;
    for (int c = threadIdx.x; c < H4; c += blockDim.x) {
        const float4 v = summed(c);
        if (branch && !rows) *(float4*)(xr + 4 * c) = v;
        ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    ss = block_sum(ss, red);
    const float rs = 1.0f / sqrtf(ss / (float)H + eps);
    for (int c = threadIdx.x; c < H4; c += blockDim.x) {
        // x holds the sum already unless only chosen rows are normed (then it is formed again)
        const float4 v = (branch && rows) ? summed(c) : *(const float4*)(xr + 4 * c);
        emit(c, v, rs);
    }
}

extern "C" const char* cpmcu_add_rms_norm(float* x, const void* branch, int branch_dtype, int nparts,
                                          long part_stride, float bscale, const float* w, float eps, void* out,
                                          int out_dtype, const int* rows, int n_out, int H, hipStream_t stream) {
    CPMCU_REQUIRE(n_out > 0 && H > 0, "add_rms_norm: empty shape rows=%d H=%d", n_out, H);
    CPMCU_REQUIRE(!branch || nparts >= 1, "add_rms_norm: nparts=%d", nparts);
    if (H % 4 == 0 && ((uintptr_t)x % 16 == 0) && (!branch || ((uintptr_t)branch % 16 == 0 && part_stride % 4 == 0)) &&
        ((uintptr_t)w % 16 == 0) && ((uintptr_t)out % 16 == 0) && (out_dtype == CPMCU_F32 || out_dtype == CPMCU_BF16) &&
        (branch_dtype == CPMCU_F32 || branch_dtype == CPMCU_BF16)) {
        const int h4 = H / 4;
        // many rows: smaller blocks keep more rows in flight on a CU; few rows: spread a row over many threads
        const int cap = n_out >= 512 ? 256 : 1024;
        int vblock = 64;
        while (vblock < cap && vblock < h4) vblock *= 2;
#define VLAUNCH(BT, OT)                                                                                             \
        add_rms_norm_vec4_kernel<BT, OT><<<n_out, vblock, 0, stream>>>(x, (const BT*)branch, nparts, part_stride,   \
                                                                       bscale, w, eps, (OT*)out, rows, H)
        if (branch_dtype == CPMCU_F32 && out_dtype == CPMCU_F32) VLAUNCH(float, float);
        else if (branch_dtype == CPMCU_F32) VLAUNCH(float, bf16_t);
        else if (out_dtype == CPMCU_F32) VLAUNCH(bf16_t, float);
        else VLAUNCH(bf16_t, bf16_t);
#undef VLAUNCH
        CPMCU_LAUNCH_CHECK("add_rms_norm");
        return nullptr;
    }
    const int block = H >= 2048 ? 512 : (H >= 512 ? 256 : 64);
#define LAUNCH(BT, OT)                                                                                         \
    add_rms_norm_kernel<BT, OT><<<n_out, block, 0, stream>>>(x, (const BT*)branch, nparts, part_stride, bscale, \
                                                             w, eps, (OT*)out, rows, H)
    if (branch_dtype == CPMCU_F32 && out_dtype == CPMCU_F32) LAUNCH(float, float);
    else if (branch_dtype == CPMCU_F32 && out_dtype == CPMCU_BF16) LAUNCH(float, bf16_t);
    else if (branch_dtype == CPMCU_BF16 && out_dtype == CPMCU_F32) LAUNCH(bf16_t, float);
    else if (branch_dtype == CPMCU_BF16 && out_dtype == CPMCU_BF16) LAUNCH(bf16_t, bf16_t);
    else CPMCU_FAIL("add_rms_norm: unknown dtypes %d %d", branch_dtype, out_dtype);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("add_rms_norm");
    return nullptr;
}

// The norm of a step of few rows, cut by columns instead of rows.  rmsnorm(x) . W^T = r * ((x * w) . W^T) with
// r = rsqrt(mean(x^2) + eps) one number a row: the product that follows can multiply by r at its end, so
// nothing here needs a whole row.  A workgroup takes 64 columns of 16 rows: x += bscale * sum of the branch's
// parts (in place), out = bf16(x * w), and row_ss[row][slice] = the slice's sum of x^2; the consumer adds the
// slices up (common.h: row_scale_of).  A row a workgroup reads its partial sums through one CU at 6-7 us for
// 8 rows of 4,096 columns; cut this way the same work is spread over 64 CUs.
// (reference: src/model/norm.cuh:53-99, add and norm in one kernel, one block a row)
template <typename BT>
__global__ __launch_bounds__(256) void add_norm_columns_kernel(float* __restrict__ x, const BT* __restrict__ branch,
                                                               int nparts, long part_stride, float bscale,
                                                               const float* __restrict__ w, bf16_t* __restrict__ out,
                                                               float* __restrict__ row_ss, int n, int H, int n_slices) {
    const int slice = blockIdx.x, l16 = threadIdx.x & 15;
    const int row = blockIdx.y * 16 + (threadIdx.x >> 4);
    const int c = slice * NORM_SLICE + l16 * 4;
    const bool ok = row < n && c < H;
    const long off = (long)min(row, n - 1) * H + min(c, H - 4);
    float4 v = *(const float4*)(x + off);
    if (branch) {
        const float4 b = sum_parts4(branch + off, nparts, part_stride);
        v.x += bscale * b.x; v.y += bscale * b.y; v.z += bscale * b.z; v.w += bscale * b.w;
    }
    float ss = 0.f;
    if (ok) {
        if (branch) *(float4*)(x + off) = v;
        const float4 wv = *(const float4*)(w + c);
        const bf16_t o0 = f32_to_bf16(v.x * wv.x), o1 = f32_to_bf16(v.y * wv.y);
        const bf16_t o2 = f32_to_bf16(v.z * wv.z), o3 = f32_to_bf16(v.w * wv.w);
        *(uint2*)(out + off) = make_uint2((uint32_t)o0.v | ((uint32_t)o1.v << 16), (uint32_t)o2.v | ((uint32_t)o3.v << 16));
        ss = v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    ss = row16_sum(ss);                      // the 16 lanes of a row of x are one row of lanes
    if (l16 == 0 && row < n) row_ss[(long)row * n_slices + slice] = ss;
}

extern "C" const char* cpmcu_add_norm_columns(float* x, const void* branch, int branch_dtype, int nparts,
                                              long part_stride, float bscale, const float* w, void* out,
                                              float* row_ss, int n, int H, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && H > 0 && H % 4 == 0, "add_norm_columns: rows=%d, H=%d must be a positive multiple of 4", n, H);
    CPMCU_REQUIRE(!branch || (nparts >= 1 && part_stride % 4 == 0), "add_norm_columns: nparts=%d stride=%ld", nparts, part_stride);
    CPMCU_REQUIRE(x && w && out && row_ss, "add_norm_columns: null pointer");
    CPMCU_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) && ((uintptr_t)out % 8 == 0) &&
                  (!branch || (uintptr_t)branch % 16 == 0), "add_norm_columns: operands must be 16-byte aligned");
    const int n_slices = (H + NORM_SLICE - 1) / NORM_SLICE;
    dim3 grid(n_slices, (n + 15) / 16);
    if (!branch || branch_dtype == CPMCU_F32)
        add_norm_columns_kernel<float><<<grid, 256, 0, stream>>>(x, (const float*)branch, nparts, part_stride, bscale, w,
                                                                 (bf16_t*)out, row_ss, n, H, n_slices);
    else if (branch_dtype == CPMCU_BF16)
        add_norm_columns_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, (const bf16_t*)branch, nparts, part_stride, bscale,
                                                                  w, (bf16_t*)out, row_ss, n, H, n_slices);
    else CPMCU_FAIL("add_norm_columns: unknown branch dtype %d", branch_dtype);
    CPMCU_LAUNCH_CHECK("add_norm_columns");
    return nullptr;
}

// ---------------------------------------------------------------------------
// out[r,c] = silu(gu[r,c]) * gu[r,c+I],  silu(g) = g / (1 + exp(-g))
// (reference: src/model/activation.cuh:6-18, gate columns first, then up)
// ---------------------------------------------------------------------------
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, long n, int I) {
    const long total = n * I;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const long r = i / I;
        const int c = (int)(i - r * I);
        const float g = to_f32(gu[r * 2 * I + c]);
        const float u = to_f32(gu[r * 2 * I + I + c]);
        out[i] = from_f32<T>(g / (1.0f + expf(-g)) * u);
    }
}

// bf16, I a multiple of 8: 8 columns a thread with 16-byte accesses, U such pieces of a row in flight a thread
// (the pieces of a thread lie a whole block apart, so every load of a wavefront is one contiguous KiB).  The
// result is rounded to bfloat16, so the exponential and the reciprocal are the bare hardware instructions
// (2^-22 relative; the 32-bit engine's kernel above keeps expf and a true division).
template <int U>
__global__ __launch_bounds__(256) void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out,
                                                              long n, int I) {
    const int I8 = I / 8;
    const long total = n * I8;
    const long base = (long)blockIdx.x * (256 * U) + threadIdx.x;
    uint4 g4[U], u4[U];
    long at[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
        const long i = min(base + k * 256, total - 1);            // a piece beyond the end repeats the last one
        const long r = i / I8;
        const int c = (int)(i - r * I8) * 8;
        at[k] = r * I + c;
        g4[k] = *(const uint4*)(gu + r * 2 * I + c);
        u4[k] = *(const uint4*)(gu + r * 2 * I + I + c);
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
        if (base + k * 256 >= total) break;
        const uint32_t gw[4] = {g4[k].x, g4[k].y, g4[k].z, g4[k].w}, uw[4] = {u4[k].x, u4[k].y, u4[k].z, u4[k].w};
        uint32_t ow[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
            const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
            const float s0 = g0 * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g0));
            const float s1 = g1 * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g1));
            const bf16_t a = f32_to_bf16(s0 * u0);
            const bf16_t b = f32_to_bf16(s1 * u1);
            ow[j] = (uint32_t)a.v | ((uint32_t)b.v << 16);
        }
        *(uint4*)(out + at[k]) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
}

extern "C" const char* cpmcu_silu_mul(const void* gu, void* out, int dtype, int n, int I, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && I > 0, "silu_mul: empty shape n=%d I=%d", n, I);
    if (dtype == CPMCU_BF16 && I % 8 == 0 && (uintptr_t)gu % 16 == 0 && (uintptr_t)out % 16 == 0) {
        const long total8 = (long)n * (I / 8);
        // many rows: 4 pieces a thread in flight; few: one, for more workgroups
        if (total8 >= 4L * 256 * 2048) {
            const long wgs = (total8 + 4 * 256 - 1) / (4 * 256);
            CPMCU_REQUIRE(wgs <= 0x7fffffffL, "silu_mul: %d rows of %d columns exceed the launch grid", n, I);
            silu_mul_bf16x8_kernel<4><<<(unsigned)wgs, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, n, I);
        } else {
            const long wgs = (total8 + 255) / 256;
            CPMCU_REQUIRE(wgs <= 0x7fffffffL, "silu_mul: %d rows of %d columns exceed the launch grid", n, I);
            silu_mul_bf16x8_kernel<1><<<(unsigned)wgs, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, n, I);
        }
        CPMCU_LAUNCH_CHECK("silu_mul");
        return nullptr;
    }
    const long total = (long)n * I;
    const int block = 256;
    const int grid = (int)((total + block - 1) / block < 65535 * 16 ? (total + block - 1) / block : 65535 * 16);
    if (dtype == CPMCU_F32)
        silu_mul_kernel<float><<<grid, block, 0, stream>>>((const float*)gu, (float*)out, n, I);
    else if (dtype == CPMCU_BF16)
        silu_mul_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, n, I);
    else
        CPMCU_FAIL("silu_mul: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("silu_mul");
    return nullptr;
}

// ---------------------------------------------------------------------------
// Rotary position encoding (rotate-half) on q and k, then k and v into the
// paged cache.  A row of `qkv` (`row_width` elements) is [q: nh*hd | k: nkv*hd | v: nkv*hd]; it may
// come as `nparts` float partial sums of a split matrix product.  q is written
// to `q_out` (row stride nh*hd).  theta = pos * inv_freq[c];
// (a, b) = (x[c], x[c+hd/2]) -> (a cos - b sin, a sin + b cos), cos and sin
// times `mscale` (reference: src/model/rotary.cuh:7-34; cache rows
// src/model/attn.cuh:14-21).  inv_freq null: no rotation.  In the cache,
// keys and values lie in their page in the matrix cores' operand order (key_index, value_index).
// ---------------------------------------------------------------------------
template <typename IT, typename T>
__global__ void rope_store_kernel(const IT* __restrict__ qkv, long width, int nparts, long part_stride,
                                  T* __restrict__ q_out, int nh, int nkv, int hd, const int* __restrict__ positions,
                                  const int* __restrict__ tok_slot, const float* __restrict__ inv_freq, float mscale,
                                  T* __restrict__ kpool, T* __restrict__ vpool, PagedView pv, int write_kv) {
    // 64 threads a (token, head) at a time: heads [0, nh) are queries, then nkv key heads, then nkv value heads.
    // The groups of 64 threads of the token's blocks take its heads in turn; a group forms the angles' cos and
    // sin once (they are the same for every head) and keeps them for the pairs c = lane and lane + 64.
    const long t = blockIdx.x;
    const int groups = gridDim.y * (blockDim.x >> 6);
    const int group = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int heads = nh + (write_kv ? 2 * nkv : 0);
    if (group >= heads) return;
    const int half = hd / 2;
    const int pos = positions[t];
    auto trig = [&](int c, float& cs, float& sn) {
        cs = 1.f;
        sn = 0.f;
        if (inv_freq && c < half) {
            const float ang = (float)pos * inv_freq[c];
            cs = cosf(ang) * mscale;
            sn = sinf(ang) * mscale;
        }
    };
    float cs0, sn0, cs1, sn1;
    trig(lane, cs0, sn0);
    trig(lane + 64, cs1, sn1);
    const long kv_row = write_kv ? paged_row(pv, tok_slot[t], pos) : 0;
    for (int head = group; head < heads; head += groups) {
        const IT* row = qkv + t * width + (long)head * hd;
        auto load = [&](int i) {
            return sum_parts(row + i, nparts, part_stride);
        };
        if (head < nh + nkv) {
            // queries go out as plain rows; keys into their page in the matrix cores' order (key_index)
            const bool is_q = head < nh;
            T* dst = is_q ? q_out + (t * nh + head) * (long)hd : kpool + key_index(kv_row, head - nh, nkv, hd);
            auto at = [&](int d) { return is_q ? d : key_d_offset(d); };
            for (int c = lane; c < half; c += 64) {
                float cs = cs0, sn = sn0;
                if (c >= 64) {
                    cs = cs1;
                    sn = sn1;
                }
                if (c >= 128) trig(c, cs, sn);
                const float a = load(c), b = load(c + half);
                dst[at(c)] = from_f32<T>(a * cs - b * sn);
                dst[at(c + half)] = from_f32<T>(a * sn + b * cs);
            }
        } else {
            // values go into their page transposed, in the matrix cores' order (value_index)
            T* dst = vpool + value_index(kv_row, head - nh - nkv, nkv, hd);
            for (int d = lane; d < hd; d += 64) dst[value_d_offset(d)] = from_f32<T>(load(d));
        }
    }
}

// The same for steps of many tokens in bf16 (one input slice): 16-byte accesses.  A block takes 8 tokens; lane
// (token, piece) of a wavefront owns the 8 rotation pairs c = 8 piece .. 8 piece + 7 of its token, forms their
// cos and sin once and applies them to every head the wavefront takes (every fourth); values are written by
// a thread a (kv head, d) for the block's 8 tokens.  head_dim is a multiple of 16, at most 128.
typedef __bf16 ebf16x8_t __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(256) void rope_store_rows_kernel(
    const bf16_t* __restrict__ qkv, long width, bf16_t* __restrict__ q_out, int n, int nh, int nkv, int hd,
    const int* __restrict__ positions, const int* __restrict__ tok_slot, const float* __restrict__ inv_freq,
    float mscale, bf16_t* __restrict__ kpool, bf16_t* __restrict__ vpool, PagedView pv, int write_kv) {
    __shared__ long rows_s[8];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int half = hd / 2, pieces = half / 8;           // pieces <= 8
    if (threadIdx.x < 8) {
        const long tk = (long)blockIdx.x * 8 + threadIdx.x;
        rows_s[threadIdx.x] = (write_kv && tk < n) ? paged_row(pv, tok_slot[tk], positions[tk]) : -1;
    }
    const long t = (long)blockIdx.x * 8 + (lane >> 3);
    const int piece = lane & 7;
    const bool mine = t < n && piece < pieces;
    float cs[8], sn[8];
    if (mine) {
        const int pos = positions[t];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            cs[e] = 1.f;
            sn[e] = 0.f;
            if (inv_freq) {
                const float ang = (float)pos * inv_freq[8 * piece + e];
                cs[e] = cosf(ang) * mscale;
                sn[e] = sinf(ang) * mscale;
            }
        }
    }
    __syncthreads();
    if (mine) {
        const long kv_row = rows_s[lane >> 3];
        const int heads = nh + (write_kv ? nkv : 0);
        const bf16_t* row = qkv + t * width + 8 * piece;
        // UH heads' loads in flight at a time (a head beyond the last asks for the last once more)
        constexpr int UH = 5;
        for (int head0 = wave; head0 < heads; head0 += 4 * UH) {
            ebf16x8_t a[UH], b[UH];
#pragma unroll
            for (int u = 0; u < UH; ++u) {
                const int head = min(head0 + 4 * u, heads - 1);
                a[u] = *(const ebf16x8_t*)(row + (long)head * hd);
                b[u] = *(const ebf16x8_t*)(row + (long)head * hd + half);
            }
#pragma unroll
            for (int u = 0; u < UH; ++u) {
                const int head = head0 + 4 * u;
                if (head >= heads) break;
                ebf16x8_t lo, hi;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float x = (float)a[u][e], y = (float)b[u][e];
                    lo[e] = (__bf16)(x * cs[e] - y * sn[e]);
                    hi[e] = (__bf16)(x * sn[e] + y * cs[e]);
                }
                if (head < nh) {
                    bf16_t* dst = q_out + (t * nh + head) * (long)hd + 8 * piece;
                    *(ebf16x8_t*)dst = lo;
                    *(ebf16x8_t*)(dst + half) = hi;
                } else {
                    // d = 8 piece + e lies at key_d_offset = piece * 128 + e: one 16-byte piece
                    bf16_t* dst = kpool + key_index(kv_row, head - nh, nkv, hd);
                    *(ebf16x8_t*)(dst + piece * 128) = lo;
                    *(ebf16x8_t*)(dst + (piece + pieces) * 128) = hi;
                }
            }
        }
    }
    if (!write_kv) return;
    // values: thread (kv head, d), the block's 8 tokens one after the other
    for (int e = threadIdx.x; e < nkv * hd; e += 256) {
        const int kvh = e / hd, d = e - kvh * hd;
        bf16_t v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const long tk = min((long)blockIdx.x * 8 + k, (long)n - 1);
            v[k] = qkv[tk * width + (long)(nh + nkv + kvh) * hd + d];
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
            if (rows_s[k] >= 0) vpool[value_index(rows_s[k], kvh, nkv, hd) + value_d_offset(d)] = v[k];
    }
}

extern "C" const char* cpmcu_rope_store(const void* qkv, long row_width, int in_dtype, int nparts, long part_stride, void* q_out,
                                        int dtype, int n, int nh, int nkv, int hd, const int* positions,
                                        const int* tok_slot, const float* inv_freq, float mscale, void* kpool,
                                        void* vpool, const int* page_table, int table_width, int page_size,
                                        int write_kv, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && nh > 0 && nkv >= 0 && hd > 0 && hd % 2 == 0,
                  "rope_store: bad shape n=%d heads=%d kv_heads=%d head_dim=%d (head_dim must be even)", n, nh, nkv, hd);
    CPMCU_REQUIRE(!write_kv || (kpool && vpool && page_table && table_width > 0 && page_size > 0),
                  "rope_store: cache pointers missing");
    CPMCU_REQUIRE(!write_kv || (page_size % 32 == 0 && hd % 16 == 0),
                  "rope_store: the cache takes pages of a multiple of 32 tokens and head sizes in steps of 16 "
                  "(page %d, head_dim %d)", page_size, hd);
    CPMCU_REQUIRE(nparts >= 1, "rope_store: nparts=%d", nparts);
    CPMCU_REQUIRE(row_width >= (long)(nh + (write_kv ? 2 * nkv : 0)) * hd,
                  "rope_store: a row of %ld elements cannot hold %d query%s heads of %d", row_width, nh,
                  write_kv ? " and key/value" : "", hd);
    PagedView pv{page_table, table_width, page_size};
    if (n >= 64 && in_dtype == CPMCU_BF16 && dtype == CPMCU_BF16 && nparts == 1 && hd % 16 == 0 && hd <= 128 &&
        row_width % 8 == 0 && ((uintptr_t)qkv % 16 == 0) && ((uintptr_t)q_out % 16 == 0)) {
        rope_store_rows_kernel<<<(n + 7) / 8, 256, 0, stream>>>((const bf16_t*)qkv, row_width, (bf16_t*)q_out, n, nh, nkv,
                                                                hd, positions, tok_slot, inv_freq, mscale,
                                                                (bf16_t*)kpool, (bf16_t*)vpool, pv, write_kv);
        CPMCU_LAUNCH_CHECK("rope_store_rows");
        return nullptr;
    }
    // few tokens (decode steps): a block a head, for more blocks; many: 4 heads a block
    const int heads = nh + (write_kv ? 2 * nkv : 0);
    const int block = n >= 64 ? 256 : 64;
    CPMCU_REQUIRE(heads <= 65535, "rope_store: %d heads exceed the launch grid", heads);
    dim3 grid(n, n >= 64 ? (heads + 3) / 4 : heads);
#define LAUNCH(IT, T)                                                                                          \
    rope_store_kernel<IT, T><<<grid, block, 0, stream>>>((const IT*)qkv, row_width, nparts, part_stride, (T*)q_out, nh, nkv, \
                                                      hd, positions, tok_slot, inv_freq, mscale, (T*)kpool,   \
                                                      (T*)vpool, pv, write_kv)
    if (in_dtype == CPMCU_F32 && dtype == CPMCU_F32) LAUNCH(float, float);
    else if (in_dtype == CPMCU_F32 && dtype == CPMCU_BF16) LAUNCH(float, bf16_t);
    else if (in_dtype == CPMCU_BF16 && dtype == CPMCU_BF16) LAUNCH(bf16_t, bf16_t);
    else CPMCU_FAIL("rope_store: unsupported dtypes in=%d out=%d", in_dtype, dtype);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("rope_store");
    return nullptr;
}

// ---------------------------------------------------------------------------
// A plain read of `bytes` of memory, for measuring what the memory system delivers to a kernel that does
// nothing else (the ceiling that the decode step's products are measured against).  Every workgroup streams
// one contiguous region, as a product's workgroup streams its strip of the weight, 16 bytes a thread and
// eight loads in flight: on the MI355X that reaches 6.9-7.0 TB/s, where threads that stride over the whole
// buffer reach 6.4-6.6.  Each workgroup folds what it read into one word.
// ---------------------------------------------------------------------------
typedef unsigned read_u32x4_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void read_bandwidth_kernel(const read_u32x4_t* __restrict__ src, long n16,
                                                             unsigned* __restrict__ out) {
    const long per = (n16 + gridDim.x - 1) / gridDim.x;
    const long begin = per * blockIdx.x, end = min(begin + per, n16);
    read_u32x4_t acc = {0, 0, 0, 0};
    long i = begin + threadIdx.x;
    for (; i + 7 * 256 < end; i += 8 * 256) {
        read_u32x4_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i + u * 256);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u];
    }
    for (; i < end; i += 256) acc ^= __builtin_nontemporal_load(src + i);
    const unsigned r = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (r == 0x9e3779b9u || threadIdx.x == 0) out[blockIdx.x] = r;      // the fold must not be optimised away
}

extern "C" const char* cpmcu_read_bandwidth(const void* src, long bytes, unsigned* out, int n_out, hipStream_t stream) {
    CPMCU_REQUIRE(src && bytes >= 16 && out && n_out > 0, "read_bandwidth: needs memory to read and words to write");
    CPMCU_REQUIRE(((uintptr_t)src & 15) == 0, "read_bandwidth: the memory must be aligned to 16 bytes");
    const int grid = n_out < 4096 ? n_out : 4096;
    read_bandwidth_kernel<<<grid, 256, 0, stream>>>((const read_u32x4_t*)src, bytes / 16, out);
    CPMCU_LAUNCH_CHECK("read_bandwidth");
    return nullptr;
}
