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
            float b = 0.f;
            for (int p = 0; p < nparts; ++p) b += to_f32(branch[p * part_stride + r * H + c]);
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
            float b = 0.f;
            for (int p = 0; p < nparts; ++p) b += to_f32(branch[p * part_stride + r * H + c]);
            v += bscale * b;
        }
        o[c] = from_f32<OT>(v * rs * w[c]);
    }
}

// The same with 4 columns a thread and 16-byte accesses (H a multiple of 4, float branch or none):
// the decode steps' norms have few rows and up to 16 partial sums to add, so the row's work
// is spread over up to 1024 threads.
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
            float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
            for (int p = 0; p < nparts; ++p) {
                const float4 t = load4(branch + p * part_stride + r * H + 4 * c);
                b.x += t.x; b.y += t.y; b.z += t.z; b.w += t.w;
            }
            v.x += bscale * b.x; v.y += bscale * b.y; v.z += bscale * b.z; v.w += bscale * b.w;
        }
        return v;
    };
    auto emit = [&](int c, float4 v, float rs) {
        const float4 wv = *(const float4*)(w + 4 * c);
        o[4 * c + 0] = from_f32<OT>(v.x * rs * wv.x);
        o[4 * c + 1] = from_f32<OT>(v.y * rs * wv.y);
        o[4 * c + 2] = from_f32<OT>(v.z * rs * wv.z);
        o[4 * c + 3] = from_f32<OT>(v.w * rs * wv.w);
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
        ((uintptr_t)w % 16 == 0) && (out_dtype == CPMCU_F32 || out_dtype == CPMCU_BF16) &&
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

// bf16, I a multiple of 8: 8 columns a thread with 16-byte accesses
__global__ void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, long n, int I) {
    const int I8 = I / 8;
    const long total = n * I8;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
        const long r = i / I8;
        const int c = (int)(i - r * I8) * 8;
        const uint4 g4 = *(const uint4*)(gu + r * 2 * I + c);
        const uint4 u4 = *(const uint4*)(gu + r * 2 * I + I + c);
        const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
        uint32_t ow[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
            const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
            const bf16_t a = f32_to_bf16(g0 / (1.0f + expf(-g0)) * u0);
            const bf16_t b = f32_to_bf16(g1 / (1.0f + expf(-g1)) * u1);
            ow[j] = (uint32_t)a.v | ((uint32_t)b.v << 16);
        }
        *(uint4*)(out + r * I + c) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
    }
}

extern "C" const char* cpmcu_silu_mul(const void* gu, void* out, int dtype, int n, int I, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && I > 0, "silu_mul: empty shape n=%d I=%d", n, I);
    if (dtype == CPMCU_BF16 && I % 8 == 0 && (uintptr_t)gu % 16 == 0 && (uintptr_t)out % 16 == 0) {
        const long total8 = (long)n * (I / 8);
        const int grid8 = (int)((total8 + 255) / 256 < 65535 * 8 ? (total8 + 255) / 256 : 65535 * 8);
        silu_mul_bf16x8_kernel<<<grid8, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, n, I);
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
    // 64 threads per (token, head): heads [0, nh) are queries, then nkv key heads, then nkv value heads;
    // a block holds blockDim.x / 64 heads of one token
    const long t = blockIdx.x;
    const int head = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (head >= nh + (write_kv ? 2 * nkv : 0)) return;
    const int half = hd / 2;
    const int pos = positions[t];
    const IT* row = qkv + t * width + (long)head * hd;
    auto load = [&](int i) {
        float s = 0.f;
        for (int p = 0; p < nparts; ++p) s += to_f32(row[p * part_stride + i]);
        return s;
    };
    long kv_row = 0;
    if (head >= nh) kv_row = paged_row(pv, tok_slot[t], pos);
    if (head < nh + nkv) {
        // queries go out as plain rows; keys into their page in the matrix cores' order (key_index)
        const bool is_q = head < nh;
        T* dst = q_out;
        if (is_q) {
            dst = q_out + (t * nh + head) * (long)hd;
        } else {
            dst = kpool + key_index(kv_row, head - nh, nkv, hd);
        }
        auto at = [&](int d) { return is_q ? d : key_d_offset(d); };
        for (int c = lane; c < half; c += 64) {
            float cs = 1.f, sn = 0.f;
            if (inv_freq) {
                const float ang = (float)pos * inv_freq[c];
                cs = cosf(ang) * mscale;
                sn = sinf(ang) * mscale;
            }
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
    // few tokens (decode steps): a block a head, for more blocks; many: 4 heads a block
    const int heads = nh + (write_kv ? 2 * nkv : 0);
    const int hpb = n >= 64 ? 4 : 1;
    const int block = 64 * hpb;
    CPMCU_REQUIRE(heads <= 65535, "rope_store: %d heads exceed the launch grid", heads);
    dim3 grid(n, (heads + hpb - 1) / hpb);
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
