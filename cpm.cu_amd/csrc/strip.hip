// Products of decode steps by strips of output columns (bf16).
//
// First: a branch's last product fused with the residual add and the column part of the norm that follows it
// (at most 64 tokens):
//     x += alpha * (a . W^T);   out = bf16(x * w_norm);   row_ss[row][strip] = sum of x^2 over the strip
// A decode step is a chain of small kernels, each of which costs a few microseconds whatever it does.  The
// split-K product leaves partial sums that a second kernel (elementwise.hip: add_norm_columns) adds into the
// residual stream; here one workgroup owns a strip of 16 output columns over the whole of K, so it holds the
// finished sums and does that kernel's work for its columns itself: one kernel of the chain less.  The norm's
// row factor rsqrt(sum / width + eps) is left to the product that reads `out`, as after add_norm_columns, with
// slices of 16 columns instead of 64.
//
// The weight is tiled as for the skinny product ([strip of 16 rows][128-column block][i][lane][8],
// ops.TiledWeight).  The NW wavefronts of a workgroup take a contiguous share of the K blocks each (a straight
// from global memory into the B operand, asked for together with the weight's block), add their results
// through LDS, and the first wavefront finishes.
//
// (reference: the output projections src/model/minicpm4/minicpm4_attn.cuh:205, 319 and src/model/ffn.cuh:77-84
// followed by add + norm src/model/norm.cuh:53-99)
#include "common.h"

typedef __bf16 pbf16x8_t __attribute__((ext_vector_type(8)));
typedef float pfloatx4_t __attribute__((ext_vector_type(4)));

// PF: 128-column blocks of the weight a wavefront keeps in flight; NW: wavefronts a workgroup; MT: tiles of 16 tokens
template <int PF, int NW, int MT>
__global__ __launch_bounds__(NW * 64) void proj_add_norm_kernel(
    const bf16_t* __restrict__ A, long lda, const bf16_t* __restrict__ W, int M, int N, int K, float alpha,
    float* __restrict__ x, const float* __restrict__ w_norm, bf16_t* __restrict__ out, float* __restrict__ row_ss,
    int n_strips) {
    __shared__ float red[NW - 1][MT][4][64];
    const int strip = blockIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int nkb = (K + 127) / 128;
    const int per_wave = (nkb + NW - 1) / NW;
    const int kb0 = wave * per_wave, kb1 = min(kb0 + per_wave, nkb);
    const bf16_t* wp = W + (long)strip * nkb * 2048 + lane * 8;
    const bf16_t* ap[MT];                                  // rows beyond the step repeat its last token
#pragma unroll
    for (int t = 0; t < MT; ++t) ap[t] = A + (long)min(t * 16 + r, M - 1) * lda;

    // Loads return in the order of their issue, so the a of a block is asked for together with its w, PF blocks
    // ahead.  No load stands in a branch that depends on data: addresses are clamped instead (a block beyond
    // the wavefront's last repeats the matrix's last and is not multiplied; columns beyond K repeat the row's
    // last 8 and meet the weight's zero padding), so the waits count exactly.
    pbf16x8_t wv[PF][4], av[PF][MT][4];
    auto load_block = [&](int kb, pbf16x8_t (&wd)[4], pbf16x8_t (&ad)[MT][4]) {
        const int kbc = min(kb, nkb - 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) wd[i] = __builtin_nontemporal_load((const pbf16x8_t*)(wp + ((long)kbc * 4 + i) * 512));
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) ad[t][i] = *(const pbf16x8_t*)(ap[t] + min(kbc * 128 + i * 32 + g * 8, K - 8));
    };
    pfloatx4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = pfloatx4_t{0.f, 0.f, 0.f, 0.f};
    // what the end needs (the residual's 4 columns of this lane's tokens, the norm's weights) is asked for
    // first: it is there when the products are, instead of costing a trip to memory after them
    const int col = strip * 16 + 4 * g;
    const bool col_ok = col < N;                                  // N is a multiple of 4
    const float4 wn = *(const float4*)(w_norm + min(col, N - 4));
    float4 xin[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) xin[t] = *(const float4*)(x + (long)min(t * 16 + r, M - 1) * N + min(col, N - 4));
    auto multiply = [&](pbf16x8_t (&wd)[4], pbf16x8_t (&ad)[MT][4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int t = 0; t < MT; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wd[i], ad[t][i], acc[t], 0, 0, 0);
    };
#pragma unroll
    for (int j = 0; j < PF; ++j) load_block(kb0 + j, wv[j], av[j]);
    int kb = kb0;
    for (; kb + 2 * PF <= kb1; kb += PF) {           // every block and every block asked for exists
#pragma unroll
        for (int j = 0; j < PF; ++j) {
            multiply(wv[j], av[j]);
            load_block(kb + j + PF, wv[j], av[j]);
        }
    }
    for (; kb < kb1; kb += PF) {                      // the last blocks: nothing more, or only what exists, is asked for
#pragma unroll
        for (int j = 0; j < PF; ++j) {
            if (kb + j < kb1) multiply(wv[j], av[j]);
            if (kb + j + PF < kb1) load_block(kb + j + PF, wv[j], av[j]);
        }
    }
    // lane (token r, g) of tile t: acc[t][i] is column 16 * strip + 4g + i; the other wavefronts hand theirs
    // to the first, which adds them in the order of the wavefronts
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave - 1][t][i][lane] = acc[t][i];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int w = 0; w < NW - 1; ++w) acc[t][i] += red[w][t][i][lane];
        const int tok = t * 16 + r;
        const bool ok = tok < M && col_ok;
        const long off = (long)min(tok, M - 1) * N + min(col, N - 4);
        float4 v = xin[t];
        v.x += alpha * acc[t][0]; v.y += alpha * acc[t][1]; v.z += alpha * acc[t][2]; v.w += alpha * acc[t][3];
        float ss = 0.f;
        if (ok) {
            *(float4*)(x + off) = v;
            const bf16_t o0 = f32_to_bf16(v.x * wn.x), o1 = f32_to_bf16(v.y * wn.y);
            const bf16_t o2 = f32_to_bf16(v.z * wn.z), o3 = f32_to_bf16(v.w * wn.w);
            *(uint2*)(out + off) = make_uint2((uint32_t)o0.v | ((uint32_t)o1.v << 16), (uint32_t)o2.v | ((uint32_t)o3.v << 16));
            ss = v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
        ss = rows_sum(ss);                                        // the four lanes (r, g = 0..3) of a token
        if (g == 0 && tok < M) row_ss[(long)tok * n_strips + strip] = ss;
    }
}

// x [M, N] float32 (in place), a [M, K] bf16, W tiled [N, K], w_norm [N] float32, out [M, N] bf16,
// row_ss [M, ceil(N / 16)] float32.  N must be a multiple of 4, K of 8; at most 64 rows.
extern "C" const char* cpmcu_proj_add_norm(const void* A, long lda, const void* W, int M, int N, int K, float alpha,
                                           float* x, const float* w_norm, void* out, float* row_ss, hipStream_t stream) {
    CPMCU_REQUIRE(M > 0 && M <= 64, "proj_add_norm: %d tokens (1..64 are taken; more go through the split product and the norm kernel)", M);
    CPMCU_REQUIRE(N > 0 && N % 4 == 0 && K > 0 && K % 8 == 0 && lda % 8 == 0 && lda >= K,
                  "proj_add_norm: N=%d must be a multiple of 4, K=%d and the row stride %ld multiples of 8", N, K, lda);
    CPMCU_REQUIRE(A && W && x && w_norm && out && row_ss, "proj_add_norm: null pointer");
    CPMCU_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0) && ((uintptr_t)x % 16 == 0) &&
                  ((uintptr_t)w_norm % 16 == 0) && ((uintptr_t)out % 8 == 0), "proj_add_norm: operands must be 16-byte aligned");
    const int strips = (N + 15) / 16;
#define LAUNCH(PFv, NWv, MTv)                                                                                   \
    proj_add_norm_kernel<PFv, NWv, MTv><<<strips, NWv * 64, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, M, N, \
                                                                        K, alpha, x, w_norm, (bf16_t*)out, row_ss, strips)
    // 4 blocks in flight in each of 4 wavefronts measured best at K = 4,096 (8 wavefronts: the same; 8 blocks:
    // slower; 16 wavefronts of 4 blocks spill)
    // (more tokens hold more of a in registers for every block in flight: fewer blocks then)
    // long rows (down: K = 16,384) in 8 wavefronts of 2 blocks in flight: 24.3 against 25.1 us at 8 tokens, 27.4
    // against 29.6 at 16; at K = 4,096 the two are level
    if (M <= 16 && K >= 8192) LAUNCH(2, 8, 1);
    else if (M <= 16) LAUNCH(4, 4, 1);
    else if (M <= 32) LAUNCH(4, 4, 2);
    else LAUNCH(2, 4, 4);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("proj_add_norm");
    return nullptr;
}

// ===========================================================================
// silu(a . Wg^T) * (a . Wu^T) for decode steps of at most 16 tokens, by strips: a workgroup owns a strip of 16
// gate rows and the strip of their up rows over all of K (W holds the gate rows, then the up rows; I gate rows,
// a multiple of 16).  Its wavefronts take a quarter of K each, with a straight from global memory into the B
// operand as above, add up through LDS, and the first one applies the norm's row factor (if a is the x * w of a
// norm cut by columns), the gate's nonlinearity and writes 16 columns.  1,024 small workgroups at 16,384 gate
// rows keep more loads in flight than the skinny product's 512 (gemm.hip), which stages a through LDS behind
// barriers: 43.4 against 45.8 us at 8 tokens and 4,096 columns (6.2 TB/s of weights).
// (reference: src/model/ffn.cuh:31-59, 77-84; src/model/activation.cuh:6-18)
// ===========================================================================
template <int PF, int NW, int MT>
__global__ __launch_bounds__(NW * 64) void gated_strip_kernel(
    const bf16_t* __restrict__ A, long lda, const bf16_t* __restrict__ W, int M, int I, int K,
    bf16_t* __restrict__ out, const float* __restrict__ row_ss, int ss_slices, float eps) {
    __shared__ float red[NW - 1][2][MT][4][64];
    __shared__ float rs_s[MT * 16];
    const int strip = blockIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int nkb = (K + 127) / 128;
    const int per_wave = (nkb + NW - 1) / NW;
    const int kb0 = wave * per_wave, kb1 = min(kb0 + per_wave, nkb);
    const bf16_t* wp[2];
    wp[0] = W + (long)strip * nkb * 2048 + lane * 8;
    wp[1] = W + (long)(strip + I / 16) * nkb * 2048 + lane * 8;
    const bf16_t* ap[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) ap[t] = A + (long)min(t * 16 + r, M - 1) * lda;
    pbf16x8_t wv[PF][2][4], av[PF][MT][4];
    auto load_block = [&](int kb, pbf16x8_t (&wd)[2][4], pbf16x8_t (&ad)[MT][4]) {
        const int kbc = min(kb, nkb - 1);
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i) wd[s][i] = __builtin_nontemporal_load((const pbf16x8_t*)(wp[s] + ((long)kbc * 4 + i) * 512));
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) ad[t][i] = *(const pbf16x8_t*)(ap[t] + min(kbc * 128 + i * 32 + g * 8, K - 8));
    };
    pfloatx4_t acc[2][MT];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[s][t] = pfloatx4_t{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](pbf16x8_t (&wd)[2][4], pbf16x8_t (&ad)[MT][4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int s = 0; s < 2; ++s) acc[s][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wd[s][i], ad[t][i], acc[s][t], 0, 0, 0);
    };
#pragma unroll
    for (int j = 0; j < PF; ++j) load_block(kb0 + j, wv[j], av[j]);
    if (row_ss) row_scales<NW * 64, MT * 16>(row_ss, ss_slices, M, 1.0f / (float)K, eps, rs_s);
    int kb = kb0;
    for (; kb + 2 * PF <= kb1; kb += PF) {
#pragma unroll
        for (int j = 0; j < PF; ++j) {
            multiply(wv[j], av[j]);
            load_block(kb + j + PF, wv[j], av[j]);
        }
    }
    for (; kb < kb1; kb += PF) {
#pragma unroll
        for (int j = 0; j < PF; ++j) {
            if (kb + j < kb1) multiply(wv[j], av[j]);
            if (kb + j + PF < kb1) load_block(kb + j + PF, wv[j], av[j]);
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) red[wave - 1][s][t][i][lane] = acc[s][t][i];
    }
    __syncthreads();
    if (wave > 0) return;
    const int col = strip * 16 + 4 * g;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int tok = t * 16 + r;
        const float rs = row_ss ? rs_s[tok] : 1.0f;
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float gt = acc[0][t][i], up = acc[1][t][i];
#pragma unroll
            for (int w = 0; w < NW - 1; ++w) {
                gt += red[w][0][t][i][lane];
                up += red[w][1][t][i][lane];
            }
            gt *= rs; up *= rs;
            o[i] = f32_to_bf16(gt / (1.0f + expf(-gt)) * up).v;
        }
        if (tok < M && col < I) *(uint2*)(out + (long)tok * I + col) = make_uint2(o[0] | (o[1] << 16), o[2] | (o[3] << 16));
    }
}

// a [M, K] bf16, W tiled [2 I, K], out [M, I] bf16; row_ss (or null): sums of squares [M][ss_slices] of a norm
// cut by columns, whose row factor rsqrt(sum / K + eps) the rows of both products are multiplied by
extern "C" const char* cpmcu_gated_strip(const void* A, long lda, const void* W, int M, int I, int K, void* out,
                                         const float* row_ss, int ss_slices, float eps, hipStream_t stream) {
    CPMCU_REQUIRE(M > 0 && M <= 16, "gated_strip: %d tokens (1..16 are taken; more go through the skinny product)", M);
    CPMCU_REQUIRE(I > 0 && I % 16 == 0 && K > 0 && K % 8 == 0 && lda % 8 == 0 && lda >= K,
                  "gated_strip: %d gate rows must be a multiple of 16, K=%d and the row stride %ld multiples of 8", I, K, lda);
    CPMCU_REQUIRE(A && W && out && (!row_ss || ss_slices > 0), "gated_strip: null pointer");
    CPMCU_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0) && ((uintptr_t)out % 8 == 0),
                  "gated_strip: operands must be 16-byte aligned");
    gated_strip_kernel<4, 4, 1><<<I / 16, 256, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, M, I, K, (bf16_t*)out,
                                                           row_ss, ss_slices, eps);
    CPMCU_LAUNCH_CHECK("gated_strip");
    return nullptr;
}
