// Matrix products of the linear layers:  Y[m,N] = alpha * X[m,K] . W[N,K]^T
// with weights stored [out, in] row-major as in the checkpoint (reference:
// src/model/linear.cuh:9-37 calls a library product with fp32 accumulation).
//
//  * gemm_tiled_kernel: LDS-tiled product with scalar float FMAs, any element
//    type, any size.  It is the whole 32-bit engine's product (true fp32: no
//    matrix-core path with reduced inputs), and the plain twin of the bf16 ones.
#include "common.h"

#define GT_BM 64
#define GT_BN 64
#define GT_BK 16

template <typename XT, typename WT, typename OT>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const XT* __restrict__ X, long ldx,
                                                         const WT* __restrict__ W, long ldw, OT* __restrict__ Y,
                                                         long ldy, int M, int N, int K, float alpha) {
    __shared__ float xs[GT_BK][GT_BM + 1];
    __shared__ float ws[GT_BK][GT_BN + 1];
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const int m0 = blockIdx.y * GT_BM, n0 = blockIdx.x * GT_BN;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += GT_BK) {
        // 64 rows x 16 k of each operand: 1024 elements, 4 per thread
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = threadIdx.x + i * 256;
            const int r = e / GT_BK, kk = e % GT_BK;
            const int k = k0 + kk;
            xs[kk][r] = (m0 + r < M && k < K) ? to_f32(X[(long)(m0 + r) * ldx + k]) : 0.f;
            ws[kk][r] = (n0 + r < N && k < K) ? to_f32(W[(long)(n0 + r) * ldw + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GT_BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) Y[(long)m * ldy + n] = from_f32<OT>(alpha * acc[i][j]);
        }
    }
}

extern "C" const char* cpmcu_gemm_nt_plain(const void* X, long ldx, const void* W, long ldw, void* Y, long ldy,
                                           int in_dtype, int out_dtype, int M, int N, int K, float alpha,
                                           hipStream_t stream) {
    CPMCU_REQUIRE(M > 0 && N > 0 && K > 0, "gemm: empty shape M=%d N=%d K=%d", M, N, K);
    CPMCU_REQUIRE(ldx >= K && ldw >= K && ldy >= N, "gemm: leading dimensions %ld %ld %ld too small for K=%d N=%d",
                  ldx, ldw, ldy, K, N);
    dim3 grid((N + GT_BN - 1) / GT_BN, (M + GT_BM - 1) / GT_BM);
    CPMCU_REQUIRE(grid.y <= 65535, "gemm: M=%d too large for one launch", M);
#define LAUNCH(T, OT)                                                                                     \
    gemm_tiled_kernel<T, T, OT><<<grid, 256, 0, stream>>>((const T*)X, ldx, (const T*)W, ldw, (OT*)Y, ldy, \
                                                          M, N, K, alpha)
    if (in_dtype == CPMCU_F32 && out_dtype == CPMCU_F32) LAUNCH(float, float);
    else if (in_dtype == CPMCU_BF16 && out_dtype == CPMCU_BF16) LAUNCH(bf16_t, bf16_t);
    else if (in_dtype == CPMCU_BF16 && out_dtype == CPMCU_F32) LAUNCH(bf16_t, float);
    else CPMCU_FAIL("gemm: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("gemm_nt_plain");
    return nullptr;
}

// ===========================================================================
// Skinny product for decode steps (bf16, at most 64 rows of X):
//   Y[m,N] = alpha * X[m,K] . W[N,K]^T
// The step is bound by reading W once from HBM, so W streams from global memory
// straight into MFMA operand registers (v_mfma_f32_16x16x32_bf16: 16 rows of W
// by 32 of K an instruction), four K-blocks of 128 ahead of their use, while X
// (small, shared by all rows of W) is staged through LDS 512 columns at a time.
// For the i-th MFMA of a K-block of 128 the lane group g = lane/16 holds columns
// [32i + 8g, 32i + 8g + 8) of its row, so the four lanes of a row read 64
// contiguous bytes an instruction; X is read from LDS with the same mapping.
// TILED: W comes re-laid for this kernel (made once when the weights are bound):
// [strip of 16 rows][K-block of 128][MFMA i][lane][8 elements], rows and K padded with
// zeros, so every load instruction of a wavefront reads 1 KiB of consecutive memory and
// a wavefront streams one contiguous region.  Measured on the MI355X this lifts the large
// products from about 4.9 to 5.8-6.1 TB/s (a plain read kernel reaches 6.3).
//   MODE 0: Y (float or bf16) = alpha * product
//   MODE 1: float partial sums of a K-split, part[blockIdx.y][m][N]
//   MODE 2: rows come in pairs (gate j, up I+j): Y[m][j] = silu(gate) * up  (bf16)
// ===========================================================================
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

#define SK_XC 512            // K columns of X staged at a time
#define SK_XS (SK_XC + 8)    // LDS row stride in elements (16 bytes of padding)

template <int MT, int MODE, typename OT, int SPW, int NW, bool TILED>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ X, long ldx,
                                                             const bf16_t* __restrict__ W, long ldw,
                                                             OT* __restrict__ Y, long ldy, int M, int N, int K, int KS,
                                                             float alpha, int I, long part_stride,
                                                             const float* __restrict__ row_ss, int ss_slices,
                                                             float eps) {
    static_assert(MODE != 2 || SPW == 2, "gated output pairs a gate strip with an up strip");
    // whether the x operands are read from LDS a step ahead (below): it pays for 4 tiles of rows in the split and
    // plain products (64 rows, us without/with: q/k/v 17.0/14.3, down 31.0/28.9, head 134/130, o 11.7/12.0), not
    // for the gated product (53.8/55.3) and not for 2 tiles (q/k/v 12.5/11.4 but down 24.4/25.8)
    constexpr bool AHEAD = MT >= 4 && MODE != 2;
    constexpr int NT = NW * 64;
    constexpr int XV = MT * 16 * 64 / NT;     // 16-byte vectors of X a thread stages per chunk
    constexpr int BPW = 4;                    // K-blocks of a chunk
    __shared__ __attribute__((aligned(16))) bf16_t xs[MT * 16 * SK_XS];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int k_begin = blockIdx.y * KS;
    const int k_end = min(K, k_begin + KS);
    const int nkb = (k_end - k_begin + 127) / 128;

    // the strips of 16 rows of W this wave owns
    int out_base[SPW];
    const bf16_t* wp[SPW];
    const long nkb_total = (K + 127) / 128;       // K-blocks of a tiled row strip
    const int n_strips = (N + 15) / 16;
    if (MODE == 2) {
        const int p = blockIdx.x * (NW * 16) + wave * 16;
        out_base[0] = out_base[SPW - 1] = p;
        if (TILED) {                              // I is a multiple of 16: up strip = gate strip + I/16
            const long gs = min(p / 16, I / 16 - 1);
            wp[0] = W + gs * nkb_total * 2048 + lane * 8;
            wp[SPW - 1] = W + (gs + I / 16) * nkb_total * 2048 + lane * 8;
        } else {
            const int pr = min(p + r, I - 1);
            wp[0] = W + (long)pr * ldw;
            wp[SPW - 1] = W + ((long)I + pr) * ldw;
        }
    } else {
        const int n0 = blockIdx.x * (NW * SPW * 16) + wave * (SPW * 16);
#pragma unroll
        for (int s = 0; s < SPW; ++s) {
            out_base[s] = n0 + s * 16;
            if (TILED) wp[s] = W + (long)min(n0 / 16 + s, n_strips - 1) * nkb_total * 2048 + lane * 8;
            else wp[s] = W + (long)min(n0 + s * 16 + r, N - 1) * ldw;
        }
    }

    // In the main loop no load stands in a branch: the compiler waits for every load in flight where such a
    // branch ends, and the weights asked for a chunk ahead would have to be there before the chunk's x is stored
    // (that wait cost the 64-row products a trip to memory a chunk).  Only the slice's last chunks (`guard`) ask
    // whether a block or a column exists.
    bf16x8_t a[BPW][SPW][4];                  // a chunk's blocks of the wavefront's strips
    auto load_w = [&](int kb, bf16x8_t (&dst)[SPW][4], const bool guard) {
        if (guard && kb >= nkb) {             // uniform; the block is multiplied by zeros of x or not at all
#pragma unroll
            for (int s = 0; s < SPW; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i) dst[s][i] = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
            return;
        }
        const int k = k_begin + kb * 128 + g * 8;
#pragma unroll
        for (int s = 0; s < SPW; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (TILED)                    // one 128-block of a strip is 2048 elements: [i][lane][8]
                    dst[s][i] = __builtin_nontemporal_load((const bf16x8_t*)(wp[s] + ((long)(k_begin / 128 + kb) * 4 + i) * 512));
                else                          // columns beyond K repeat the row's last 8 and meet zeros of x
                    dst[s][i] = __builtin_nontemporal_load((const bf16x8_t*)(wp[s] + min(k + i * 32, K - 8)));
            }
    };
    // rows beyond the step repeat its last row (their results are not written); columns beyond the slice are
    // read from the row's end and replaced by zeros when the chunk is stored
    bf16x8_t xr[XV];
    auto load_x = [&](int chunk) {
        const int k0 = k_begin + chunk * SK_XC;
#pragma unroll
        for (int v = 0; v < XV; ++v) {
            const int idx = tid + v * NT;
            const int xrow = idx >> 6, vec = idx & 63;
            xr[v] = *(const bf16x8_t*)(X + (long)min(xrow, M - 1) * ldx + min(k0 + vec * 8, K - 8));
        }
    };
    auto store_x = [&](int chunk, const bool guard) {
        const int k0 = k_begin + chunk * SK_XC;
#pragma unroll
        for (int v = 0; v < XV; ++v) {
            const int idx = tid + v * NT;
            const int xrow = idx >> 6, vec = idx & 63;
            const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
            *(bf16x8_t*)(xs + xrow * SK_XS + vec * 8) = (!guard || k0 + vec * 8 < k_end) ? xr[v] : zero;
        }
    };

    floatx4_t acc[SPW][MT];
#pragma unroll
    for (int s = 0; s < SPW; ++s)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[s][t] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    // x first: loads return in the order of their issue, and the loop's first store of x must not wait for more
    // weights than its later ones do (the compiler takes the stricter of the two for all)
    load_x(0);
#pragma unroll
    for (int jj = 0; jj < BPW; ++jj) load_w(min(jj, nkb - 1), a[jj], false);   // beyond a short slice: its last block again
    // X may be x * w of a norm whose row factor is still to come (common.h: row_scales); the loop's first
    // barrier makes rs_s visible
    __shared__ float rs_s[MT * 16];
    if (row_ss) row_scales<NT, MT * 16>(row_ss, ss_slices, M, 1.0f / (float)K, eps, rs_s);
    const int nchunk = (nkb + 3) / 4, nfull = nkb / 4;       // chunks in all, chunks of 4 whole blocks
    // a block's weights are asked for again, a chunk ahead, as soon as the block is multiplied
    auto one_chunk = [&](int c, bf16x8_t (&ap)[BPW][SPW][4], const bool guard) {
        __syncthreads();
        store_x(c, guard);
        __syncthreads();
        if (!guard || c + 1 < nchunk) load_x(c + 1);
        if (!AHEAD) {
#pragma unroll
            for (int jj = 0; jj < BPW; ++jj) {
                const int j = jj;
                // consecutive matrix instructions go to different accumulators (tiles of rows, then strips)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
#pragma unroll
                    for (int t = 0; t < MT; ++t) {
                        const bf16x8_t b = *(const bf16x8_t*)(xs + (t * 16 + r) * SK_XS + j * 128 + g * 8 + i * 32);
#pragma unroll
                        for (int s = 0; s < SPW; ++s)
                            acc[s][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ap[jj][s][i], b, acc[s][t], 0, 0, 0);
                    }
                }
                load_w((c + 1) * 4 + j, ap[jj], guard);
            }
            return;
        }
        // the x operands of a step (32 columns) are read from LDS a step ahead of the matrix instructions that use
        // them; with one or two wavefronts a SIMD nothing else hides that latency
        auto read_b = [&](int jj, int i, bf16x8_t (&b)[MT]) {
            const int j = jj;
#pragma unroll
            for (int t = 0; t < MT; ++t) b[t] = *(const bf16x8_t*)(xs + (t * 16 + r) * SK_XS + j * 128 + g * 8 + i * 32);
        };
        bf16x8_t bq[2][MT];
        read_b(0, 0, bq[0]);
#pragma unroll
        for (int jj = 0; jj < BPW; ++jj) {
            const int j = jj;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int step = jj * 4 + i;
                if (step + 1 < BPW * 4) read_b((step + 1) / 4, (step + 1) % 4, bq[(step + 1) & 1]);
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int s = 0; s < SPW; ++s)
                        acc[s][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ap[jj][s][i], bq[step & 1][t], acc[s][t], 0, 0, 0);
            }
            load_w((c + 1) * 4 + j, ap[jj], guard);
        }
        if (!guard) {
            // the order the scheduler is to keep: x of the next chunk asked for, then step by step the next
            // step's operands read from LDS before this step's matrix instructions, a block's weights asked for
            // again when its last step is through (left alone, the scheduler reads each operand just before its
            // use to save registers)
            __builtin_amdgcn_sched_group_barrier(0x020, XV, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);
#pragma unroll
            for (int step = 0; step < BPW * 4; ++step) {
                if (step + 1 < BPW * 4) __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, MT * SPW, 0);
                if (step % 4 == 3) __builtin_amdgcn_sched_group_barrier(0x020, SPW * 4, 0);
            }
        }
    };
    int c0 = 0;
    for (; c0 + 2 <= nfull; ++c0) one_chunk(c0, a, false);   // this chunk, the next x and the blocks asked for are whole
    for (; c0 < nchunk; ++c0) one_chunk(c0, a, true);        // the slice's end
    // lane (r, g) of tile t holds token t*16 + r, rows 4g .. 4g+3 of each strip
    OT* Yp = Y + (MODE == 1 ? (long)blockIdx.y * part_stride : 0);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int tok = t * 16 + r;
        if (tok >= M) continue;
        const float rs_t = row_ss ? rs_s[tok] : 1.0f;
        if (MODE == 2) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int col = out_base[0] + 4 * g + i;
                if (col < I) {
                    const float gt = acc[0][t][i] * rs_t, up = acc[SPW - 1][t][i] * rs_t;
                    Yp[(long)tok * ldy + col] = from_f32<OT>(gt / (1.0f + expf(-gt)) * up);
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < SPW; ++s)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int col = out_base[s] + 4 * g + i;
                    if (col < N) Yp[(long)tok * ldy + col] = from_f32<OT>(alpha * rs_t * acc[s][t][i]);
                }
        }
    }
}

// out_mode: 0 = Y[m,N] in out_dtype; 1 = float partial sums Y[ksplit][m][N]; 2 = gated (N = 2*I rows of W, Y[m,I] bf16)
// row_ss (or null): X is x * w of a norm cut by columns, whose sums of squares [M][ss_slices] these are (a
// slice for every 64 columns after add_norm_columns, for every 16 after proj_add_norm); the output is multiplied
// by rsqrt(sum of the row's slices / K + eps) row by row.
// Workgroups that measured best on the MI355X: 4 wavefronts of one strip each (more, smaller workgroups balance
// better over 256 CUs); for the gated output 2 wavefronts of a gate and an up strip each at every number of rows
// (32,768 x 4,096, us with 4 wavefronts / 2 / two groups of 4 that share the staged x: 17 rows 50.9/46.5/52.9,
// 32 rows 49.5/46.1/52.2, 64 rows 51.9/49.5/52.8).
extern "C" const char* cpmcu_gemm_skinny(const void* X, long ldx, const void* W, long ldw, void* Y, long ldy,
                                         int out_dtype, int out_mode, int M, int N, int K, int ksplit, float alpha,
                                         int tiled, const float* row_ss, int ss_slices, float eps, hipStream_t stream) {
    CPMCU_REQUIRE(M > 0 && M <= 64, "gemm_skinny: %d rows (1..64 are taken; more rows belong to the tiled product)", M);
    CPMCU_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "gemm_skinny: K=%d must be a positive multiple of 8 (N=%d)", K, N);
    CPMCU_REQUIRE(ldx % 8 == 0 && ldx >= K && (tiled || (ldw % 8 == 0 && ldw >= K)),
                  "gemm_skinny: leading dimensions %ld %ld must be multiples of 8 and >= K", ldx, ldw);
    CPMCU_REQUIRE(!tiled || out_mode != 2 || (N / 2) % 16 == 0,
                  "gemm_skinny: gated output from tiled weights needs a multiple of 16 gate rows, got %d", N / 2);
    CPMCU_REQUIRE(((uintptr_t)X % 16 == 0) && ((uintptr_t)W % 16 == 0), "gemm_skinny: operands must be 16-byte aligned");
    CPMCU_REQUIRE(ksplit >= 1 && (out_mode == 1 || ksplit == 1), "gemm_skinny: a K-split (%d) needs partial-sum output", ksplit);
    CPMCU_REQUIRE(out_mode != 2 || N % 2 == 0, "gemm_skinny: gated output needs an even number of rows, got %d", N);
    int KS = (K + ksplit - 1) / ksplit;
    KS = (KS + 127) / 128 * 128;
    const int splits = (K + KS - 1) / KS;
    CPMCU_REQUIRE(splits == ksplit, "gemm_skinny: K=%d cannot be cut into %d slices of whole 128-blocks (would be %d)", K, ksplit, splits);
    const int MT = (M + 15) / 16 == 3 ? 4 : (M + 15) / 16;
    const int I = N / 2;
    const long part_stride = (long)M * ldy;
#define LAUNCH(MTv, MODEv, OT, SPW, NW)                                                                           \
    do {                                                                                                          \
        const int rows_wg = (MODEv == 2) ? NW * 16 : NW * SPW * 16;                                               \
        dim3 grid(((MODEv == 2 ? I : N) + rows_wg - 1) / rows_wg, ksplit);                                        \
        if (tiled)                                                                                                \
            gemm_skinny_kernel<MTv, MODEv, OT, SPW, NW, true><<<grid, NW * 64, 0, stream>>>(                      \
                (const bf16_t*)X, ldx, (const bf16_t*)W, ldw, (OT*)Y, ldy, M, N, K, KS, alpha, I, part_stride,    \
                row_ss, ss_slices, eps);                                                                          \
        else                                                                                                      \
            gemm_skinny_kernel<MTv, MODEv, OT, SPW, NW, false><<<grid, NW * 64, 0, stream>>>(                     \
                (const bf16_t*)X, ldx, (const bf16_t*)W, ldw, (OT*)Y, ldy, M, N, K, KS, alpha, I, part_stride,    \
                row_ss, ss_slices, eps);                                                                          \
    } while (0)
#define BY_MT(MODEv, OT, SPW, NW)                     \
    do {                                              \
        if (MT == 1) LAUNCH(1, MODEv, OT, SPW, NW);   \
        else if (MT == 2) LAUNCH(2, MODEv, OT, SPW, NW); \
        else LAUNCH(4, MODEv, OT, SPW, NW);           \
    } while (0)
    if (out_mode == 0 && out_dtype == CPMCU_F32) BY_MT(0, float, 1, 4);
    else if (out_mode == 0 && out_dtype == CPMCU_BF16) BY_MT(0, bf16_t, 1, 4);
    else if (out_mode == 1) BY_MT(1, float, 1, 4);
    else if (out_mode == 2) BY_MT(2, bf16_t, 2, 2);
    else CPMCU_FAIL("gemm_skinny: unknown output mode %d / dtype %d", out_mode, out_dtype);
#undef BY_MT
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("gemm_skinny");
    return nullptr;
}
