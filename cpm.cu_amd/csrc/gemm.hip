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
