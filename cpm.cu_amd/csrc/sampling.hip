// Next-token choice from float logits: argmax, and a draw from
// softmax(logits / temperature).
//
// The reference samples with library calls on one row: argmax, or
// multinomial(softmax(logits/temperature)) (cpmcu/llm.py:282-285).  Here a
// row's random number comes from a counter-based generator keyed by
// (seed, request id, step), so what a request draws does not depend on which
// other requests share its batch.
#include "common.h"

// ties go to the lowest index
__device__ inline void argmax_take(float v, int i, float& best, int& idx) {
    if (v > best || (v == best && i < idx)) {
        best = v;
        idx = i;
    }
}
// VEC: rows are 16-byte aligned and V is a multiple of 4: four logits a load, four loads in flight
template <bool VEC>
__global__ void argmax_kernel(const float* __restrict__ logits, long ld, int V, int* __restrict__ out) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    const float* row = logits + (long)blockIdx.x * ld;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    if (VEC) {
        const int V4 = V / 4, step = blockDim.x;
        int i = threadIdx.x;
        for (; i + 3 * step < V4; i += 4 * step) {
            float4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = *(const float4*)(row + 4 * (i + u * step));
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = 4 * (i + u * step);
                argmax_take(v[u].x, c, best, idx);
                argmax_take(v[u].y, c + 1, best, idx);
                argmax_take(v[u].z, c + 2, best, idx);
                argmax_take(v[u].w, c + 3, best, idx);
            }
        }
        for (; i < V4; i += step) {
            const float4 v = *(const float4*)(row + 4 * i);
            argmax_take(v.x, 4 * i, best, idx);
            argmax_take(v.y, 4 * i + 1, best, idx);
            argmax_take(v.z, 4 * i + 2, best, idx);
            argmax_take(v.w, 4 * i + 3, best, idx);
        }
    } else {
        for (int i = threadIdx.x; i < V; i += blockDim.x) argmax_take(row[i], i, best, idx);
    }
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(idx, o, 64);
        argmax_take(ov, oi, best, idx);
    }
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    if (lane == 0) { bv[w] = best; bi[w] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < nw; ++i) argmax_take(bv[i], bi[i], best, idx);
        out[blockIdx.x] = idx == 0x7fffffff ? 0 : idx;
    }
}

extern "C" const char* cpmcu_argmax(const float* logits, long ld, int rows, int V, int* out, hipStream_t stream) {
    CPMCU_REQUIRE(rows > 0 && V > 0 && ld >= V, "argmax: bad shape rows=%d V=%d ld=%ld", rows, V, ld);
    const int block = V >= 4096 ? 1024 : 256;
    if (V % 4 == 0 && ld % 4 == 0 && ((uintptr_t)logits % 16 == 0))
        argmax_kernel<true><<<rows, block, 0, stream>>>(logits, ld, V, out);
    else
        argmax_kernel<false><<<rows, block, 0, stream>>>(logits, ld, V, out);
    CPMCU_LAUNCH_CHECK("argmax");
    return nullptr;
}

// Philox-4x32-10: counter (c0..c3), key (k0,k1) -> 4 random words
__device__ inline void philox4x32(uint32_t c[4], uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0;
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
        const uint32_t n3 = (uint32_t)p0;
        c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
}

// One block per row.  Thread i owns the vocabulary entries i, i + T, i + 2T, ... (T threads: neighbouring
// threads read neighbouring logits).  The cumulative distribution runs over the entries in the order (thread 0's,
// thread 1's, ...): any fixed order of the vocabulary gives a draw from the same distribution, and this one
// depends on the row alone.  The thread whose range of the cumulative sum holds u * total walks its entries.
__global__ __launch_bounds__(1024) void sample_kernel(const float* __restrict__ logits, long ld, int V,
                                                     float inv_temperature, uint32_t seed_lo, uint32_t seed_hi,
                                                     const int* __restrict__ request_ids, const int* __restrict__ steps,
                                                     int* __restrict__ out, float* __restrict__ u_out) {
    __shared__ float red[17];
    __shared__ float wave_incl[16];
    __shared__ int owner;
    const int r = blockIdx.x, tid = threadIdx.x, T = blockDim.x, lane = tid & 63, wave = tid >> 6;
    const float* row = logits + (long)r * ld;
    float mx = -INFINITY;
#pragma unroll 8
    for (int i = tid; i < V; i += T) mx = fmaxf(mx, row[i]);
    mx = block_max(mx, red);
    float s = 0.f;
#pragma unroll 8
    for (int i = tid; i < V; i += T) s += expf((row[i] - mx) * inv_temperature);
    // inclusive prefix of the threads' sums: inside a wavefront, then the wavefronts before it
    float incl = s;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
    }
    if (lane == 63) wave_incl[wave] = incl;
    if (tid == 0) owner = 0;
    __syncthreads();
    float before = 0.f, total = 0.f;
    for (int w = 0; w < (T >> 6); ++w) {
        if (w < wave) before += wave_incl[w];
        total += wave_incl[w];
    }
    const float pre = before + incl - s;                  // sum of the threads before this one
    uint32_t ctr[4] = {(uint32_t)request_ids[r], (uint32_t)steps[r], 0u, 0u};
    philox4x32(ctr, seed_lo, seed_hi);
    const float u = (float)(ctr[0] >> 8) * (1.0f / 16777216.0f);   // [0, 1)
    const float target = u * total;
    if (tid == 0 && u_out) u_out[r] = u;
    // the owner: the last thread with a non-empty share that starts at or before the target
    if (s > 0.f && pre <= target) atomicMax(&owner, tid);
    __syncthreads();
    if (tid == owner) {
        float c = pre;
        int pick = -1, last = tid < V ? tid : 0;
        for (int i = tid; i < V; i += T) {
            const float e = expf((row[i] - mx) * inv_temperature);
            if (e > 0.f) last = i;
            c += e;
            if (c > target) {
                pick = i;
                break;
            }
        }
        out[r] = pick >= 0 ? pick : last;
    }
}

extern "C" const char* cpmcu_sample(const float* logits, long ld, int rows, int V, float temperature,
                                    unsigned long long seed, const int* request_ids, const int* steps, int* out,
                                    float* u_out, hipStream_t stream) {
    CPMCU_REQUIRE(rows > 0 && V > 0 && ld >= V, "sample: bad shape rows=%d V=%d ld=%ld", rows, V, ld);
    CPMCU_REQUIRE(temperature > 0.f, "sample: temperature %g must be positive (0 is greedy: use argmax)", temperature);
    sample_kernel<<<rows, V >= 4096 ? 1024 : 256, 0, stream>>>(logits, ld, V, 1.0f / temperature, (uint32_t)seed,
                                            (uint32_t)(seed >> 32), request_ids, steps, out, u_out);
    CPMCU_LAUNCH_CHECK("sample");
    return nullptr;
}
