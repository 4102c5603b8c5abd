// Attention over the paged cache.
//
// attention_paged_kernel is the plain kernel: one wavefront per (query token,
// query head), one lane per key for the scores, one lane per output column for
// P.V, float softmax with a running maximum.  It takes any head size up to 256,
// any number of heads and groups, both element types, prompts and single
// tokens alike, and an optional list of key blocks per (token, kv head) for
// block-sparse attention.  It is the 32-bit engine's attention and the twin
// against which the tuned bf16 kernels are checked.
//
// Formula (reference: src/model/attn.cuh:200-227, src/flash_attn/flash_api.hpp:294-394):
// s_j = (q.k_j) * scale for keys j <= position of the query, softmax over j in
// float, out = sum_j p_j v_j; query head h reads kv head h / (nh/nkv).
#include "common.h"

template <typename T>
__global__ __launch_bounds__(64) void attention_paged_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ kpool, const T* __restrict__ vpool,
    PagedView pv, const int* __restrict__ positions, const int* __restrict__ tok_slot, int nh, int nkv, int hd,
    float scale, const int* __restrict__ sel_blocks, const int* __restrict__ sel_count, int max_sel, int block_size) {
    __shared__ float qs[256];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int g = h / (nh / nkv);
    const int pos = positions[t], slot = tok_slot[t];
    const T* qrow = q + ((long)t * nh + h) * hd;
    for (int d = lane; d < hd; d += 64) qs[d] = to_f32(qrow[d]);
    __syncthreads();
    const long kv_stride = (long)nkv * hd;
    const int nd = (hd + 63) / 64;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    int n_seg = 1;
    const int* sel = nullptr;
    if (sel_count) {
        const int c = sel_count[(long)t * nkv + g];
        if (c >= 0) {
            n_seg = c;
            sel = sel_blocks + ((long)t * nkv + g) * max_sel;
        }
    }
    for (int si = 0; si < n_seg; ++si) {
        int s0 = 0, s1 = pos + 1;
        if (sel) {
            s0 = sel[si] * block_size;
            s1 = min(s0 + block_size, pos + 1);
        }
        for (int j0 = s0; j0 < s1; j0 += 64) {
            const int j = j0 + lane;
            const bool valid = j < s1;
            int row = 0;
            float s = -INFINITY;
            if (valid) {
                row = (int)paged_row(pv, slot, j);
                const T* kr = kpool + (long)row * kv_stride + (long)g * hd;
                float dot = 0.f;
                for (int d = 0; d < hd; ++d) dot += qs[d] * to_f32(kr[d]);
                s = dot * scale;
            }
            const float m_new = fmaxf(m, wave_max(s));
            const float p = valid ? expf(s - m_new) : 0.f;
            const float corr = expf(m - m_new);
            l = l * corr + wave_sum(p);
            m = m_new;
            const int cnt = min(64, s1 - j0);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] *= corr;
            for (int jj = 0; jj < cnt; ++jj) {
                const float pj = __shfl(p, jj, 64);
                const int rj = __shfl(row, jj, 64);
                const T* vr = vpool + (long)rj * kv_stride + (long)g * hd;
                for (int i = 0; i < nd; ++i) {
                    const int d = lane + 64 * i;
                    if (d < hd) acc[i] += pj * to_f32(vr[d]);
                }
            }
        }
    }
    T* orow = out + ((long)t * nh + h) * hd;
    const float inv = 1.0f / l;
    for (int i = 0; i < nd; ++i) {
        const int d = lane + 64 * i;
        if (d < hd) orow[d] = from_f32<T>(acc[i] * inv);
    }
}

extern "C" const char* cpmcu_attention_plain(const void* q, void* out, int dtype, int n, int nh, int nkv, int hd,
                                             float scale, const void* kpool, const void* vpool,
                                             const int* page_table, int table_width, int page_size,
                                             const int* positions, const int* tok_slot, const int* sel_blocks,
                                             const int* sel_count, int max_sel, int block_size, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && nh > 0 && nkv > 0 && hd > 0, "attention: empty shape n=%d heads=%d kv_heads=%d head_dim=%d",
                  n, nh, nkv, hd);
    CPMCU_REQUIRE(nh % nkv == 0, "attention: %d heads are not a multiple of %d kv heads", nh, nkv);
    CPMCU_REQUIRE(hd <= 256, "attention: head_dim %d > 256 is not supported", hd);
    CPMCU_REQUIRE(nh <= 65535, "attention: %d heads exceed the launch grid", nh);
    CPMCU_REQUIRE(!sel_count || (sel_blocks && max_sel > 0 && block_size > 0), "attention: block list incomplete");
    PagedView pv{page_table, table_width, page_size};
    dim3 grid(n, nh);
    if (dtype == CPMCU_F32)
        attention_paged_kernel<float><<<grid, 64, 0, stream>>>((const float*)q, (float*)out, (const float*)kpool,
                                                               (const float*)vpool, pv, positions, tok_slot, nh, nkv,
                                                               hd, scale, sel_blocks, sel_count, max_sel, block_size);
    else if (dtype == CPMCU_BF16)
        attention_paged_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kpool,
                                                                (const bf16_t*)vpool, pv, positions, tok_slot, nh,
                                                                nkv, hd, scale, sel_blocks, sel_count, max_sel,
                                                                block_size);
    else
        CPMCU_FAIL("attention: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("attention_plain");
    return nullptr;
}
