// InfLLM-v2 block selection: compressed keys, their scores, block pooling and
// top-k, as a function of a query's prefix only (so that the chosen blocks do
// not depend on how tokens were cut into steps).
//
// Stages (reference: src/model/minicpm4/minicpm4_attn.cuh:107-202 runs them per
// call; kernels src/model/minicpm4/minicpm4_kvcache.cuh:6-142, src/model/topk.cuh):
//   ck[j]    = mean(K[st*j : st*j+ks])                      (compress_keys)
//   score[j] = sum_{h in group} softmax_j(q_h.ck[j]*scale)  over ck with st*j+ks <= p
//   pool[b]  = max score[j] over ck overlapping block b; +inf for b < init_blocks
//   chosen   = the min(topk, #candidates) candidates b <= p/bs - lb of largest
//              pool, ties to the lower index
//   list     = chosen U window (p/bs - lb < b <= p/bs), ascending
// The attention kernels then visit exactly the listed blocks.
#include "common.h"

// ---------------------------------------------------------------------------
// One block per token of the step.  The token at position p completes the
// compressed key j = (p+1-ks)/st when (p+1-ks) is a non-negative multiple of
// st.  The compressed keys live in a paged stream with page_size/st rows a page.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void compress_keys_kernel(const T* __restrict__ kpool, T* __restrict__ ckpool, PagedView pv,
                                     const int* __restrict__ positions, const int* __restrict__ tok_slot, int nkv,
                                     int hd, int ks, int st) {
    const int width = nkv * hd;
    const int t = blockIdx.x;
    const int p = positions[t];
    if (p + 1 < ks || (p + 1 - ks) % st != 0) return;
    const int j = (p + 1 - ks) / st;
    const int slot = tok_slot[t];
    const int first = st * j;
    const int page = pv.page_table[(long)slot * pv.table_width + first / pv.page_size];
    const int rpp = pv.page_size / st;
    for (int e = threadIdx.x; e < width; e += blockDim.x) {
        float s = 0.f;
        const int kvh = e / hd, d = e - kvh * hd;
        for (int r = 0; r < ks; ++r) {
            s += to_f32(kpool[key_index(paged_row(pv, slot, first + r), kvh, nkv, hd) + key_d_offset(d)]);
        }
        ckpool[ck_index(page, (first % pv.page_size) / st, kvh, nkv, hd, rpp) + ck_d_offset(d, rpp)] = from_f32<T>(s / (float)ks);
    }
}

extern "C" const char* cpmcu_compress_keys(const void* kpool, void* ckpool, int dtype, int n, int nkv, int hd,
                                           const int* page_table, int table_width, int page_size,
                                           const int* positions, const int* tok_slot, int ks, int st,
                                           hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && nkv > 0 && hd > 0, "compress_keys: empty shape");
    CPMCU_REQUIRE(page_size % 32 == 0 && hd % 16 == 0,
                  "compress_keys: the cache takes pages of a multiple of 32 tokens and head sizes in steps of 16 "
                  "(page %d, head_dim %d)", page_size, hd);
    CPMCU_REQUIRE(st > 0 && ks >= st && page_size % st == 0,
                  "compress_keys: kernel_stride %d must divide the cache page of %d tokens (kernel_size %d)", st,
                  page_size, ks);
    PagedView pv{page_table, table_width, page_size};
    if (dtype == CPMCU_F32)
        compress_keys_kernel<float><<<n, 128, 0, stream>>>((const float*)kpool, (float*)ckpool, pv, positions,
                                                           tok_slot, nkv, hd, ks, st);
    else if (dtype == CPMCU_BF16)
        compress_keys_kernel<bf16_t><<<n, 128, 0, stream>>>((const bf16_t*)kpool, (bf16_t*)ckpool, pv, positions,
                                                            tok_slot, nkv, hd, ks, st);
    else
        CPMCU_FAIL("compress_keys: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("compress_keys");
    return nullptr;
}

// ---------------------------------------------------------------------------
// One block per (token, kv head).  LDS: tmp[max_ck] score[max_ck] pool[max_blocks]
// flag[max_blocks] q[hd].
// ---------------------------------------------------------------------------
struct SelectParams {
    int nh, nkv, hd;
    float scale;
    int ks, st, bs, init_blocks, topk, window_blocks, dense_len;
    int max_ck, max_blocks, max_sel;
};

template <typename T>
__global__ __launch_bounds__(256) void sparse_select_kernel(const T* __restrict__ q, const T* __restrict__ ckpool,
                                                           PagedView pv, const int* __restrict__ positions,
                                                           const int* __restrict__ tok_slot, SelectParams sp,
                                                           int* __restrict__ sel_blocks, int* __restrict__ sel_count) {
    extern __shared__ float lds[];
    __shared__ float red[17];
    float* tmp = lds;
    float* score = tmp + sp.max_ck;
    float* pool = score + sp.max_ck;
    int* flag = (int*)(pool + sp.max_blocks);
    float* qs = (float*)(flag + sp.max_blocks);

    const int t = blockIdx.x, g = blockIdx.y, tid = threadIdx.x;
    const int p = positions[t];
    const long out_idx = (long)t * sp.nkv + g;
    if (p + 1 <= sp.dense_len) {
        if (tid == 0) sel_count[out_idx] = -1;
        return;
    }
    const int slot = tok_slot[t];
    const int G = sp.nh / sp.nkv;
    const int n_vis = p < sp.ks ? 0 : (p - sp.ks) / sp.st + 1;
    const int q_block = p / sp.bs;
    const int n_cand = max(q_block - sp.window_blocks + 1, 0);
    const int rows_per_page = pv.page_size / sp.st;

    for (int j = tid; j < n_vis; j += blockDim.x) score[j] = 0.f;
    for (int hh = 0; hh < G; ++hh) {
        __syncthreads();
        const T* qrow = q + ((long)t * sp.nh + (long)g * G + hh) * sp.hd;
        for (int d = tid; d < sp.hd; d += blockDim.x) qs[d] = to_f32(qrow[d]);
        __syncthreads();
        float mx = -INFINITY;
        for (int j = tid; j < n_vis; j += blockDim.x) {
            const int first = sp.st * j;
            const int page = pv.page_table[(long)slot * pv.table_width + first / pv.page_size];
            const T* ck = ckpool + ck_index(page, (first % pv.page_size) / sp.st, g, sp.nkv, sp.hd, rows_per_page);
            float dot = 0.f;
            for (int d = 0; d < sp.hd; ++d) dot += qs[d] * to_f32(ck[ck_d_offset(d, rows_per_page)]);
            const float s = dot * sp.scale;
            tmp[j] = s;
            mx = fmaxf(mx, s);
        }
        mx = block_max(mx, red);
        float sum = 0.f;
        for (int j = tid; j < n_vis; j += blockDim.x) {
            const float e = expf(tmp[j] - mx);
            tmp[j] = e;
            sum += e;
        }
        sum = block_sum(sum, red);
        for (int j = tid; j < n_vis; j += blockDim.x) score[j] += tmp[j] / sum;
    }
    __syncthreads();
    // pool the scores of the compressed keys that overlap each candidate block
    for (int b = tid; b < n_cand; b += blockDim.x) {
        float v = -INFINITY;
        if (b < sp.init_blocks) {
            v = INFINITY;
        } else {
            const int lo_tok = sp.bs * b - sp.ks + 1;                 // st*j >= lo_tok
            const int j_lo = lo_tok <= 0 ? 0 : (lo_tok + sp.st - 1) / sp.st;
            const int j_hi = min((sp.bs * (b + 1) - 1) / sp.st, n_vis - 1);
            for (int j = j_lo; j <= j_hi; ++j) v = fmaxf(v, score[j]);
        }
        pool[b] = v;
    }
    __syncthreads();
    // rank by (larger pool, lower index); the first `topk` ranks are chosen
    for (int b = tid; b <= q_block; b += blockDim.x) {
        int f = 0;
        if (b < n_cand) {
            const float v = pool[b];
            int rank = 0;
            for (int o = 0; o < n_cand; ++o) {
                const float w = pool[o];
                rank += (w > v || (w == v && o < b)) ? 1 : 0;
            }
            f = rank < sp.topk;
        } else {
            f = 1;   // sliding window, the query's own block included
        }
        flag[b] = f;
    }
    __syncthreads();
    if (tid == 0) {
        int* dst = sel_blocks + out_idx * sp.max_sel;
        int c = 0;
        for (int b = 0; b <= q_block; ++b)
            if (flag[b] && c < sp.max_sel) dst[c++] = b;
        sel_count[out_idx] = c;
    }
}

template <int HD, int NW>
__global__ void sparse_select_mfma_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ ckpool, PagedView pv,
                                          const int* __restrict__ positions, const int* __restrict__ tok_slot,
                                          SelectParams sp, int* __restrict__ sel_blocks, int* __restrict__ sel_count);

extern "C" const char* cpmcu_sparse_select(const void* q, const void* ckpool, int dtype, int n, int nh, int nkv,
                                           int hd, float scale, const int* page_table, int table_width,
                                           int page_size, const int* positions, const int* tok_slot, int ks, int st,
                                           int bs, int init_blocks, int topk, int window_blocks, int dense_len,
                                           int max_pos, int* sel_blocks, int* sel_count, int max_sel,
                                           int force_plain, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && nh > 0 && nkv > 0 && hd > 0 && nh % nkv == 0, "sparse_select: bad shape");
    CPMCU_REQUIRE(hd % 8 == 0, "sparse_select: compressed keys lie in pieces of 8 elements; head_dim %d is no multiple", hd);
    CPMCU_REQUIRE(st > 0 && ks >= st && bs % st == 0 && page_size % st == 0,
                  "sparse_select: kernel_stride %d must divide block_size %d and the cache page of %d tokens", st, bs,
                  page_size);
    CPMCU_REQUIRE(window_blocks >= 1 && max_sel >= topk + window_blocks,
                  "sparse_select: block list of %d entries cannot hold topk %d + window %d", max_sel, topk,
                  window_blocks);
    SelectParams sp;
    sp.nh = nh; sp.nkv = nkv; sp.hd = hd; sp.scale = scale;
    sp.ks = ks; sp.st = st; sp.bs = bs; sp.init_blocks = init_blocks; sp.topk = topk;
    sp.window_blocks = window_blocks; sp.dense_len = dense_len;
    sp.max_ck = max_pos < ks ? 1 : (max_pos - ks) / st + 1;
    sp.max_blocks = max_pos / bs + 1;
    sp.max_sel = max_sel;
    const size_t lds = sizeof(float) * ((size_t)2 * sp.max_ck + 2 * sp.max_blocks + hd);
    CPMCU_REQUIRE(lds <= 60 * 1024,
                  "sparse_select: a context of %d tokens needs %zu bytes of LDS for its block scores (limit 61440)",
                  max_pos + 1, lds);
    dim3 grid(n, nkv);
    PagedView pv{page_table, table_width, page_size};
    if (dtype == CPMCU_BF16 && !force_plain && (hd == 16 || hd == 32 || hd == 64 || hd == 128)) {
        const size_t lds2 = sizeof(float) * ((size_t)sp.max_ck + 2 * sp.max_blocks);
        // few tokens (decode steps): 16 wavefronts share a (token, kv head)'s compressed keys; many: 4
#define LAUNCH(HDv)                                                                                          \
        do {                                                                                                 \
            if (n * nkv <= 256)                                                                              \
                sparse_select_mfma_kernel<HDv, 16><<<grid, 1024, lds2, stream>>>(                            \
                    (const bf16_t*)q, (const bf16_t*)ckpool, pv, positions, tok_slot, sp, sel_blocks, sel_count); \
            else                                                                                             \
                sparse_select_mfma_kernel<HDv, 4><<<grid, 256, lds2, stream>>>(                              \
                    (const bf16_t*)q, (const bf16_t*)ckpool, pv, positions, tok_slot, sp, sel_blocks, sel_count); \
        } while (0)
        if (hd == 16) LAUNCH(16);
        else if (hd == 32) LAUNCH(32);
        else if (hd == 64) LAUNCH(64);
        else LAUNCH(128);
#undef LAUNCH
        CPMCU_LAUNCH_CHECK("sparse_select_mfma");
        return nullptr;
    }
    if (dtype == CPMCU_F32)
        sparse_select_kernel<float><<<grid, 256, lds, stream>>>((const float*)q, (const float*)ckpool, pv, positions,
                                                                tok_slot, sp, sel_blocks, sel_count);
    else if (dtype == CPMCU_BF16)
        sparse_select_kernel<bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)q, (const bf16_t*)ckpool, pv,
                                                                 positions, tok_slot, sp, sel_blocks, sel_count);
    else
        CPMCU_FAIL("sparse_select: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("sparse_select");
    return nullptr;
}

// ===========================================================================
// The same selection with the scores on the matrix cores (bf16, head size 16,
// 32, 64 or 128).  One workgroup of 4 or 16 wavefronts per (token, kv head); tiles
// of 16 compressed keys are dealt to the wavefronts in turn.
//   S = Q . CK^T      A = the group's heads (rows) from registers, B = 16
//                     compressed keys straight from their cache rows;
//                     D: lane (key n, g) holds heads 4g..4g+3
//   pass 1: every lane keeps a running max and sum per head over its keys; the
//           lanes and wavefronts merge them once at the end
//   pass 2: the scores again, p = 2^(s - max) / sum, summed over the heads of
//           the group (in-lane and two cross-lane steps) into LDS score[key]
// Pooling, ranking and the list are those of sparse_select_kernel.
// ===========================================================================
typedef __bf16 sbf16x8_t __attribute__((ext_vector_type(8)));
typedef float sfloatx4_t __attribute__((ext_vector_type(4)));

template <int HD, int NW>
__global__ __launch_bounds__(NW * 64) void sparse_select_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ ckpool, PagedView pv,
    const int* __restrict__ positions, const int* __restrict__ tok_slot, SelectParams sp,
    int* __restrict__ sel_blocks, int* __restrict__ sel_count) {
    constexpr int KSTEPS = (HD + 31) / 32;
    extern __shared__ float lds[];
    __shared__ float stat_s[NW][16][2];
    __shared__ int wave_tot[NW];
    float* score = lds;
    float* pool = score + sp.max_ck;
    int* flag = (int*)(pool + sp.max_blocks);

    const int t = blockIdx.x, kvh = blockIdx.y, tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int p = positions[t];
    const long out_idx = (long)t * sp.nkv + kvh;
    if (p + 1 <= sp.dense_len) {
        if (tid == 0) sel_count[out_idx] = -1;
        return;
    }
    const int slot = tok_slot[t];
    const int* ptab = pv.page_table + (long)slot * pv.table_width;
    const int G = sp.nh / sp.nkv;
    const int n_vis = p < sp.ks ? 0 : (p - sp.ks) / sp.st + 1;
    const int q_block = p / sp.bs;
    const int n_cand = max(q_block - sp.window_blocks + 1, 0);
    const int rows_per_page = pv.page_size / sp.st;
    const float scale_log2e = sp.scale * 1.4426950408889634f;
    const int n_tiles = (n_vis + 15) / 16;

    for (int j = tid; j < n_vis; j += blockDim.x) score[j] = 0.f;
    __syncthreads();

    for (int ht = 0; ht * 16 < G; ++ht) {
        // A operand: lane (head r = n, g) holds Q[head][32*ks + 8g .. +8]
        sbf16x8_t qf[KSTEPS];
        const bool head_ok = ht * 16 + n < G;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            sbf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            const int d = ks * 32 + g * 8;
            if (head_ok && d < HD) v = *(const sbf16x8_t*)(q + ((long)t * sp.nh + (long)kvh * G + ht * 16 + n) * HD + d);
            qf[ks] = v;
        }
        auto scores_of_tile = [&](int tile) {
            // B operand: lane (key n, g) holds CK[key][32*ks + 8g .. +8]
            const int j = min(tile * 16 + n, n_vis - 1);
            const int first = sp.st * j;
            const int page = ptab[first / pv.page_size];
            const bf16_t* ck = ckpool + ck_index(page, (first % pv.page_size) / sp.st, kvh, sp.nkv, HD, rows_per_page) +
                               g * rows_per_page * 8;
            sfloatx4_t st = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                sbf16x8_t b = {0, 0, 0, 0, 0, 0, 0, 0};
                if (ks * 32 + g * 8 < HD) b = *(const sbf16x8_t*)(ck + ks * 4 * rows_per_page * 8);
                st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], b, st, 0, 0, 0);
            }
            return st;                      // st[i]: head 4g+i (of this head tile) x key tile*16+n
        };
        // pass 1: running max and sum per head, per lane
        float m[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY}, l[4] = {0.f, 0.f, 0.f, 0.f};
        for (int tile = wave; tile < n_tiles; tile += NW) {
            const sfloatx4_t st = scores_of_tile(tile);
            if (tile * 16 + n < n_vis) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float s = st[i] * scale_log2e;
                    const float m_new = fmaxf(m[i], s);
                    l[i] = l[i] * exp2f(m[i] - m_new) + exp2f(s - m_new);
                    m[i] = m_new;
                }
            }
        }
        // merge over the 16 key lanes of a group, then over the wavefronts
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float om = __shfl_xor(m[i], off, 64), ol = __shfl_xor(l[i], off, 64);
                const float m_new = fmaxf(m[i], om);
                const float a = m[i] == -INFINITY ? 0.f : l[i] * exp2f(m[i] - m_new);
                const float b = om == -INFINITY ? 0.f : ol * exp2f(om - m_new);
                l[i] = a + b;
                m[i] = m_new;
            }
        }
        __syncthreads();
        if (n == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                stat_s[wave][4 * g + i][0] = m[i];
                stat_s[wave][4 * g + i][1] = l[i];
            }
        }
        __syncthreads();
        float M[4], invL[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float mm = -INFINITY;
            for (int w = 0; w < NW; ++w) mm = fmaxf(mm, stat_s[w][4 * g + i][0]);
            float ll = 0.f;
            for (int w = 0; w < NW; ++w) {
                const float wm = stat_s[w][4 * g + i][0];
                if (wm != -INFINITY) ll += stat_s[w][4 * g + i][1] * exp2f(wm - mm);
            }
            M[i] = mm;
            // heads beyond the group (padding rows of the tile) must add nothing
            invL[i] = (ht * 16 + 4 * g + i < G && ll > 0.f) ? 1.0f / ll : 0.f;
        }
        // pass 2: normalised scores summed over the heads of the group
        for (int tile = wave; tile < n_tiles; tile += NW) {
            const sfloatx4_t st = scores_of_tile(tile);
            float v = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (invL[i] > 0.f) v += exp2f(st[i] * scale_log2e - M[i]) * invL[i];
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            const int j = tile * 16 + n;
            if (g == 0 && j < n_vis) score[j] += v;
        }
    }
    __syncthreads();
    // pool the scores of the compressed keys that overlap each candidate block
    for (int b = tid; b < n_cand; b += blockDim.x) {
        float v = -INFINITY;
        if (b < sp.init_blocks) {
            v = INFINITY;
        } else {
            const int lo_tok = sp.bs * b - sp.ks + 1;
            const int j_lo = lo_tok <= 0 ? 0 : (lo_tok + sp.st - 1) / sp.st;
            const int j_hi = min((sp.bs * (b + 1) - 1) / sp.st, n_vis - 1);
            for (int j = j_lo; j <= j_hi; ++j) v = fmaxf(v, score[j]);
        }
        pool[b] = v;
    }
    __syncthreads();
    for (int b = tid; b <= q_block; b += blockDim.x) {
        int f = 1;                                   // sliding window, the query's own block included
        if (b < n_cand) {
            const float v = pool[b];
            int rank = 0;
            for (int o = 0; o < n_cand; ++o) {
                const float w = pool[o];
                rank += (w > v || (w == v && o < b)) ? 1 : 0;
            }
            f = rank < sp.topk;
        }
        flag[b] = f;
    }
    __syncthreads();
    // ascending list: a prefix count over the flags, one block a thread a round
    int* dst = sel_blocks + out_idx * sp.max_sel;
    int base = 0;
    for (int b0 = 0; b0 <= q_block; b0 += NW * 64) {
        const int b = b0 + tid;
        const int f = (b <= q_block) ? flag[b] : 0;
        const unsigned long long mask = __builtin_amdgcn_ballot_w64(f != 0);
        const int before = __popcll(mask & ((1ull << lane) - 1ull));
        if (lane == 0) wave_tot[wave] = __popcll(mask);
        __syncthreads();
        int off = base;
        for (int w = 0; w < wave; ++w) off += wave_tot[w];
        if (f && off + before < sp.max_sel) dst[off + before] = b;
        for (int w = 0; w < NW; ++w) base += wave_tot[w];
        __syncthreads();
    }
    if (tid == 0) sel_count[out_idx] = min(base, sp.max_sel);
}
