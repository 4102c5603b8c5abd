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
    if constexpr (sizeof(T) == 2) {
        // bf16: a thread takes 8 neighbouring features, which lie in one 16-byte piece of every key and of
        // the compressed key (head sizes are multiples of 16); the sums run over the keys in the same order
        // as below, feature by feature
        for (int e = threadIdx.x; e < width / 8; e += blockDim.x) {
            const int kvh = (e * 8) / hd, d = e * 8 - kvh * hd;
            float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
            for (int r = 0; r < ks; ++r) {
                const uint4 u = *(const uint4*)(kpool + key_index(paged_row(pv, slot, first + r), kvh, nkv, hd) +
                                                key_d_offset(d));
                const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[2 * j] += __uint_as_float(w[j] << 16);
                    acc[2 * j + 1] += __uint_as_float(w[j] & 0xffff0000u);
                }
            }
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                o[j] = (uint32_t)f32_to_bf16(acc[2 * j] / (float)ks).v | ((uint32_t)f32_to_bf16(acc[2 * j + 1] / (float)ks).v << 16);
            *(uint4*)(ckpool + ck_index(page, (first % pv.page_size) / st, kvh, nkv, hd, rpp) + ck_d_offset(d, rpp)) =
                make_uint4(o[0], o[1], o[2], o[3]);
        }
        return;
    }
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
    // Contexts whose scores and ranking arrays do not fit into LDS keep them in global scratch instead, a row
    // of spill_stride floats for every (token, kv head): [scores ...][ranking arrays]; null: all in LDS
    float* spill;
    long spill_stride;
    int score_spilled, work_spilled;
};

// SPILL: the arrays lie in global scratch rows (a template switch, so that without it the compiler knows them
// to be LDS and reads them with LDS instructions instead of generic ones)
template <typename T, bool SPILL>
__global__ __launch_bounds__(256) void sparse_select_kernel(const T* __restrict__ q, const T* __restrict__ ckpool,
                                                           PagedView pv, const int* __restrict__ positions,
                                                           const int* __restrict__ tok_slot, SelectParams sp,
                                                           int* __restrict__ sel_blocks, int* __restrict__ sel_count) {
    extern __shared__ float lds[];
    __shared__ float red[17];
    const int t = blockIdx.x, g = blockIdx.y, tid = threadIdx.x;
    const int p = positions[t];
    const long out_idx = (long)t * sp.nkv + g;
    // tmp[max_ck] score[max_ck] pool[max_blocks] flag[max_blocks] in LDS, or in this row of the global scratch
    float* tmp = lds;
    if constexpr (SPILL) tmp = sp.spill + out_idx * sp.spill_stride;
    float* score = tmp + sp.max_ck;
    float* pool = score + sp.max_ck;
    int* flag = (int*)(pool + sp.max_blocks);
    float* qs = (float*)(flag + sp.max_blocks);
    if constexpr (SPILL) qs = lds;
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

// ---------------------------------------------------------------------------
// From the scores of the visible compressed keys (LDS score[0, n_vis)) to the ascending block list of one
// (token, kv head): pool the scores over each candidate block, rank the candidates by (larger pooled score,
// lower index), flag the first topk ranks and the window, write the flagged blocks in ascending order.
// A candidate's pooled score and index make one 64-bit key (the float's bits made monotone, then the index
// counted down), so that its rank is the number of larger keys: one comparison a pair.  When the block has
// more threads than candidates, several threads share a candidate's scan.
// work: LDS for select_work_floats(max_blocks) floats, 16-byte aligned; every thread of the block calls this.
// ---------------------------------------------------------------------------
__host__ __device__ inline int select_work_floats(int max_blocks) { return 4 * ((max_blocks + 3) / 4 * 4) + 4; }

template <int NW>
__device__ inline void blocks_from_scores(const float* score, float* work, int* wave_tot, const SelectParams& sp,
                                          int n_vis, int q_block, int n_cand, long out_idx,
                                          int* __restrict__ sel_blocks, int* __restrict__ sel_count) {
    constexpr int NT = NW * 64;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int mb4 = (sp.max_blocks + 3) / 4 * 4;
    unsigned long long* keys = (unsigned long long*)work;        // [mb4]
    int* rank = (int*)(work + 2 * mb4);                          // [mb4]
    int* flag = rank + mb4;                                      // [mb4]
    const int n_cand2 = (n_cand + 1) / 2 * 2;
    for (int b = tid; b < n_cand2; b += NT) {
        float v = -INFINITY;
        if (b < sp.init_blocks && b < n_cand) {
            v = INFINITY;
        } else if (b < n_cand) {
            const int lo_tok = sp.bs * b - sp.ks + 1;
            const int j_lo = lo_tok <= 0 ? 0 : (lo_tok + sp.st - 1) / sp.st;
            const int j_hi = min((sp.bs * (b + 1) - 1) / sp.st, n_vis - 1);
            for (int j = j_lo; j <= j_hi; ++j) v = fmaxf(v, score[j]);
        }
        unsigned u = __float_as_uint(v);
        u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);           // larger float, larger unsigned
        // the padding entry (n_cand odd) gets the smallest key of all: it is counted by nobody
        keys[b] = b < n_cand ? (((unsigned long long)u << 32) | (unsigned)(0x7fffffff - b)) : 0ull;
        rank[b] = 0;
    }
    __syncthreads();
    if (n_cand > 0) {
        const int nb_pad = (n_cand + 63) / 64 * 64;
        const int parts = nb_pad < NT ? NT / nb_pad : 1;          // threads that share a candidate's scan
        const int chunk = ((n_cand2 + parts - 1) / parts + 1) / 2 * 2;
        for (int e = tid; e < parts * nb_pad; e += NT) {
            const int b = e % nb_pad, part = e / nb_pad;
            if (b >= n_cand) continue;
            const unsigned long long mine = keys[b];
            const int o0 = part * chunk, o1 = min(o0 + chunk, n_cand2);
            int r = 0;
            // two keys a read, eight reads in flight, so that the latencies of LDS overlap
#pragma unroll 8
            for (int o = o0; o < o1; o += 2) {
                const ulonglong2 k2 = *(const ulonglong2*)(keys + o);
                r += (k2.x > mine ? 1 : 0) + (k2.y > mine ? 1 : 0);
            }
            if (parts > 1) atomicAdd(&rank[b], r);                // integers: the order does not matter
            else rank[b] = r;
        }
    }
    __syncthreads();
    for (int b = tid; b <= q_block; b += NT) flag[b] = b < n_cand ? (rank[b] < sp.topk ? 1 : 0) : 1;   // window: all
    __syncthreads();
    // ascending list: a prefix count over the flags, one block a thread a round
    int* dst = sel_blocks + out_idx * sp.max_sel;
    int base = 0;
    for (int b0 = 0; b0 <= q_block; b0 += NT) {
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

// steps of few tokens: three kernels (defined at the end of this file)
struct SelectScratch {
    float* sraw;      // [token * kv head][head of the group][max_ck]      raw scores * scale * log2(e)
    float* stats;     // [token * kv head][group of 64 keys][head][2]      (max, sum of 2^(s - max)) of the group
    float* score;     // [token * kv head][max_ck]                          softmax summed over the heads
    int n_groups;
};
template <int HD>
__global__ void select_scores_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ ckpool, PagedView pv,
                                     const int* __restrict__ positions, const int* __restrict__ tok_slot,
                                     SelectParams sp, SelectScratch sc);
__global__ void select_normalise_kernel(const int* __restrict__ positions, SelectParams sp, SelectScratch sc,
                                        int stats_in_lds);
template <int SPILL>
__global__ void select_blocks_kernel(const int* __restrict__ positions, SelectParams sp, SelectScratch sc,
                                     int* __restrict__ sel_blocks, int* __restrict__ sel_count, int stats_off);
template <int HD, int NW, int SPILL>
__global__ void sparse_select_mfma_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ ckpool, PagedView pv,
                                          const int* __restrict__ positions, const int* __restrict__ tok_slot,
                                          SelectParams sp, int* __restrict__ sel_blocks, int* __restrict__ sel_count);

// ---------------------------------------------------------------------------
// Which kernels a selection runs as and where their arrays lie: decided on the host from the sizes alone, by
// cpmcu_sparse_select and by cpmcu_sparse_select_scratch (which tells the caller how much scratch to bring).
//   plain:        the plain kernel (float32 engine, or asked for): scores and ranking arrays in LDS, or all of
//                 them in a row of scratch when they exceed it
//   few tokens:   scratch = [raw scores][groups' statistics][scores] (+ [ranking arrays] when LDS cannot hold them)
//   many tokens:  the fused matrix-core kernel; scores, then also the ranking arrays, move to scratch rows when
//                 LDS cannot hold them
// ---------------------------------------------------------------------------
static constexpr size_t SELECT_LDS_LIMIT = 60 * 1024;

struct SelectPlan {
    bool mfma, few;
    int max_ck, max_ck4, max_blocks, n_groups, G;
    bool score_spilled, work_spilled, fused_blocks, stats_in_lds;
    size_t lds_main, lds_stats;
    long off_stats, off_score, off_spill, spill_stride, need;     // in floats
};

static long round4(long v) { return (v + 3) / 4 * 4; }

static SelectPlan select_plan(int dtype, int n, int nh, int nkv, int hd, int ks, int st, int bs, int max_pos,
                              int force_plain, bool have_scratch) {
    SelectPlan pl{};
    pl.G = nh / nkv;
    pl.max_ck = max_pos < ks ? 1 : (max_pos - ks) / st + 1;
    pl.max_ck4 = (int)round4(pl.max_ck);
    pl.max_blocks = max_pos / bs + 1;
    pl.n_groups = (pl.max_ck + 63) / 64;
    const long rows = (long)n * nkv;
    pl.mfma = dtype == CPMCU_BF16 && force_plain != 1 && hd >= 16 && hd <= 128 && hd % 16 == 0;
    if (!pl.mfma) {
        const size_t all = sizeof(float) * ((size_t)2 * pl.max_ck + 2 * pl.max_blocks + hd + 8);
        pl.score_spilled = pl.work_spilled = all > SELECT_LDS_LIMIT;
        pl.lds_main = pl.score_spilled ? sizeof(float) * (hd + 8) : all;
        pl.spill_stride = round4(2L * pl.max_ck + 2L * pl.max_blocks);
        pl.need = pl.score_spilled ? rows * pl.spill_stride : 0;
        return pl;
    }
    const size_t score_b = sizeof(float) * (size_t)(pl.max_ck4 + 4);
    const size_t work_b = sizeof(float) * (size_t)select_work_floats(pl.max_blocks);
    pl.score_spilled = score_b + work_b > SELECT_LDS_LIMIT;
    pl.work_spilled = work_b > SELECT_LDS_LIMIT;
    pl.lds_main = (pl.score_spilled ? 0 : score_b) + (pl.work_spilled ? 0 : work_b);
    if (pl.lds_main == 0) pl.lds_main = 16;
    pl.few = rows <= 256 && (have_scratch || pl.score_spilled);
    if (pl.few) {
        pl.off_stats = round4(rows * pl.max_ck * pl.G);
        pl.off_score = pl.off_stats + round4(rows * pl.n_groups * pl.G * 2);
        pl.off_spill = pl.off_score + round4(rows * pl.max_ck);
        pl.spill_stride = pl.work_spilled ? round4(select_work_floats(pl.max_blocks)) : 0;
        pl.need = pl.off_spill + rows * pl.spill_stride;
        pl.lds_stats = sizeof(float) * ((size_t)pl.n_groups * pl.G * 2 + 2 * pl.G);
        const size_t main8 = (pl.lds_main + 7) / 8 * 8;
        pl.fused_blocks = !pl.score_spilled && main8 + pl.lds_stats <= SELECT_LDS_LIMIT && force_plain != 2;
        pl.stats_in_lds = pl.lds_stats <= SELECT_LDS_LIMIT;
        if (!pl.stats_in_lds) pl.lds_stats = sizeof(float) * 2 * pl.G;
    } else {
        pl.spill_stride = pl.score_spilled ? pl.max_ck4 + (pl.work_spilled ? round4(select_work_floats(pl.max_blocks)) : 0) : 0;
        pl.need = rows * pl.spill_stride;
    }
    return pl;
}

// Floats of scratch that cpmcu_sparse_select wants for these sizes (0: none).  bf16 steps of few tokens run
// faster with it (three kernels of many small workgroups); contexts beyond what LDS holds need it.
extern "C" long cpmcu_sparse_select_scratch(int dtype, int n, int nh, int nkv, int hd, int ks, int st, int bs,
                                            int max_pos, int force_plain) {
    if (n <= 0 || nkv <= 0 || nh <= 0 || nh % nkv || st <= 0 || bs <= 0 || ks <= 0) return 0;
    return select_plan(dtype, n, nh, nkv, hd, ks, st, bs, max_pos, force_plain, true).need;
}

extern "C" const char* cpmcu_sparse_select(const void* q, const void* ckpool, int dtype, int n, int nh, int nkv,
                                           int hd, float scale, const int* page_table, int table_width,
                                           int page_size, const int* positions, const int* tok_slot, int ks, int st,
                                           int bs, int init_blocks, int topk, int window_blocks, int dense_len,
                                           int max_pos, int* sel_blocks, int* sel_count, int max_sel,
                                           int force_plain, float* scratch, long scratch_floats, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && nh > 0 && nkv > 0 && hd > 0 && nh % nkv == 0, "sparse_select: bad shape");
    CPMCU_REQUIRE(hd % 8 == 0, "sparse_select: compressed keys lie in pieces of 8 elements; head_dim %d is no multiple", hd);
    CPMCU_REQUIRE(st > 0 && ks >= st && bs % st == 0 && page_size % st == 0,
                  "sparse_select: kernel_stride %d must divide block_size %d and the cache page of %d tokens", st, bs,
                  page_size);
    CPMCU_REQUIRE(window_blocks >= 1 && max_sel >= topk + window_blocks,
                  "sparse_select: block list of %d entries cannot hold topk %d + window %d", max_sel, topk,
                  window_blocks);
    CPMCU_REQUIRE(dtype == CPMCU_F32 || dtype == CPMCU_BF16, "sparse_select: unknown dtype %d", dtype);
    CPMCU_REQUIRE(max_pos >= 0, "sparse_select: negative position bound");
    const SelectPlan pl = select_plan(dtype, n, nh, nkv, hd, ks, st, bs, max_pos, force_plain, scratch != nullptr);
    CPMCU_REQUIRE(pl.need == 0 || (scratch && scratch_floats >= pl.need),
                  "sparse_select: %d tokens at a context of up to %d tokens need %ld floats of scratch, %ld were given",
                  n, max_pos + 1, pl.need, scratch ? scratch_floats : 0L);
    CPMCU_REQUIRE(((uintptr_t)scratch & 15) == 0, "sparse_select: the scratch must be aligned to 16 bytes");
    SelectParams sp;
    sp.nh = nh; sp.nkv = nkv; sp.hd = hd; sp.scale = scale;
    sp.ks = ks; sp.st = st; sp.bs = bs; sp.init_blocks = init_blocks; sp.topk = topk;
    sp.window_blocks = window_blocks; sp.dense_len = dense_len;
    sp.max_ck = pl.max_ck;
    sp.max_blocks = pl.max_blocks;
    sp.max_sel = max_sel;
    sp.spill = nullptr;
    sp.spill_stride = pl.spill_stride;
    sp.score_spilled = pl.score_spilled ? 1 : 0;
    sp.work_spilled = pl.work_spilled ? 1 : 0;
    dim3 grid(n, nkv);
    PagedView pv{page_table, table_width, page_size};
    if (!pl.mfma) {
        sp.spill = pl.score_spilled ? scratch : nullptr;
#define PLAIN(T, SP)                                                                                               \
        sparse_select_kernel<T, SP><<<grid, 256, pl.lds_main, stream>>>((const T*)q, (const T*)ckpool, pv, positions, \
                                                                        tok_slot, sp, sel_blocks, sel_count)
        if (dtype == CPMCU_F32) {
            if (pl.score_spilled) PLAIN(float, true); else PLAIN(float, false);
        } else {
            if (pl.score_spilled) PLAIN(bf16_t, true); else PLAIN(bf16_t, false);
        }
#undef PLAIN
        CPMCU_LAUNCH_CHECK("sparse_select");
        return nullptr;
    }
    // force_plain: 1 = the plain kernel whatever the type; 2 = matrix cores, but steps of few tokens with the
    // kernel that normalises the scores kept apart (as for contexts whose statistics do not fit into LDS)
    if (pl.few) {
        // few tokens: raw scores and their softmax by many small workgroups through `scratch`, then one
        // workgroup a (token, kv head) for the block list
        SelectScratch sc;
        sc.n_groups = pl.n_groups;
        sc.sraw = scratch;
        sc.stats = scratch + pl.off_stats;
        sc.score = scratch + pl.off_score;
        sp.spill = scratch + pl.off_spill;
        const int G = pl.G;
        dim3 sgrid(n, nkv * ((G + 15) / 16), sc.n_groups);
        CPMCU_REQUIRE(sgrid.y <= 65535 && sgrid.z <= 65535, "sparse_select: too many head tiles or compressed keys");
        CPMCU_REQUIRE(G <= 256, "sparse_select: %d heads a kv head (256 are taken)", G);
#define SCORES(HDv)                                                                                               \
        select_scores_kernel<HDv><<<sgrid, 256, 0, stream>>>((const bf16_t*)q, (const bf16_t*)ckpool, pv, positions, \
                                                             tok_slot, sp, sc)
        switch (hd) {
            case 16: SCORES(16); break;
            case 32: SCORES(32); break;
            case 48: SCORES(48); break;
            case 64: SCORES(64); break;
            case 80: SCORES(80); break;
            case 96: SCORES(96); break;
            case 112: SCORES(112); break;
            default: SCORES(128); break;
        }
#undef SCORES
        CPMCU_LAUNCH_CHECK("select_scores");
        if (pl.fused_blocks) {
            // the last kernel normalises the scores itself (the same sums in the same order): one kernel
            // of the chain less
            const size_t main8 = (pl.lds_main + 7) / 8 * 8;
            select_blocks_kernel<0><<<grid, 1024, main8 + pl.lds_stats, stream>>>(positions, sp, sc, sel_blocks, sel_count,
                                                                                 (int)(main8 / sizeof(float)));
            CPMCU_LAUNCH_CHECK("select_blocks");
            return nullptr;
        }
        select_normalise_kernel<<<dim3(n, nkv, (sp.max_ck + 255) / 256), 256, pl.lds_stats, stream>>>(
            positions, sp, sc, pl.stats_in_lds ? 1 : 0);
        CPMCU_LAUNCH_CHECK("select_normalise");
        const int spill = pl.work_spilled ? 2 : (pl.score_spilled ? 1 : 0);
        if (spill == 2) select_blocks_kernel<2><<<grid, 1024, pl.lds_main, stream>>>(positions, sp, sc, sel_blocks, sel_count, 0);
        else if (spill == 1) select_blocks_kernel<1><<<grid, 1024, pl.lds_main, stream>>>(positions, sp, sc, sel_blocks, sel_count, 0);
        else select_blocks_kernel<0><<<grid, 1024, pl.lds_main, stream>>>(positions, sp, sc, sel_blocks, sel_count, 0);
        CPMCU_LAUNCH_CHECK("select_blocks");
        return nullptr;
    }
    sp.spill = pl.score_spilled ? scratch : nullptr;
    // few tokens (decode steps): 16 wavefronts share a (token, kv head)'s compressed keys; many: 4
    const int spill = pl.work_spilled ? 2 : (pl.score_spilled ? 1 : 0);
#define LAUNCH_S(HDv, NWv, SPv)                                                                              \
    sparse_select_mfma_kernel<HDv, NWv, SPv><<<grid, NWv * 64, pl.lds_main, stream>>>(                       \
        (const bf16_t*)q, (const bf16_t*)ckpool, pv, positions, tok_slot, sp, sel_blocks, sel_count)
#define LAUNCH(HDv)                                                                                          \
    do {                                                                                                     \
        if (n * nkv <= 256) {                                                                                \
            if (spill == 2) LAUNCH_S(HDv, 16, 2); else if (spill == 1) LAUNCH_S(HDv, 16, 1); else LAUNCH_S(HDv, 16, 0); \
        } else {                                                                                             \
            if (spill == 2) LAUNCH_S(HDv, 4, 2); else if (spill == 1) LAUNCH_S(HDv, 4, 1); else LAUNCH_S(HDv, 4, 0);    \
        }                                                                                                    \
    } while (0)
    switch (hd) {
        case 16: LAUNCH(16); break;
        case 32: LAUNCH(32); break;
        case 48: LAUNCH(48); break;
        case 64: LAUNCH(64); break;
        case 80: LAUNCH(80); break;
        case 96: LAUNCH(96); break;
        case 112: LAUNCH(112); break;
        default: LAUNCH(128); break;
    }
#undef LAUNCH
#undef LAUNCH_S
    CPMCU_LAUNCH_CHECK("sparse_select_mfma");
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

// SPILL: 0 = scores and ranking arrays in LDS, 1 = scores in a scratch row, 2 = both (template switches, so that
// the compiler knows which accesses are LDS)
template <int HD, int NW, int SPILL>
__global__ __launch_bounds__(NW * 64) void sparse_select_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ ckpool, PagedView pv,
    const int* __restrict__ positions, const int* __restrict__ tok_slot, SelectParams sp,
    int* __restrict__ sel_blocks, int* __restrict__ sel_count) {
    constexpr int KSTEPS = (HD + 31) / 32;
    extern __shared__ float lds[];
    __shared__ float stat_s[NW][16][2];
    __shared__ int wave_tot[NW];
    const int t = blockIdx.x, kvh = blockIdx.y, tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int p = positions[t];
    const long out_idx = (long)t * sp.nkv + kvh;
    const int max_ck4 = (sp.max_ck + 3) / 4 * 4;
    float* score = lds;
    float* work = lds + max_ck4;
    if constexpr (SPILL >= 1) {
        score = sp.spill + out_idx * sp.spill_stride;
        work = lds;
    }
    if constexpr (SPILL == 2) work = sp.spill + out_idx * sp.spill_stride + max_ck4;
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
    const unsigned rpp_magic = (unsigned)(((1ull << 32) + rows_per_page - 1) / (unsigned)rows_per_page);
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
        // The wavefront's tiles of 16 compressed keys in turn, f(tile, scores).  B operand: lane (key n, g) holds
        // CK[key][32*ks + 8g .. +8].  A tile's page is looked up two tiles ahead and its keys are asked for one
        // tile ahead, so that neither latency stands between two tiles' arithmetic.
        // (a division by rows_per_page for every tile and lane would be a third of this kernel's vector
        // instructions: floor(j / r) = umulhi(j, ceil(2^32 / r)) for j < 2^32 / r)
        auto locate = [&](int tile, int& page, int& row) {
            const int j = min(tile * 16 + n, n_vis - 1);
            const int pg = rows_per_page == 1 ? j : (int)__umulhi((unsigned)j, rpp_magic);
            row = j - pg * rows_per_page;
            page = ptab[pg];
        };
        auto load_b = [&](int page, int row, sbf16x8_t (&b)[KSTEPS]) {
            const bf16_t* ck = ckpool + ck_index(page, row, kvh, sp.nkv, HD, rows_per_page) + g * rows_per_page * 8;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                sbf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
                if (ks * 32 + g * 8 < HD) v = *(const sbf16x8_t*)(ck + ks * 4 * rows_per_page * 8);
                b[ks] = v;
            }
        };
        auto for_tiles = [&](auto f) {
            if (wave >= n_tiles) return;
            sbf16x8_t b[KSTEPS], bn[KSTEPS];
            int page, row, page_next, row_next;
            locate(wave, page, row);
            load_b(page, row, b);
            locate(wave + NW, page_next, row_next);           // (tiles beyond the last repeat the last key)
            for (int tile = wave; tile < n_tiles; tile += NW) {
                int page_after, row_after;
                locate(tile + 2 * NW, page_after, row_after);
                load_b(page_next, row_next, bn);
                sfloatx4_t st = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ++ks) st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], b[ks], st, 0, 0, 0);
                f(tile, st);                    // st[i]: head 4g+i (of this head tile) x key tile*16+n
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ++ks) b[ks] = bn[ks];
                page_next = page_after;
                row_next = row_after;
            }
        };
        // pass 1: running max and sum per head, per lane
        float m[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY}, l[4] = {0.f, 0.f, 0.f, 0.f};
        for_tiles([&](int tile, const sfloatx4_t& st) {
            if (tile * 16 + n < n_vis) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // one exponential an element: of the two terms of the running sum, the one that belongs to
                    // the larger of (old max, new score) has weight 1 (the bare hardware exponential: its
                    // argument is <= 0, and what underflows adds nothing)
                    const float s = st[i] * scale_log2e;
                    const float e = __builtin_amdgcn_exp2f(-fabsf(s - m[i]));
                    l[i] = s > m[i] ? l[i] * e + 1.0f : l[i] + e;
                    m[i] = fmaxf(m[i], s);
                }
            }
        });
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
        for_tiles([&](int tile, const sfloatx4_t& st) {
            float v = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (invL[i] > 0.f) v += __builtin_amdgcn_exp2f(__builtin_fmaf(st[i], scale_log2e, -M[i])) * invL[i];
            v = rows_sum(v);
            const int j = tile * 16 + n;
            if (g == 0 && j < n_vis) score[j] += v;
        });
    }
    __syncthreads();
    blocks_from_scores<NW>(score, work, wave_tot, sp, n_vis, q_block, n_cand, out_idx, sel_blocks, sel_count);
}

// ===========================================================================
// Steps of few tokens (decode): three kernels, because one workgroup for a (token, kv head) would pull the
// compressed keys of a long context through a single CU, one memory latency after the other.
//   select_scores_kernel:    a wavefront a tile of 16 compressed keys, a workgroup 64 keys: raw scores
//                            sraw = q_head . ck_key * scale * log2(e), and per head the group's (max, sum)
//   select_normalise_kernel: a thread a key: merges the groups' (max, sum) per head, then
//                            score[key] = sum over heads of 2^(s - max) / sum
//   select_blocks_kernel:    a workgroup a (token, kv head): blocks_from_scores
// ===========================================================================
template <int HD>
__global__ __launch_bounds__(256) void select_scores_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ ckpool, PagedView pv,
    const int* __restrict__ positions, const int* __restrict__ tok_slot, SelectParams sp, SelectScratch sc) {
    constexpr int KSTEPS = (HD + 31) / 32;
    __shared__ float st_s[4][16][2];
    const int G = sp.nh / sp.nkv;
    const int t = blockIdx.x, kvh = blockIdx.y % sp.nkv, ht = blockIdx.y / sp.nkv, grp = blockIdx.z;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    const int tile = grp * 4 + wave;
    const int p = positions[t];
    if (p + 1 <= sp.dense_len) return;
    const int n_vis = p < sp.ks ? 0 : (p - sp.ks) / sp.st + 1;
    if (grp * 64 >= n_vis) return;
    const long row = (long)t * sp.nkv + kvh;
    const int* ptab = pv.page_table + (long)tok_slot[t] * pv.table_width;
    const int rpp = pv.page_size / sp.st;
    // B operand first (two dependent loads): lane (key n, g) holds CK[key][32*ks + 8g .. +8]
    const int j = min(tile * 16 + n, n_vis - 1);
    const int pg = j / rpp;
    const bf16_t* ck = ckpool + ck_index(ptab[pg], j - pg * rpp, kvh, sp.nkv, HD, rpp) + g * rpp * 8;
    sbf16x8_t bf[KSTEPS], qf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        sbf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (ks * 32 + g * 8 < HD) v = *(const sbf16x8_t*)(ck + ks * 4 * rpp * 8);
        bf[ks] = v;
    }
    // A operand: lane (head r = n, g) holds Q[head][32*ks + 8g .. +8]
    const bool head_ok = ht * 16 + n < G;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        sbf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
        const int d = ks * 32 + g * 8;
        if (head_ok && d < HD) v = *(const sbf16x8_t*)(q + ((long)t * sp.nh + (long)kvh * G + ht * 16 + n) * HD + d);
        qf[ks] = v;
    }
    sfloatx4_t st = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[ks], bf[ks], st, 0, 0, 0);
    // st[i]: head ht*16 + 4g + i x key tile*16 + n
    const bool key_ok = tile * 16 + n < n_vis;
    const float c = sp.scale * 1.4426950408889634f;
    float m[4], l[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float v = st[i] * c;
        if (key_ok && ht * 16 + 4 * g + i < G) sc.sraw[(row * G + ht * 16 + 4 * g + i) * sp.max_ck + tile * 16 + n] = v;
        m[i] = row16_max(key_ok ? v : -INFINITY);                 // over the tile's 16 keys
        l[i] = row16_sum(key_ok ? exp2f(v - m[i]) : 0.f);
    }
    // the workgroup's 4 tiles into one (max, sum) per head
    if (n == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            st_s[wave][4 * g + i][0] = m[i];
            st_s[wave][4 * g + i][1] = l[i];
        }
    }
    __syncthreads();
    if (threadIdx.x < 16 && ht * 16 + (int)threadIdx.x < G) {
        const int h = threadIdx.x;
        float mm = -INFINITY;
        for (int w = 0; w < 4; ++w) mm = fmaxf(mm, st_s[w][h][0]);
        float ll = 0.f;
        for (int w = 0; w < 4; ++w)
            if (st_s[w][h][0] != -INFINITY) ll += st_s[w][h][1] * exp2f(st_s[w][h][0] - mm);
        float* dst = sc.stats + ((row * sc.n_groups + grp) * G + ht * 16 + h) * 2;
        dst[0] = mm;
        dst[1] = ll;
    }
}

__global__ __launch_bounds__(256) void select_normalise_kernel(const int* __restrict__ positions, SelectParams sp,
                                                               SelectScratch sc, int stats_in_lds) {
    extern __shared__ float2 gst[];          // [group][head] (max, sum) if they fit, then ms/inv behind them
    const int t = blockIdx.x, kvh = blockIdx.y, tid = threadIdx.x;
    const int p = positions[t];
    if (p + 1 <= sp.dense_len) return;
    const int G = sp.nh / sp.nkv;
    const int n_vis = p < sp.ks ? 0 : (p - sp.ks) / sp.st + 1;
    if ((int)blockIdx.z * 256 >= n_vis) return;
    const long row = (long)t * sp.nkv + kvh;
    const int groups = (n_vis + 63) / 64;
    float* ms = stats_in_lds ? (float*)(gst + (long)sc.n_groups * G) : (float*)gst;
    float* inv = ms + G;
    // all threads fetch the groups' (max, sum) at once; then a wavefront a head in turn, a lane a group of 64
    // keys, maximum and sum by wave reductions: the same sums in the same order as select_blocks_kernel forms
    // when it normalises the scores itself, so both forms give the same scores to the last bit, and the
    // result does not depend on which workgroup forms it
    const float2* st = (const float2*)(sc.stats + row * sc.n_groups * G * 2);
    const float2* src = st;
    if (stats_in_lds) {
        for (int i = tid; i < groups * G; i += 256) gst[i] = st[i];
        __syncthreads();
        src = gst;
    }
    const int wave = tid >> 6, lane = tid & 63;
    for (int h = wave; h < G; h += 4) {
        float mm = -INFINITY;
        for (int gi = lane; gi < groups; gi += 64) mm = fmaxf(mm, src[gi * G + h].x);
        mm = wave_max(mm);
        float ll = 0.f;
        for (int gi = lane; gi < groups; gi += 64) {
            const float2 v = src[gi * G + h];
            ll += v.y * exp2f(v.x - mm);
        }
        ll = wave_sum(ll);
        if (lane == 0) {
            ms[h] = mm;
            inv[h] = ll > 0.f ? 1.0f / ll : 0.f;
        }
    }
    __syncthreads();
    const int j = blockIdx.z * 256 + tid;
    if (j < n_vis) {
        const float* s = sc.sraw + row * G * sp.max_ck + j;
        float a = 0.f;
#pragma unroll 16
        for (int h = 0; h < G; ++h) a += exp2f(s[(long)h * sp.max_ck] - ms[h]) * inv[h];
        sc.score[row * sp.max_ck + j] = a;
    }
}

// stats_off (in floats, or 0): where in LDS the groups' (max, sum) pairs go when this kernel does the work of
// select_normalise_kernel itself; 0: the scores come ready in sc.score (and are read from there, not copied
// into LDS, when sp.score_spilled says that LDS cannot hold them)
template <int SPILL>
__global__ __launch_bounds__(1024) void select_blocks_kernel(const int* __restrict__ positions, SelectParams sp,
                                                             SelectScratch sc, int* __restrict__ sel_blocks,
                                                             int* __restrict__ sel_count, int stats_off) {
    constexpr int NW = 16;
    extern __shared__ float lds[];
    __shared__ int wave_tot[NW];
    const int t = blockIdx.x, kvh = blockIdx.y, tid = threadIdx.x;
    const int p = positions[t];
    const long out_idx = (long)t * sp.nkv + kvh;
    float* score = lds;
    float* work = lds + (sp.max_ck + 3) / 4 * 4;
    if constexpr (SPILL >= 1) {
        score = sc.score + out_idx * sp.max_ck;
        work = lds;
    }
    if constexpr (SPILL == 2) work = sp.spill + out_idx * sp.spill_stride;
    if (p + 1 <= sp.dense_len) {
        if (tid == 0) sel_count[out_idx] = -1;
        return;
    }
    const int n_vis = p < sp.ks ? 0 : (p - sp.ks) / sp.st + 1;
    const int q_block = p / sp.bs;
    const int n_cand = max(q_block - sp.window_blocks + 1, 0);
    if (stats_off) {
        const int G = sp.nh / sp.nkv;
        const int groups = (n_vis + 63) / 64;
        float2* gst = (float2*)(lds + stats_off);
        float* ms = (float*)(gst + (long)sc.n_groups * G);
        float* inv = ms + G;
        // a wavefront a head in turn, a lane a group of 64 keys: the head's maximum and sum are wave reductions
        // (one thread a head walking through the groups one LDS read at a time took 2.7 us of the kernel's 13.5
        // at 32k keys)
        const float2* st = (const float2*)(sc.stats + out_idx * sc.n_groups * G * 2);
        for (int i = tid; i < groups * G; i += NW * 64) gst[i] = st[i];
        __syncthreads();
        const int wave = tid >> 6, lane = tid & 63;
        for (int h = wave; h < G; h += NW) {
            float mm = -INFINITY;
            for (int gi = lane; gi < groups; gi += 64) mm = fmaxf(mm, gst[gi * G + h].x);
            mm = wave_max(mm);
            float ll = 0.f;
            for (int gi = lane; gi < groups; gi += 64) {
                const float2 v = gst[gi * G + h];
                ll += v.y * exp2f(v.x - mm);
            }
            ll = wave_sum(ll);
            if (lane == 0) {
                ms[h] = mm;
                inv[h] = ll > 0.f ? 1.0f / ll : 0.f;
            }
        }
        __syncthreads();
        for (int j = tid; j < n_vis; j += NW * 64) {
            const float* s = sc.sraw + out_idx * G * sp.max_ck + j;
            float a = 0.f;
#pragma unroll 16
            for (int h = 0; h < G; ++h) a += exp2f(s[(long)h * sp.max_ck] - ms[h]) * inv[h];
            score[j] = a;
        }
    } else if constexpr (SPILL == 0) {
        for (int j = tid; j < n_vis; j += NW * 64) score[j] = sc.score[out_idx * sp.max_ck + j];
    }
    __syncthreads();
    blocks_from_scores<NW>(score, work, wave_tot, sp, n_vis, q_block, n_cand, out_idx, sel_blocks, sel_count);
}
