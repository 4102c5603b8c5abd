// q, k, v projection of a decode step fused with the rotation and the cache write (bf16, at most 64 tokens).
//
// A decode step is a chain of small kernels, each of which costs a few microseconds whatever it does; this one
// replaces the split-K product + the kernel that summed its partial sums, rotated and stored.
//
// The weight [q heads; k heads; v heads] x hidden is re-laid (ops.qkv_rope_weight) so that
//   * the rows of every q and k head stand as rotation pairs side by side: c, c + hd/2, c + 1, c + 1 + hd/2, ...
//     (any even run of rows then holds whole pairs, and a lane's accumulators hold both halves of its pairs);
//     v heads keep their order;
//   * a workgroup owns R consecutive rows, R even, 16 <= R <= 32.  R is chosen so that the workgroups spread
//     evenly over the 256 CUs: with strips of 16 rows the 4,608 rows of the 8B shape are 288 workgroups, 32 CUs
//     get two of them and the kernel takes as long as those (12.3 us against 8.4 for 256 strips); with R = 18
//     they are 256.
//   * per workgroup and 128-column block: a tile of 16 rows as the matrix cores take it ([i][lane][8], lane =
//     16 g + r holding row r, columns 32 i + 8 g ..), then the R - 16 further rows packed as [i][g][row][8].
// One workgroup of 4 wavefronts: the wavefronts take a quarter of the columns each (x straight from global
// memory into the B operand, asked for together with the weight's block), add their results through LDS, and
// the first wavefront rotates and writes: queries to q_out [token][head][d], keys and values into the cache
// pages in the matrix cores' order (common.h: key_index, value_index).
// theta = pos * inv_freq[c]; (a, b) = (x[c], x[c+hd/2]) -> (a cos - b sin, a sin + b cos), cos and sin times
// `mscale` (reference: src/model/rotary.cuh:7-34; cache rows src/model/attn.cuh:14-21; the fused decode
// projection src/model/minicpm4/minicpm4_attn.cuh:209-223).
#include "common.h"

typedef __bf16 qbf16x8_t __attribute__((ext_vector_type(8)));
typedef float qfloatx4_t __attribute__((ext_vector_type(4)));

// PF: 128-column blocks of the weight a wavefront keeps in flight; NW: wavefronts a workgroup; MT: tiles of 16
// tokens; TILES: 1 (R = 16) or 2 (16 < R <= 32) tiles of weight rows
template <int PF, int NW, int MT, int TILES>
__global__ __launch_bounds__(NW * 64) void qkv_rope_kernel(
    const bf16_t* __restrict__ X, long ldx, const bf16_t* __restrict__ W, int M, int K, int R, bf16_t* __restrict__ q_out,
    int nh, int nkv, int hd, const int* __restrict__ positions, const int* __restrict__ tok_slot,
    const float* __restrict__ inv_freq, float mscale, bf16_t* __restrict__ kpool, bf16_t* __restrict__ vpool,
    PagedView pv, const float* __restrict__ row_ss, int ss_slices, float eps, bf16_t* __restrict__ ckpool,
    int ck_size, int ck_stride) {
    __shared__ float red[NW - 1][MT][TILES][4][64];
    __shared__ float rs_s[MT * 16];            // the norm's row factors (common.h: row_scales), if x lacks them
    const int wg = blockIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int nkb = (K + 127) / 128;
    const int per_wave = (nkb + NW - 1) / NW;
    const int kb0 = wave * per_wave, kb1 = min(kb0 + per_wave, nkb);
    const int R2 = R - 16;                                       // rows of the second, packed tile
    const long block_elems = 2048 + 128L * R2;
    const bf16_t* wp = W + (long)wg * nkb * block_elems;
    const bf16_t* wp1 = wp + lane * 8;
    const bf16_t* wp2 = wp + 2048 + (g * R2 + min(r, max(R2 - 1, 0))) * 8;
    const bool row2 = TILES > 1 && r < R2;
    const bf16_t* xp[MT];                                  // rows beyond the step repeat its last token
#pragma unroll
    for (int t = 0; t < MT; ++t) xp[t] = X + (long)min(t * 16 + r, M - 1) * ldx;

    // Loads return in the order of their issue, so the x of a block is asked for together with its w, PF blocks
    // ahead (asked for only at its use, it would make the wavefront wait for every w behind it: one trip to
    // memory a block).  No load stands in a branch that depends on data: addresses are clamped instead (a block
    // beyond the wavefront's last repeats it and is not multiplied; columns beyond K repeat the row's last 8
    // and meet the weight's zero padding), so the waits count exactly.
    qbf16x8_t a[PF][TILES][4], bx[PF][MT][4];
    auto load_block = [&](int kb, qbf16x8_t (&wd)[TILES][4], qbf16x8_t (&xd)[MT][4]) {
        const int kbc = min(kb, nkb - 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) wd[0][i] = __builtin_nontemporal_load((const qbf16x8_t*)(wp1 + kbc * block_elems + i * 512));
        if constexpr (TILES > 1) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                qbf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
                if (row2) v = __builtin_nontemporal_load((const qbf16x8_t*)(wp2 + kbc * block_elems + i * (32L * R2)));
                wd[1][i] = v;
            }
        }
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) xd[t][i] = *(const qbf16x8_t*)(xp[t] + min(kbc * 128 + i * 32 + g * 8, K - 8));
    };
    qfloatx4_t acc[MT][TILES];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int T = 0; T < TILES; ++T) acc[t][T] = qfloatx4_t{0.f, 0.f, 0.f, 0.f};
    // what the end needs (positions, the tokens' cache rows through two dependent lookups, the pairs'
    // frequencies) is asked for first: it is there when the products are, instead of costing three trips to
    // memory after them.  A lane holds, per tile, rows 4g .. 4g+3 of the workgroup's: two pairs (or 4 rows of v).
    const int total_rows = (nh + 2 * nkv) * hd;
    int tok_pos[MT];
    long tok_row[MT];
    const bool has_kv = (long)(wg + 1) * R > (long)nh * hd;      // some row of this workgroup goes into the cache
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int tok = min(t * 16 + r, M - 1);
        tok_pos[t] = positions[tok];
        tok_row[t] = has_kv ? paged_row(pv, tok_slot[tok], tok_pos[t]) : 0;
    }
    // row P of the re-laid weight: head P / hd; inside a q or k head, pair (P % hd) / 2, half (P % hd) % 2
    int pair_head[TILES][2], pair_in[TILES][2];                  // head and first row inside it (even) of a lane's pairs
    bool pair_ok[TILES][2];
    float freq[TILES][2];
#pragma unroll
    for (int T = 0; T < TILES; ++T)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int rho = 16 * T + 4 * g + 2 * j;
            const long P = (long)wg * R + rho;
            pair_ok[T][j] = rho < R && P < total_rows;
            const long Pc = pair_ok[T][j] ? P : 0;
            pair_head[T][j] = (int)(Pc / hd);
            pair_in[T][j] = (int)(Pc - (long)pair_head[T][j] * hd);
            freq[T][j] = (inv_freq && pair_head[T][j] < nh + nkv) ? inv_freq[pair_in[T][j] >> 1] : 0.f;
        }
    auto multiply = [&](qbf16x8_t (&wd)[TILES][4], qbf16x8_t (&xd)[MT][4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int T = 0; T < TILES; ++T)
                    acc[t][T] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wd[T][i], xd[t][i], acc[t][T], 0, 0, 0);
    };
#pragma unroll
    for (int j = 0; j < PF; ++j) load_block(kb0 + j, a[j], bx[j]);
    // the pairs' cosines and sines are formed while the first blocks are on their way
    float rot_cs[MT][TILES][2], rot_sn[MT][TILES][2];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int T = 0; T < TILES; ++T)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                rot_cs[t][T][j] = 1.f;
                rot_sn[t][T][j] = 0.f;
                if (inv_freq && pair_head[T][j] < nh + nkv) {
                    const float ang = (float)tok_pos[t] * freq[T][j];
                    rot_cs[t][T][j] = cosf(ang) * mscale;
                    rot_sn[t][T][j] = sinf(ang) * mscale;
                }
            }
    if (row_ss) row_scales<NW * 64, MT * 16>(row_ss, ss_slices, M, 1.0f / (float)K, eps, rs_s);
    int kb = kb0;
    for (; kb + 2 * PF <= kb1; kb += PF) {           // every block and every block asked for exists
#pragma unroll
        for (int j = 0; j < PF; ++j) {
            multiply(a[j], bx[j]);
            load_block(kb + j + PF, a[j], bx[j]);
        }
    }
    for (; kb < kb1; kb += PF) {                      // the last blocks: nothing more, or only what exists, is asked for
#pragma unroll
        for (int j = 0; j < PF; ++j) {
            if (kb + j < kb1) multiply(a[j], bx[j]);
            if (kb + j + PF < kb1) load_block(kb + j + PF, a[j], bx[j]);
        }
    }
    // lane (token r, g) of tile t: acc[t][T][i] is row 16T + 4g + i of the workgroup; the other wavefronts hand
    // theirs to the first
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int T = 0; T < TILES; ++T)
#pragma unroll
                for (int i = 0; i < 4; ++i) red[wave - 1][t][T][i][lane] = acc[t][T][i];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
        for (int T = 0; T < TILES; ++T)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int w = 0; w < NW - 1; ++w) acc[t][T][i] += red[w][t][T][i][lane];
        if (row_ss) {          // X was x * w of a norm whose row factor comes now
            const float rs = rs_s[t * 16 + r];
#pragma unroll
            for (int T = 0; T < TILES; ++T)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[t][T][i] *= rs;
        }
    }

    float own[MT][TILES][2][2];                    // a key head's values as the cache holds them: [pair][half]
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int tok = t * 16 + r;
        const bool tok_ok = tok < M;
#pragma unroll
        for (int T = 0; T < TILES; ++T)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                own[t][T][j][0] = own[t][T][j][1] = 0.f;
                if (!pair_ok[T][j]) continue;
                const int head = pair_head[T][j], in = pair_in[T][j];
                const float lo = acc[t][T][2 * j], hi = acc[t][T][2 * j + 1];
                if (head < nh + nkv) {
                    const int c = in >> 1;
                    const float cs = rot_cs[t][T][j], sn = rot_sn[t][T][j];
                    const bf16_t v0 = f32_to_bf16(lo * cs - hi * sn), v1 = f32_to_bf16(lo * sn + hi * cs);
                    own[t][T][j][0] = to_f32(v0);
                    own[t][T][j][1] = to_f32(v1);
                    if (!tok_ok) continue;
                    if (head < nh) {
                        bf16_t* dst = q_out + ((long)tok * nh + head) * hd;
                        dst[c] = v0;
                        dst[c + hd / 2] = v1;
                    } else {
                        bf16_t* dst = kpool + key_index(tok_row[t], head - nh, nkv, hd);
                        dst[key_d_offset(c)] = v0;
                        dst[key_d_offset(c + hd / 2)] = v1;
                    }
                } else if (tok_ok) {
                    bf16_t* dst = vpool + value_index(tok_row[t], head - nh - nkv, nkv, hd);
                    dst[value_d_offset(in)] = f32_to_bf16(lo);
                    dst[value_d_offset(in + 1)] = f32_to_bf16(hi);
                }
            }
    }

    // Compressed keys (sparse.hip: compress_keys_kernel, the same sums in the same order): the token at position
    // p completes the mean of the keys p+1-ck_size .. p when p+1-ck_size is a non-negative multiple of ck_stride.
    // This workgroup wrote its features of all the step's keys itself; the fence makes them readable, and is
    // paid only in the steps in which a token completes one.
    if (ckpool && has_kv) {
        bool mine[MT], any = false;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int p1 = tok_pos[t] + 1;
            mine[t] = t * 16 + r < M && p1 >= ck_size && (p1 - ck_size) % ck_stride == 0;
            any = any || mine[t];
        }
        if (__any(any)) {
            __threadfence();
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                if (!mine[t]) continue;
                const int slot = tok_slot[t * 16 + r];
                const int first = tok_pos[t] + 1 - ck_size;
                const int page = pv.page_table[(long)slot * pv.table_width + first / pv.page_size];
                const int rpp = pv.page_size / ck_stride;
#pragma unroll
                for (int T = 0; T < TILES; ++T)
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const int head = pair_head[T][j];
                        if (!pair_ok[T][j] || head < nh || head >= nh + nkv) continue;
                        const int kvh = head - nh, c = pair_in[T][j] >> 1;
                        float s0 = 0.f, s1 = 0.f;
#pragma unroll 4
                        for (int k = 0; k < ck_size - 1; ++k) {
                            const bf16_t* src = kpool + key_index(paged_row(pv, slot, first + k), kvh, nkv, hd);
                            s0 += to_f32(src[key_d_offset(c)]);
                            s1 += to_f32(src[key_d_offset(c + hd / 2)]);
                        }
                        bf16_t* dst = ckpool + ck_index(page, (first % pv.page_size) / ck_stride, kvh, nkv, hd, rpp);
                        dst[ck_d_offset(c, rpp)] = f32_to_bf16((s0 + own[t][T][j][0]) / (float)ck_size);
                        dst[ck_d_offset(c + hd / 2, rpp)] = f32_to_bf16((s1 + own[t][T][j][1]) / (float)ck_size);
                    }
            }
        }
    }
}

// Rows a workgroup owns for a weight of `total_rows` rows (even, 16..32): 16, unless that leaves some CUs with
// one workgroup more than the others and a few more rows each even that out.
extern "C" int cpmcu_qkv_rope_rows_per_workgroup(int total_rows) {
    static int device_cus = 0;              // asked of the current device once; 256 (the MI355X) if it cannot say
    if (device_cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = 256;
        }
        device_cus = n;
    }
    const int cus = device_cus;
    const int strips = (total_rows + 15) / 16;
    if (strips <= cus || strips % cus == 0) return 16;
    const int rounds = strips / cus;
    const int R = ((total_rows + cus * rounds - 1) / (cus * rounds) + 1) / 2 * 2;
    return R <= 32 ? R : 16;
}

extern "C" const char* cpmcu_qkv_rope(const void* X, long ldx, const void* W, int rows_per_wg, int M, int K, void* q_out,
                                      int nh, int nkv, int hd, const int* positions, const int* tok_slot,
                                      const float* inv_freq, float mscale, void* kpool, void* vpool,
                                      const int* page_table, int table_width, int page_size, const float* row_ss,
                                      int ss_slices, float eps, void* ckpool, int ck_size, int ck_stride, hipStream_t stream) {
    CPMCU_REQUIRE(M > 0 && M <= 64, "qkv_rope: %d tokens (1..64 are taken; more go through the split product and the rotary kernel)", M);
    CPMCU_REQUIRE(nh > 0 && nkv > 0 && hd > 0 && hd % 16 == 0, "qkv_rope: bad shape heads=%d kv_heads=%d head_dim=%d", nh, nkv, hd);
    CPMCU_REQUIRE(K > 0 && K % 8 == 0 && ldx % 8 == 0 && ldx >= K, "qkv_rope: K=%d, row stride %ld must be multiples of 8", K, ldx);
    CPMCU_REQUIRE(((uintptr_t)X % 16 == 0) && ((uintptr_t)W % 16 == 0), "qkv_rope: operands must be 16-byte aligned");
    CPMCU_REQUIRE(q_out && kpool && vpool && page_table && positions && tok_slot, "qkv_rope: null pointer");
    CPMCU_REQUIRE(page_size % 32 == 0, "qkv_rope: a cache page of %d tokens is not a multiple of 32", page_size);
    CPMCU_REQUIRE(!ckpool || (ck_stride > 0 && ck_size >= ck_stride && page_size % ck_stride == 0),
                  "qkv_rope: kernel_stride %d must divide the cache page of %d tokens (kernel_size %d)", ck_stride,
                  page_size, ck_size);
    const int R = rows_per_wg;
    CPMCU_REQUIRE(R >= 16 && R <= 32 && R % 2 == 0, "qkv_rope: %d rows a workgroup (an even number from 16 to 32)", R);
    PagedView pv{page_table, table_width, page_size};
    const int total_rows = (nh + 2 * nkv) * hd;
    const int wgs = (total_rows + R - 1) / R;
#define LAUNCH(PFv, MTv, TLv)                                                                                    \
    qkv_rope_kernel<PFv, 4, MTv, TLv><<<wgs, 256, 0, stream>>>((const bf16_t*)X, ldx, (const bf16_t*)W, M, K, R,  \
                                                           (bf16_t*)q_out,                                           \
                                                           nh, nkv, hd, positions, tok_slot, inv_freq, mscale,       \
                                                           (bf16_t*)kpool, (bf16_t*)vpool, pv, row_ss, ss_slices, eps, \
                                                           (bf16_t*)ckpool, ck_size, ck_stride)
    // more tokens hold more of x in registers for every block in flight: fewer blocks then
    if (R == 16) {
        if (M <= 16) LAUNCH(4, 1, 1);
        else if (M <= 32) LAUNCH(4, 2, 1);
        else LAUNCH(2, 4, 1);
    } else {
        if (M <= 16) LAUNCH(4, 1, 2);
        else if (M <= 32) LAUNCH(2, 2, 2);
        else LAUNCH(2, 4, 2);
    }
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("qkv_rope");
    return nullptr;
}
