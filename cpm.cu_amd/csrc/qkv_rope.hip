// q, k, v projection of a decode step fused with the rotation and the cache write (bf16, at most 64 tokens).
//
// A decode step is a chain of small kernels, each of which costs a few microseconds whatever it does; this one
// replaces the split-K product + the kernel that summed its partial sums, rotated and stored.
//
// The weight [q heads; k heads; v heads] x hidden is tiled as for the skinny product ([strip of 16 rows]
// [128-column block][i][lane][8], ops.TiledWeight) but with the rows of every q and k head permuted so that
// strip s of a head holds the features 8s .. 8s+7 and their rotation partners hd/2 + 8s .. hd/2 + 8s+7: a
// workgroup that owns one strip then holds both halves of 8 rotation pairs.  v heads keep their order.
//
// One workgroup of 4 wavefronts a strip: the wavefronts take a quarter of the columns each (x straight from
// global memory into the B operand, asked for together with the weight's block), add their results through LDS, and the
// first wavefront rotates and writes: queries to q_out [token][head][d], keys and values into the cache pages
// in the matrix cores' order (common.h: key_index, value_index).
// theta = pos * inv_freq[c]; (a, b) = (x[c], x[c+hd/2]) -> (a cos - b sin, a sin + b cos), cos and sin times
// `mscale` (reference: src/model/rotary.cuh:7-34; cache rows src/model/attn.cuh:14-21; the fused decode
// projection src/model/minicpm4/minicpm4_attn.cuh:209-223).
#include "common.h"

typedef __bf16 qbf16x8_t __attribute__((ext_vector_type(8)));
typedef float qfloatx4_t __attribute__((ext_vector_type(4)));

// PF: 128-column blocks of the weight a wavefront keeps in flight; NW: wavefronts a workgroup; MT: tiles of 16 tokens
template <int PF, int NW, int MT>
__global__ __launch_bounds__(NW * 64) void qkv_rope_kernel(
    const bf16_t* __restrict__ X, long ldx, const bf16_t* __restrict__ W, int M, int K, bf16_t* __restrict__ q_out,
    int nh, int nkv, int hd, const int* __restrict__ positions, const int* __restrict__ tok_slot,
    const float* __restrict__ inv_freq, float mscale, bf16_t* __restrict__ kpool, bf16_t* __restrict__ vpool,
    PagedView pv, const float* __restrict__ row_ss, int ss_slices, float eps, bf16_t* __restrict__ ckpool,
    int ck_size, int ck_stride) {
    __shared__ float red[NW - 1][MT][4][64];
    __shared__ float rs_s[MT * 16];            // the norm's row factors (common.h: row_scales), if x lacks them
    const int strip = blockIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int nkb = (K + 127) / 128;
    const int per_wave = (nkb + NW - 1) / NW;
    const int kb0 = wave * per_wave, kb1 = min(kb0 + per_wave, nkb);
    const bf16_t* wp = W + (long)strip * nkb * 2048 + lane * 8;
    const bf16_t* xp[MT];                                  // rows beyond the step repeat its last token
#pragma unroll
    for (int t = 0; t < MT; ++t) xp[t] = X + (long)min(t * 16 + r, M - 1) * ldx;

    // Loads return in the order of their issue, so the x of a block is asked for together with its w, PF blocks
    // ahead (asked for only at its use, it would make the wavefront wait for every w behind it: one trip to
    // memory a block).  No load stands in a branch that depends on data: addresses are clamped instead (a block
    // beyond the wavefront's last repeats it and is not multiplied; columns beyond K repeat the row's last 8
    // and meet the weight's zero padding), so the waits count exactly.
    qbf16x8_t a[PF][4], bx[PF][MT][4];
    auto load_block = [&](int kb, qbf16x8_t (&wd)[4], qbf16x8_t (&xd)[MT][4]) {
        const int kbc = min(kb, nkb - 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) wd[i] = __builtin_nontemporal_load((const qbf16x8_t*)(wp + ((long)kbc * 4 + i) * 512));
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) xd[t][i] = *(const qbf16x8_t*)(xp[t] + min(kbc * 128 + i * 32 + g * 8, K - 8));
    };
    qfloatx4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = qfloatx4_t{0.f, 0.f, 0.f, 0.f};
    // what the end needs (positions, the tokens' cache rows through two dependent lookups, the pairs'
    // frequencies) is asked for first: it is there when the products are, instead of costing three trips to
    // memory after them
    const int spt = hd / 16;                       // strips a head
    const int head = strip / spt, s = strip - head * spt;
    int tok_pos[MT];
    long tok_row[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int tok = min(t * 16 + r, M - 1);
        tok_pos[t] = positions[tok];
        tok_row[t] = head >= nh ? paged_row(pv, tok_slot[tok], tok_pos[t]) : 0;
    }
    float freq[4] = {0.f, 0.f, 0.f, 0.f};
    if (inv_freq && head < nh + nkv) {
#pragma unroll
        for (int i = 0; i < 4; ++i) freq[i] = inv_freq[8 * s + 4 * (g & 1) + i];
    }
    auto multiply = [&](qbf16x8_t (&wd)[4], qbf16x8_t (&xd)[MT][4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wd[i], xd[t][i], acc[t], 0, 0, 0);
    };
#pragma unroll
    for (int j = 0; j < PF; ++j) load_block(kb0 + j, a[j], bx[j]);
    // the pairs' cosines and sines are formed while the first blocks are on their way
    float rot_cs[MT][4], rot_sn[MT][4];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            rot_cs[t][i] = 1.f;
            rot_sn[t][i] = 0.f;
            if (inv_freq && head < nh + nkv) {
                const float ang = (float)tok_pos[t] * freq[i];
                rot_cs[t][i] = cosf(ang) * mscale;
                rot_sn[t][i] = sinf(ang) * mscale;
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
    // lane (token r, g) of tile t: acc[t][i] is feature row 4g + i of the strip; the other wavefronts hand theirs
    // to the first
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
        if (row_ss) {          // X was x * w of a norm whose row factor comes now
            const float rs = rs_s[t * 16 + r];
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[t][i] *= rs;
        }
    }

    float own[MT][4];                              // a key head's values as the cache holds them
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int tok = t * 16 + r;
        const bool tok_ok = tok < M;
        const int pos = tok_pos[t];
        if (head < nh + nkv) {
            // rows 0..7 of the strip are d = 8s .. 8s+7, rows 8..15 their partners d + hd/2: lanes g and g+2 hold
            // a pair; after the swap every lane has both (the first half of the wavefront's value, then the second's)
            float lo[4], hi[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const cpmcu_u32x2_t sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[t][i]),
                                                                          __float_as_uint(acc[t][i]), false, false);
                lo[i] = __uint_as_float(sw[0]);
                hi[i] = __uint_as_float(sw[1]);
            }
            const bool second = g >= 2;
            const bool is_q = head < nh;
            bf16_t* dst = nullptr;
            if (tok_ok) {
                if (is_q) dst = q_out + ((long)tok * nh + head) * hd;
                else dst = kpool + key_index(tok_row[t], head - nh, nkv, hd);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = 8 * s + 4 * (g & 1) + i;             // index of the pair
                const float cs = rot_cs[t][i], sn = rot_sn[t][i];
                const float v = second ? lo[i] * sn + hi[i] * cs : lo[i] * cs - hi[i] * sn;
                const int d = second ? c + hd / 2 : c;
                const bf16_t vb = f32_to_bf16(v);
                own[t][i] = to_f32(vb);
                if (tok_ok) dst[is_q ? d : key_d_offset(d)] = vb;
            }
        } else if (tok_ok) {
            bf16_t* dst = vpool + value_index(tok_row[t], head - nh - nkv, nkv, hd);
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[value_d_offset(16 * s + 4 * g + i)] = f32_to_bf16(acc[t][i]);
        }
    }

    // Compressed keys (sparse.hip: compress_keys_kernel, the same sums in the same order): the token at position
    // p completes the mean of the keys p+1-ck_size .. p when p+1-ck_size is a non-negative multiple of ck_stride.
    // This workgroup wrote its 16 features of all the step's keys itself; the fence makes them readable, and
    // is paid only in the steps in which a token completes one.
    if (ckpool && head >= nh && head < nh + nkv) {
        const int kvh = head - nh;
        const int d0 = 8 * s + 4 * (g & 1) + (g >= 2 ? hd / 2 : 0);        // this lane's 4 features
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
                float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
                for (int k = 0; k < ck_size - 1; ++k) {
                    const uint2 u = *(const uint2*)(kpool + key_index(paged_row(pv, slot, first + k), kvh, nkv, hd) +
                                                    key_d_offset(d0));
                    sum[0] += __uint_as_float(u.x << 16);
                    sum[1] += __uint_as_float(u.x & 0xffff0000u);
                    sum[2] += __uint_as_float(u.y << 16);
                    sum[3] += __uint_as_float(u.y & 0xffff0000u);
                }
                uint32_t o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = f32_to_bf16((sum[i] + own[t][i]) / (float)ck_size).v;
                const int page = pv.page_table[(long)slot * pv.table_width + first / pv.page_size];
                const int rpp = pv.page_size / ck_stride;
                bf16_t* dst = ckpool + ck_index(page, (first % pv.page_size) / ck_stride, kvh, nkv, hd, rpp) +
                              ck_d_offset(d0, rpp);
                *(uint2*)dst = make_uint2(o[0] | (o[1] << 16), o[2] | (o[3] << 16));
            }
        }
    }
}

extern "C" const char* cpmcu_qkv_rope(const void* X, long ldx, const void* W, int M, int K, void* q_out, int nh,
                                      int nkv, int hd, const int* positions, const int* tok_slot,
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
    PagedView pv{page_table, table_width, page_size};
    const int strips = (nh + 2 * nkv) * (hd / 16);
#define LAUNCH(PFv, MTv)                                                                                         \
    qkv_rope_kernel<PFv, 4, MTv><<<strips, 256, 0, stream>>>((const bf16_t*)X, ldx, (const bf16_t*)W, M, K, (bf16_t*)q_out, \
                                                           nh, nkv, hd, positions, tok_slot, inv_freq, mscale,       \
                                                           (bf16_t*)kpool, (bf16_t*)vpool, pv, row_ss, ss_slices, eps, \
                                                           (bf16_t*)ckpool, ck_size, ck_stride)
    // more tokens hold more of x in registers for every block in flight: fewer blocks then
    if (M <= 16) LAUNCH(4, 1);
    else if (M <= 32) LAUNCH(4, 2);
    else LAUNCH(2, 4);
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("qkv_rope");
    return nullptr;
}
