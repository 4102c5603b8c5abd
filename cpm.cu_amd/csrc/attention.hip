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
// float, out = sum_j p_j v_j; query head h reads kv head h / (nh/nkv).  With head_slopes (one number a query
// head) the score of key j for the query at position p is lowered by slope * (p - j): the seam for position
// encodings that bias scores instead of rotating vectors (the reference has none).
#include "common.h"
#include "no_alloc.h"

#include <mutex>

template <typename T>
__global__ __launch_bounds__(64) void attention_paged_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ kpool, const T* __restrict__ vpool,
    PagedView pv, const int* __restrict__ positions, const int* __restrict__ tok_slot, int nh, int nkv, int hd,
    float scale, const int* __restrict__ sel_blocks, const int* __restrict__ sel_count, int max_sel, int block_size,
    const float* __restrict__ head_slopes) {
    __shared__ float qs[256];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int g = h / (nh / nkv);
    const int pos = positions[t], slot = tok_slot[t];
    const T* qrow = q + ((long)t * nh + h) * hd;
    for (int d = lane; d < hd; d += 64) qs[d] = to_f32(qrow[d]);
    __syncthreads();
    const int nd = (hd + 63) / 64;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    // a position encoding that biases the scores by distance: s_j -= slope[head] * (position - j)
    const float slope = head_slopes ? head_slopes[h] : 0.f;

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
                const T* kr = kpool + key_index(row, g, nkv, hd);
                float dot = 0.f;
                for (int d = 0; d < hd; ++d) dot += qs[d] * to_f32(kr[key_d_offset(d)]);
                s = dot * scale - slope * (float)(pos - j);
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
                const T* vr = vpool + value_index(rj, g, nkv, hd);
                for (int i = 0; i < nd; ++i) {
                    const int d = lane + 64 * i;
                    if (d < hd) acc[i] += pj * to_f32(vr[value_d_offset(d)]);
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
                                             const int* sel_count, int max_sel, int block_size,
                                             const float* head_slopes, hipStream_t stream) {
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
                                                               hd, scale, sel_blocks, sel_count, max_sel, block_size,
                                                               head_slopes);
    else if (dtype == CPMCU_BF16)
        attention_paged_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kpool,
                                                                (const bf16_t*)vpool, pv, positions, tok_slot, nh,
                                                                nkv, hd, scale, sel_blocks, sel_count, max_sel,
                                                                block_size, head_slopes);
    else
        CPMCU_FAIL("attention: unknown dtype %d", dtype);
    CPMCU_LAUNCH_CHECK("attention_plain");
    return nullptr;
}

// ===========================================================================
// bf16 attention on the matrix cores, for prompts and single tokens alike.
//
// One wavefront owns one query token, one kv head and up to 16 of that kv
// head's query heads (the 16:1 grouping of MiniCPM4-8B fills an MFMA tile
// exactly), and a share of that token's keys (split-KV for decode steps, where
// few tokens must fill 256 CUs).  Keys are visited in chunks of 32:
//   S^T = K . Q^T      A = 16 keys x head_dim straight from the cache rows,
//                      B = Q^T held in registers for the whole kernel
//   P^T = exp2(S^T*c - m) in float, per head (a D column), running max/sum
//   O^T += V^T . P^T   A = V^T: 16 d x 32 keys, one 16-byte load a lane
// Keys and values lie in their pages in the order of these operands (key_index, value_index), so every
// operand load of a wavefront is one contiguous KiB.
// The two key tiles of a chunk take keys {8g..8g+3} and {8g+4..8g+7} of every
// group of 8 so that a lane's 8 probabilities are 8 consecutive keys, the order
// the V^T vector has.  With 4 wavefronts a workgroup (decode steps) the wavefronts take
// the workgroup's chunks in turn and merge their running results through LDS at the end.
// Output: out (bf16) when n_splits == 1, else unnormalised partial results
// part_o[token][head][split][d], part_ml[token][head][split] = (max, sum) for
// attention_combine_kernel.
// (reference: src/flash_attn/src/flash_fwd_kernel.h:580-1171 is its kernel of
// one query token x 16 grouped heads; split and combine :1175-1766, :2320-2501)
// ===========================================================================
typedef __bf16 abf16x8_t __attribute__((ext_vector_type(8)));
typedef float afloatx4_t __attribute__((ext_vector_type(4)));

// 2^x for x <= 8 (weights and rescale factors): the bare hardware instruction; results below the
// normal range come out as 0, which is what a weight that small contributes anyway
__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int HD, int NW, int TW>
__global__ __launch_bounds__(NW * TW * 64) void attention_mfma_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, float* __restrict__ part_o, float2* __restrict__ part_ml,
    const bf16_t* __restrict__ kpool, const bf16_t* __restrict__ vtpool, PagedView pv,
    const int* __restrict__ positions, const int* __restrict__ tok_slot, int nh, int nkv, float scale_log2e,
    const int* __restrict__ sel_blocks, const int* __restrict__ sel_count, int max_sel, int block_size, int n_splits,
    int xcd_major, int n_tokens, int last_blocks_first) {
    static_assert(NW == 1 || TW == 1, "either the wavefronts of a workgroup share a token or each has its own");
    constexpr int KSTEPS = (HD + 31) / 32;
    constexpr int DT = HD / 16;
    int t = blockIdx.x, by = blockIdx.y;
    if (xcd_major) {
        // Workgroups are dealt to the 8 XCDs in turn.  For prompts, give each XCD one run of consecutive
        // tokens of one kv head: neighbours read nearly the same keys, so they meet in that XCD's L2.
        const int total = gridDim.x * gridDim.y, per = total / 8;
        const int lin = blockIdx.y * gridDim.x + blockIdx.x;
        const int logical = lin < per * 8 ? (lin % 8) * per + lin / 8 : lin;
        t = logical % gridDim.x;
        by = logical / gridDim.x;
    }
    const int kvh = by % nkv, ht = by / nkv;
    const int split = blockIdx.z;
    // TW > 1: the wavefronts of a workgroup take neighbouring tokens, which visit mostly the same keys at the
    // same time and so meet in the CU's L1
    // (the wavefront's number is the same in all its lanes: saying so keeps what follows from it in scalar registers)
    const int wave_id = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int wave = TW > 1 ? 0 : wave_id;
    if (TW > 1) {
        t = t * TW + wave_id;
        if (t >= n_tokens) return;
    }
    const int lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    const int G = nh / nkv;
    const int head = kvh * G + ht * 16 + n;            // the head this lane's D column belongs to
    const bool head_ok = ht * 16 + n < G;
    const int pos = positions[t], slot = tok_slot[t];

    abf16x8_t qf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        abf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
        const int d = ks * 32 + g * 8;
        if (head_ok && d < HD) v = *(const abf16x8_t*)(q + ((long)t * nh + head) * HD + d);
        qf[ks] = v;
    }

    // which chunks of 32 keys are this workgroup's; its wavefronts take them in turn
    const int* sel = nullptr;
    int total_chunks = pos / 32 + 1;
    int cpb = 1, rot = 0;
    if (sel_count) {
        const int cnt = sel_count[(long)t * nkv + kvh];
        if (cnt >= 0) {
            sel = sel_blocks + ((long)t * nkv + kvh) * max_sel;
            cpb = block_size / 32;
            total_chunks = cnt * cpb;
            // the list's last blocks (the window, which neighbouring tokens share) are visited first
            rot = max(cnt - last_blocks_first, 0) * cpb;
        }
    }
    const int per_split = (total_chunks + n_splits - 1) / n_splits;
    const int c0 = split * per_split, c1 = min(c0 + per_split, total_chunks);

    afloatx4_t acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = afloatx4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    auto chunk_key0 = [&](int c) {
        if (!sel) return c * 32;
        c += rot;
        if (c >= total_chunks) c -= total_chunks;
        return sel[c / cpb] * block_size + (c % cpb) * 32;
    };
    // Where the wavefront's chunks lie is looked up for 64 chunks at a time, one chunk a lane (its first key and
    // its physical chunk of the pool), a batch ahead, and read back lane by lane: the loads of keys and values
    // then wait for no address lookup, and the loop holds no division.
    const int n_mine = c1 > c0 + wave ? (c1 - c0 - wave + NW - 1) / NW : 0;      // chunks of this wavefront
    auto lookup = [&](int kb, int& key0_v, int& pchunk_v) {
        const int kj = kb + lane;
        int k0 = 0, pc = 0;
        if (kj < n_mine) {
            k0 = chunk_key0(c0 + wave + kj * NW);
            pc = (int)(paged_row(pv, slot, k0) >> 5);
        }
        key0_v = k0;
        pchunk_v = pc;
    };
    const long chunk_elems = 32L * HD;
    const int lane_off = (g * 16 + n) * 8;
    const bf16_t* kbase_p = kpool + (long)kvh * chunk_elems + lane_off;
    const bf16_t* vbase_p = vtpool + (long)kvh * chunk_elems + lane_off;
    const long chunk_stride = (long)nkv * chunk_elems;
    // key slot r of tile u is key key0 + r + 4*(r/4) + 4u; a tile lies [d / 8][slot][d % 8]
    auto load_k = [&](int pchunk, abf16x8_t (&kf)[2][KSTEPS]) {
        const bf16_t* kp = kbase_p + pchunk * chunk_stride;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                abf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
                if (ks * 32 + g * 8 < HD) v = *(const abf16x8_t*)(kp + (u * (HD / 8) + ks * 4) * 128);
                kf[u][ks] = v;
            }
        }
    };
    auto load_v = [&](int pchunk, abf16x8_t (&vf)[DT]) {
        const bf16_t* vp = vbase_p + pchunk * chunk_stride;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vf[dt] = *(const abf16x8_t*)(vp + dt * 512);
    };
    // One buffer each for keys and values: the next chunk's keys are asked for as soon as this chunk's scores
    // are issued, its values as soon as this chunk's P.V is, so both arrive behind the other half of the work
    // (and behind the other wavefronts of the SIMD).  The loads stand outside every branch (the last chunk
    // asks for itself once more) so that the waits for them are counted exactly.
    if (n_mine > 0) {
        abf16x8_t kf[2][KSTEPS], vf[DT];
        int key0_c, pchunk_c, key0_x, pchunk_x;
        lookup(0, key0_c, pchunk_c);
        int key0 = __builtin_amdgcn_readlane(key0_c, 0);
        int pchunk = __builtin_amdgcn_readlane(pchunk_c, 0);
        load_k(pchunk, kf);
        load_v(pchunk, vf);
        for (int kb = 0; kb < n_mine; kb += 64) {
            lookup(kb + 64, key0_x, pchunk_x);
            const int lim = min(64, n_mine - kb);
            for (int i = 0; i < lim; ++i) {
                int key0n = i < 63 ? __builtin_amdgcn_readlane(key0_c, (i + 1) & 63) : __builtin_amdgcn_readlane(key0_x, 0);
                int pchunkn = i < 63 ? __builtin_amdgcn_readlane(pchunk_c, (i + 1) & 63)
                                     : __builtin_amdgcn_readlane(pchunk_x, 0);
                if (kb + i + 1 >= n_mine) {
                    key0n = key0;
                    pchunkn = pchunk;
                }
                afloatx4_t st[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    st[u] = afloatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KSTEPS; ++ks)
                        st[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[u][ks], qf[ks], st[u], 0, 0, 0);
                }
                load_k(pchunkn, kf);
                // lane (head n, g): st[u][i] is key key0 + 8g + 4u + i; only a chunk that reaches beyond the
                // token's own position needs the causal mask (a listed block may even lie wholly beyond it)
                if (key0 + 31 > pos) {
#pragma unroll
                    for (int u = 0; u < 2; ++u)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (key0 + 8 * g + 4 * u + e > pos) st[u][e] = -INFINITY;
                }
                float mx = fmaxf(fmaxf(fmaxf(st[0][0], st[0][1]), fmaxf(st[0][2], st[0][3])),
                                 fmaxf(fmaxf(st[1][0], st[1][1]), fmaxf(st[1][2], st[1][3])));
                mx = rows_max(mx);
                // m is kept in units of the exponent: scores times scale*log2(e)
                // The exponent's reference m follows the maximum only when some row's maximum has moved up by
                // more than 8 (weights then reach 2^8 at most, which float sums and bf16 weights take as well
                // as 1): the 16 rows' maxima of random scores move in half of all chunks, by that much almost
                // never after the first, and every move costs a pass over the accumulators.
                const float m_top = fmaxf(m, mx * scale_log2e);
                const bool moved = __builtin_amdgcn_ballot_w64(m_top > m + 8.0f) != 0;
                const float m_new = moved ? m_top : m;
                const float m_ref = m_new == -INFINITY ? 0.f : m_new;      // nothing seen yet: all weights 0
                const float corr = fast_exp2(m - m_ref);
                float rs = 0.f;
                abf16x8_t pb;
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float p = fast_exp2(__builtin_fmaf(st[u][e], scale_log2e, -m_ref));
                        rs += p;
                        pb[u * 4 + e] = (__bf16)p;
                    }
                rs = rows_sum(rs);
                l = l * corr + rs;
                if (moved) {
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[dt][e] *= corr;
                }
                m = m_new;
                // O^T += V^T . P^T ; A operand: lane (d row n, g) holds V^T[d][key0 + 8g .. +8]
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pb, acc[dt], 0, 0, 0);
                load_v(pchunkn, vf);
                key0 = key0n;
                pchunk = pchunkn;
            }
            key0_c = key0_x;
            pchunk_c = pchunk_x;
        }
    }

    if (NW > 1) {
        // merge the wavefronts' running results: wavefront w then finishes the d tiles w, w+NW, ...
        __shared__ float ml_s[NW][16][2];
        __shared__ float acc_s[NW * DT * 4 * 64];
        if (g == 0) {
            ml_s[wave][n][0] = m;
            ml_s[wave][n][1] = l;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc_s[((wave * DT + dt) * 4 + i) * 64 + lane] = acc[dt][i];
        __syncthreads();
        float m_all = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; ++w)
            if (ml_s[w][n][1] > 0.f) m_all = fmaxf(m_all, ml_s[w][n][0]);
        float l_all = 0.f;
        float sw[NW];
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            sw[w] = ml_s[w][n][1] > 0.f ? exp2f(ml_s[w][n][0] - m_all) : 0.f;
            l_all += sw[w] * ml_s[w][n][1];
        }
        m = m_all;
        l = l_all;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            if (dt % NW != wave) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float a = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) a += sw[w] * acc_s[((w * DT + dt) * 4 + i) * 64 + lane];
                acc[dt][i] = a;
            }
        }
    }
    if (!head_ok) return;
    // lane (head n, g): acc[dt][i] is O[head][dt*16 + 4g + i]; with NW > 1 this wavefront owns d tiles dt % NW == wave
    if (n_splits == 1) {
        const float inv = 1.0f / l;
        bf16_t* o = out + ((long)t * nh + head) * HD;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            if (NW > 1 && dt % NW != wave) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) o[dt * 16 + 4 * g + i] = f32_to_bf16(acc[dt][i] * inv);
        }
    } else {
        const long idx = ((long)t * nh + head) * n_splits + split;
        float* o = part_o + idx * HD;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            if (NW > 1 && dt % NW != wave) continue;
            *(afloatx4_t*)(o + dt * 16 + 4 * g) = acc[dt];
        }
        if (g == 0 && wave == 0) part_ml[idx] = make_float2(m, l);
    }
}

// out[token][head][:] = sum_s 2^(m_s - m) o_s / sum_s 2^(m_s - m) l_s   (splits without keys have l = 0)
// Up to 64 shares: lane s of every wavefront holds share s's (max, sum), so that all of them come back in one
// trip to memory and the common maximum and the denominator are wave reductions; a share's weight is then read
// from its lane (the launcher takes no more than 64 shares).
__device__ inline float share_weight(float w, int s) {       // lane s's w, for a uniform s
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w), s));
}
// HELD > 0: up to HELD shares and one feature a thread: the shares' outputs are asked for before anything
// waits for the (max, sum) pairs, so that both come back in one trip to memory instead of two.
template <int HELD>
__global__ void attention_combine_kernel(const float* __restrict__ part_o, const float2* __restrict__ part_ml,
                                         bf16_t* __restrict__ out, int hd, int n_splits) {
    const long row = blockIdx.x;             // token * nh + head
    const float2* ml = part_ml + row * n_splits;
    const float* po = part_o + row * n_splits * hd;
    const int lane = threadIdx.x & 63;
    float held_o[HELD > 0 ? HELD : 1];
    if (HELD > 0) {
        const int d = min((int)threadIdx.x, hd - 1);
#pragma unroll
        for (int s = 0; s < HELD; ++s) held_o[s] = po[(long)min(s, n_splits - 1) * hd + d];
    }
    float2 v = make_float2(-INFINITY, 0.f);
    if (lane < n_splits) v = ml[lane];
    const bool live = v.y > 0.f;
    const float m = wave_max(live ? v.x : -INFINITY);
    const float wv = live ? exp2f(v.x - m) : 0.f;
    const float inv = 1.0f / wave_sum(wv * v.y);
    if (HELD > 0) {
        float a = 0.f;
#pragma unroll
        for (int s = 0; s < HELD; ++s) a += share_weight(wv, s) * held_o[s];   // lanes >= n_splits hold 0
        if ((int)threadIdx.x < hd) out[row * hd + threadIdx.x] = f32_to_bf16(a * inv);
        return;
    }
    for (int d = threadIdx.x; d < hd; d += blockDim.x) {
        float a = 0.f;
#pragma unroll 8
        for (int s = 0; s < n_splits; ++s) a += share_weight(wv, s) * po[(long)s * hd + d];
        out[row * hd + d] = f32_to_bf16(a * inv);
    }
}

// Checks and launches of the matrix-core attention; part_o / part_ml are the scratch of its shares, wherever
// the caller keeps them.
static const char* attention_mfma_launch(const void* q, void* out, float* part_o, float* part_ml, int n, int nh,
                                         int nkv, int hd, float scale, const void* kpool, const void* vtpool,
                                         const int* page_table, int table_width, int page_size,
                                         const int* positions, const int* tok_slot, const int* sel_blocks,
                                         const int* sel_count, int max_sel, int block_size, int n_splits,
                                         int waves_per_group, int last_blocks_first, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention_mfma: bad shape n=%d heads=%d kv_heads=%d", n, nh, nkv);
    CPMCU_REQUIRE(hd >= 16 && hd <= 128 && hd % 16 == 0,
                  "attention_mfma: head_dim %d has no matrix-core kernel (16, 32, ... 128 have; the plain kernel takes the rest)", hd);
    CPMCU_REQUIRE(page_size % 32 == 0, "attention_mfma: a cache page of %d tokens is not a multiple of 32", page_size);
    CPMCU_REQUIRE(!sel_count || (sel_blocks && max_sel > 0 && block_size > 0 && block_size % 32 == 0),
                  "attention_mfma: key blocks of %d tokens are not a multiple of 32", block_size);
    CPMCU_REQUIRE(n_splits >= 1 && n_splits <= 64 && (n_splits == 1 || (part_o && part_ml)),
                  "attention_mfma: %d shares of the keys (1..64 are taken)", n_splits);
    const int G = nh / nkv;
    const int HT = (G + 15) / 16;
    CPMCU_REQUIRE((long)nkv * HT <= 65535, "attention_mfma: too many head tiles");
    PagedView pv{page_table, table_width, page_size};
    const float sl = scale * 1.4426950408889634f;
    // few tokens (decode steps): 4 wavefronts share a workgroup's keys; many tokens (prompts): a wavefront a
    // token, 4 neighbouring tokens a workgroup
    const int nw = waves_per_group > 0 ? waves_per_group : (n <= 256 ? 4 : 1);
    CPMCU_REQUIRE(nw == 1 || nw == 4, "attention_mfma: %d wavefronts a workgroup (1 or 4 are built)", nw);
    const int tw = nw == 1 && n_splits == 1 && n >= 64 ? 4 : 1;
    const int xcd_major = tw > 1 ? 1 : 0;
    dim3 grid((n + tw - 1) / tw, nkv * HT, n_splits);
#define LAUNCH(HDv, NWv, TWv)                                                                                      \
    attention_mfma_kernel<HDv, NWv, TWv><<<grid, NWv * TWv * 64, 0, stream>>>(                                    \
        (const bf16_t*)q, (bf16_t*)out, part_o, (float2*)part_ml, (const bf16_t*)kpool, (const bf16_t*)vtpool, pv, \
        positions, tok_slot, nh, nkv, sl, sel_blocks, sel_count, max_sel, block_size, n_splits, xcd_major, n,      \
        last_blocks_first)
#define BY_NW(HDv)                            \
    do {                                      \
        if (nw == 4) LAUNCH(HDv, 4, 1);       \
        else if (tw == 4) LAUNCH(HDv, 1, 4);  \
        else LAUNCH(HDv, 1, 1);               \
    } while (0)
    switch (hd) {
        case 16: BY_NW(16); break;
        case 32: BY_NW(32); break;
        case 48: BY_NW(48); break;
        case 64: BY_NW(64); break;
        case 80: BY_NW(80); break;
        case 96: BY_NW(96); break;
        case 112: BY_NW(112); break;
        default: BY_NW(128); break;
    }
#undef BY_NW
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("attention_mfma");
    if (n_splits > 1) {
        const unsigned rows = (unsigned)((long)n * nh), threads = hd > 64 ? 128 : 64;     // threads >= hd
#define COMBINE(HELDv) attention_combine_kernel<HELDv><<<rows, threads, 0, stream>>>( \
            part_o, (const float2*)part_ml, (bf16_t*)out, hd, n_splits)
        if (n_splits <= 8) COMBINE(8);
        else if (n_splits <= 16) COMBINE(16);
        else if (n_splits <= 32) COMBINE(32);
        else COMBINE(0);
#undef COMBINE
        CPMCU_LAUNCH_CHECK("attention_combine");
    }
    return nullptr;
}

extern "C" const char* cpmcu_attention_mfma(const void* q, void* out, float* part_o, float* part_ml, int n, int nh,
                                            int nkv, int hd, float scale, const void* kpool, const void* vtpool,
                                            const int* page_table, int table_width, int page_size,
                                            const int* positions, const int* tok_slot, const int* sel_blocks,
                                            const int* sel_count, int max_sel, int block_size, int n_splits,
                                            int waves_per_group, int last_blocks_first, hipStream_t stream) {
    return attention_mfma_launch(q, out, part_o, part_ml, n, nh, nkv, hd, scale, kpool, vtpool, page_table,
                                 table_width, page_size, positions, tok_slot, sel_blocks, sel_count, max_sel,
                                 block_size, n_splits, waves_per_group, last_blocks_first, stream);
}

// ---------------------------------------------------------------------------
// The same attention for callers that cannot allocate (declared in no_alloc.h): the shares of a split-KV
// run lie in an array of the library's own instead of a workspace the caller brings.
//
// `static_scratch` is the array; in host code that name is only a stand-in for the symbol, not a device
// address, so the address is asked for once per device (each GPU holds its own copy at its own address) and
// only that pointer is handed to kernels.  Every share's output and (max, sum) pair is written by the
// attention kernel before the merge kernel reads it (a share without keys writes sum 0), so nothing has to
// be cleared between calls.
// ---------------------------------------------------------------------------
static __device__ __align__(256) float static_scratch[CPMCU_STATIC_SCRATCH_FLOATS];

namespace {
constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices];          // per device, set at the first call on that device
std::mutex g_scratch_mutex;

const char* static_scratch_address(float** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) CPMCU_FAIL("attention_mfma_static: hipGetDevice failed: %s", hipGetErrorString(e));
    CPMCU_REQUIRE(dev >= 0 && dev < kMaxDevices, "attention_mfma_static: device %d (0..%d are taken)", dev,
                  kMaxDevices - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch));
        if (e != hipSuccess || !p)
            CPMCU_FAIL("attention_mfma_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = (float*)p;
    }
    *ptr = g_scratch_ptr[dev];
    return nullptr;
}
}  // namespace

extern "C" const char* cpmcu_attention_mfma_static(const void* q, void* out, int n, int nh, int nkv, int hd,
                                                   float scale, const void* kpool, const void* vtpool,
                                                   const int* page_table, int table_width, int page_size,
                                                   const int* positions, const int* tok_slot, const int* sel_blocks,
                                                   const int* sel_count, int max_sel, int block_size, int n_splits,
                                                   int waves_per_group, int last_blocks_first, hipStream_t stream) {
    CPMCU_REQUIRE(n > 0 && nh > 0 && hd > 0 && n_splits >= 1, "attention_mfma_static: bad shape n=%d heads=%d head_dim=%d shares=%d",
                  n, nh, hd, n_splits);
    float* part_o = nullptr;
    float* part_ml = nullptr;
    if (n_splits > 1) {
        // shares' outputs [n][heads][shares][hd], then their (max, sum) pairs [n][heads][shares][2]
        const long rows = (long)n * nh * n_splits;
        const long need = rows * hd + rows * 2;
        CPMCU_REQUIRE(need <= (long)CPMCU_STATIC_SCRATCH_FLOATS,
                      "attention_mfma_static: %d tokens x %d heads x %d shares x (head_dim %d + 2) = %ld floats of "
                      "shares exceed the library's own scratch of %ld floats (%ld MiB); use fewer shares or tokens, "
                      "or cpmcu_attention_mfma with a workspace",
                      n, nh, n_splits, hd, need, (long)CPMCU_STATIC_SCRATCH_FLOATS,
                      (long)CPMCU_STATIC_SCRATCH_FLOATS * 4 / (1 << 20));
        float* base = nullptr;
        if (const char* err = static_scratch_address(&base)) return err;
        part_o = base;
        part_ml = base + rows * hd;
    }
    return attention_mfma_launch(q, out, part_o, part_ml, n, nh, nkv, hd, scale, kpool, vtpool, page_table,
                                 table_width, page_size, positions, tok_slot, sel_blocks, sel_count, max_sel,
                                 block_size, n_splits, waves_per_group, last_blocks_first, stream);
}

// ===========================================================================
// bf16 attention for prompts on the matrix cores (dense, causal).
//
// One wavefront owns R row tiles of 16 rows for one kv head: a row is one
// (token, query head) pair, a tile holds the grouped heads of one token (or of
// several tokens when the group is smaller than 16), and the tokens of a
// wavefront are consecutive positions of one sequence.  For every chunk of 32
// keys the K and V^T operands are loaded once and used by all R tiles, which
// divides the cache traffic of a prompt by the tokens a wavefront holds.  The
// arithmetic of a tile is that of attention_mfma_kernel; the causal mask is per
// row, and a tile is skipped for chunks that lie behind all of its rows.
// `tiles` holds, per wavefront, the first packed token and the number of tokens.
// ===========================================================================
template <int HD, int R, int NW>
__global__ __launch_bounds__(NW * 64) void attention_prefill_mfma_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ kpool,
    const bf16_t* __restrict__ vtpool, PagedView pv, const int* __restrict__ tiles,
    const int* __restrict__ positions, const int* __restrict__ tok_slot, int nh, int nkv, float scale_log2e,
    int rows_per_token, int tokens_per_tile) {
    constexpr int KSTEPS = (HD + 31) / 32;
    constexpr int DT = HD / 16;
    const int tile_id = gridDim.x - 1 - blockIdx.x;      // later tiles of a prompt see more keys: start them first
    const int kvh = blockIdx.y % nkv, ht = blockIdx.y / nkv;
    // (the wavefront's number is the same in all its lanes: saying so keeps what follows from it in scalar registers)
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    const int G = nh / nkv;
    const int t0 = tiles[2 * tile_id], n_tok = tiles[2 * tile_id + 1];
    const int slot = tok_slot[t0];
    const int* ptab = pv.page_table + (long)slot * pv.table_width;
    const int pos0 = positions[t0];

    // this lane's row in each tile: token and head; rows beyond the tile's tokens repeat its first token
    int row_tok[R], row_pos[R], row_head[R];
    bool row_ok[R];
    int tile_last_pos[R], tile_first_pos[R];
    abf16x8_t qf[R][KSTEPS];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int tk = r * tokens_per_tile + n / rows_per_token;
        const int hh = ht * 16 + n % rows_per_token;        // head inside the group (rows_per_token = min(G,16) or 16)
        const bool ok = tk < n_tok && hh < G && (n / rows_per_token) < tokens_per_tile;
        row_ok[r] = ok;
        row_tok[r] = t0 + (tk < n_tok ? tk : 0);
        row_pos[r] = pos0 + (tk < n_tok ? tk : 0);
        row_head[r] = kvh * G + (hh < G ? hh : 0);
        tile_last_pos[r] = pos0 + min((r + 1) * tokens_per_tile, n_tok) - 1;
        tile_first_pos[r] = pos0 + min(r * tokens_per_tile, n_tok - 1);
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            abf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
            const int d = ks * 32 + g * 8;
            if (d < HD) v = *(const abf16x8_t*)(q + ((long)row_tok[r] * nh + row_head[r]) * HD + d);
            qf[r][ks] = v;
        }
    }
    const int n_tiles_used = (n_tok + tokens_per_tile - 1) / tokens_per_tile;
    const int last_pos = pos0 + n_tok - 1;
    const int total_chunks = last_pos / 32 + 1;

    afloatx4_t acc[R][DT];
    float m[R], l[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        m[r] = -INFINITY;
        l[r] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[r][dt] = afloatx4_t{0.f, 0.f, 0.f, 0.f};
    }
    const long chunk_elems = 32L * HD;
    const bf16_t* kbase_p = kpool + (long)kvh * chunk_elems + (g * 16 + n) * 8;
    const bf16_t* vbase_p = vtpool + (long)kvh * chunk_elems + (g * 16 + n) * 8;
    const long chunk_stride = (long)nkv * chunk_elems;
    auto load_k = [&](int pchunk, abf16x8_t (&kf)[2][KSTEPS]) {
        const bf16_t* kp = kbase_p + pchunk * chunk_stride;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                abf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
                if (ks * 32 + g * 8 < HD) v = *(const abf16x8_t*)(kp + (u * (HD / 8) + ks * 4) * 128);
                kf[u][ks] = v;
            }
        }
    };
    auto load_v = [&](int pchunk, abf16x8_t (&vf)[DT]) {
        const bf16_t* vp = vbase_p + pchunk * chunk_stride;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vf[dt] = *(const abf16x8_t*)(vp + dt * 512);
    };
    // the wavefront's chunks in turn: page number and chunk inside the page advance without a division
    const int cpp = pv.page_size / 32;
    int pg_i = wave / cpp, in_pg = wave % cpp;
    const int pg_step = NW / cpp, in_step = NW % cpp;      // (without a branch: the loop's code stays one stretch)
    auto next_pchunk = [&]() {
        in_pg += in_step;
        const int carry = in_pg >= cpp ? 1 : 0;
        in_pg -= carry * cpp;
        pg_i += pg_step + carry;
        return ptab[pg_i] * cpp + in_pg;
    };
    // one buffer each for keys and values: the next chunk's keys are asked for as soon as the last tile's
    // scores are issued, its values as soon as the last tile's P.V is, so both arrive behind other work
    // with NW wavefronts a workgroup the chunks are dealt to them in turn and merged at the end
    abf16x8_t kf[2][KSTEPS], vf[DT];
    if (wave < total_chunks) {
        const int pchunk = ptab[pg_i] * cpp + in_pg;
        load_k(pchunk, kf);
        load_v(pchunk, vf);
    }
    // the three stages of a tile's work on a chunk of keys
    auto scores = [&](int r, afloatx4_t (&st)[2]) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            st[u] = afloatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks)
                st[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[u][ks], qf[r][ks], st[u], 0, 0, 0);
        }
    };
    // MASKED false: the caller knows that every key of the chunk lies before every row of the tile.  The
    // accumulators' rescale (rare: the maximum moved by more than 8) is the caller's: `moved` and `corr` say
    // whether and by what.
    auto weights_of = [&](int r, int key0, const afloatx4_t (&st)[2], bool masked, bool& moved, float& corr) {
        // raw scores; only a chunk that reaches past a row's position needs the causal mask
        float sc[8];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) sc[u * 4 + i] = st[u][i];
        if (masked && key0 + 31 > tile_first_pos[r]) {
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (key0 + 8 * g + 4 * u + i > row_pos[r]) sc[u * 4 + i] = -INFINITY;
        }
        float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])),
                         fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
        mx = rows_max(mx);
        // running maximum in units of scaled scores (scale > 0); a row whose position lies before
        // this chunk sees none of its keys: nothing changes for it
        // the reference follows the maximum only past a move of more than 8 (see attention_mfma_kernel)
        const float m_top = fmaxf(m[r], mx * scale_log2e);
        moved = __builtin_amdgcn_ballot_w64(m_top > m[r] + 8.0f) != 0;
        const float m_new = moved ? m_top : m[r];
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        corr = fast_exp2(m[r] - m_use);
        float rs = 0.f;
        abf16x8_t pb;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float p = fast_exp2(fmaf(sc[j], scale_log2e, -m_use));
            rs += p;
            pb[j] = (__bf16)p;
        }
        rs = rows_sum(rs);
        l[r] = l[r] * corr + rs;
        m[r] = m_new;
        return pb;
    };
    auto rescale = [&](int r, float corr) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[r][dt][i] *= corr;
    };
    auto weights = [&](int r, int key0, const afloatx4_t (&st)[2]) {
        bool moved;
        float corr;
        const abf16x8_t pb = weights_of(r, key0, st, true, moved, corr);
        if (moved) rescale(r, corr);
        return pb;
    };
    auto values = [&](int r, abf16x8_t pb) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            acc[r][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pb, acc[r][dt], 0, 0, 0);
    };
    if constexpr (R == 2) {
        // The scores of a chunk are issued one chunk ahead of their use: while the vector unit turns the
        // current chunk's scores into weights, the matrix cores already multiply the next chunk's keys, and the
        // values' products of one tile run under the other tile's vector work (a wavefront issues in order, and
        // a matrix instruction holds only its own pipe).  A tile that does not see a chunk (the first tile at
        // the last chunk of the second, an unused tile) is computed all the same: the mask leaves it weights of 0.
        if (wave < total_chunks) {
            afloatx4_t s0[2], s1[2];
            scores(0, s0);
            scores(1, s1);
            int pchunk_v = 0;                                  // the chunk whose keys kf holds or awaits
            if (wave + NW < total_chunks) {
                pchunk_v = next_pchunk();
                load_k(pchunk_v, kf);
            }
            int c = wave;
            // The chunks that lie before both tiles' rows and have two more behind them: no mask, no test
            // for the end, so that the matrix instructions and the vector work stand in one stretch of code
            // and are issued in turn (the order is said below: a wavefront issues in order, and a matrix
            // instruction that waits for its pipe holds up the vector instructions behind it).
            const int steady_end = min(total_chunks - 2 * NW, (pos0 + 1) / 32);
            for (; c < steady_end; c += NW) {
                afloatx4_t n0[2], n1[2];
                const int pchunk_next = pchunk_v;
                scores(0, n0);
                scores(1, n1);
                pchunk_v = next_pchunk();
                load_k(pchunk_v, kf);
                bool moved0, moved1;
                float corr0, corr1;
                const abf16x8_t p0 = weights_of(0, c * 32, s0, false, moved0, corr0);
                // 16 matrix instructions among the vector work of one tile's weights
#pragma unroll
                for (int k = 0; k < 16; ++k) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                }
                if (moved0) rescale(0, corr0);
                values(0, p0);
                const abf16x8_t p1 = weights_of(1, c * 32, s1, false, moved1, corr1);
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
                }
                if (moved1) rescale(1, corr1);
                values(1, p1);
                load_v(pchunk_next, vf);
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    s0[u] = n0[u];
                    s1[u] = n1[u];
                }
            }
            for (; c < total_chunks; c += NW) {
                const int key0 = c * 32;
                const bool more = c + NW < total_chunks;
                afloatx4_t n0[2], n1[2];
                const int pchunk_next = pchunk_v;
                if (more) {
                    scores(0, n0);
                    scores(1, n1);
                    if (c + 2 * NW < total_chunks) {
                        pchunk_v = next_pchunk();
                        load_k(pchunk_v, kf);
                    }
                }
                const abf16x8_t p0 = weights(0, key0, s0);
                values(0, p0);
                const abf16x8_t p1 = weights(1, key0, s1);
                values(1, p1);
                if (more) {
                    load_v(pchunk_next, vf);
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        s0[u] = n0[u];
                        s1[u] = n1[u];
                    }
                }
            }
        }
    } else {
        for (int c = wave; c < total_chunks; c += NW) {
            const int key0 = c * 32;
            const bool more = c + NW < total_chunks;
            int pchunkn = 0;
            if (more) pchunkn = next_pchunk();
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const bool active = r < n_tiles_used && key0 <= tile_last_pos[r];
                afloatx4_t st[2];
                if (active) scores(r, st);
                if (r == R - 1 && more) load_k(pchunkn, kf);      // the last tile's scores are issued: keys are free
                if (active) values(r, weights(r, key0, st));
            }
            if (more) load_v(pchunkn, vf);
        }
    }
    if (NW > 1) {
        // wavefronts 1.. hand their running results to wavefront 0, one after the other through one buffer
        __shared__ float ml_s[R][16][2];
        __shared__ float acc_s[R * DT * 4 * 64];
        for (int w = 1; w < NW; ++w) {
            __syncthreads();
            if (wave == w) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    if (g == 0) {
                        ml_s[r][n][0] = m[r];
                        ml_s[r][n][1] = l[r];
                    }
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) acc_s[((r * DT + dt) * 4 + i) * 64 + lane] = acc[r][dt][i];
                }
            }
            __syncthreads();
            if (wave == 0) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const float om = ml_s[r][n][0], ol = ml_s[r][n][1];
                    if (ol > 0.f) {
                        const float m_new = fmaxf(m[r], om);
                        const float sa = l[r] > 0.f ? fast_exp2(m[r] - m_new) : 0.f;
                        const float sb = fast_exp2(om - m_new);
                        l[r] = l[r] * sa + ol * sb;
                        m[r] = m_new;
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                acc[r][dt][i] = acc[r][dt][i] * sa + acc_s[((r * DT + dt) * 4 + i) * 64 + lane] * sb;
                    }
                }
            }
        }
        if (wave != 0) return;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (!row_ok[r]) continue;
        const float inv = 1.0f / l[r];
        bf16_t* o = out + ((long)row_tok[r] * nh + row_head[r]) * HD;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) o[dt * 16 + 4 * g + i] = f32_to_bf16(acc[r][dt][i] * inv);
    }
}

// tokens a wavefront holds: `tiles_per_wave` (2 or 4) tiles of 16 rows
extern "C" int cpmcu_attention_prefill_tokens_per_wave(int nh, int nkv, int tiles_per_wave) {
    const int G = nh / nkv;
    const int rpt = (G < 16 && 16 % G == 0) ? G : 16;
    return tiles_per_wave * (16 / rpt);
}

// tiles: int32 [n_tiles, 2] = (first packed token, tokens) with tokens <= cpmcu_attention_prefill_tokens_per_wave
extern "C" const char* cpmcu_attention_prefill_mfma(const void* q, void* out, int n_tiles, const int* tiles,
                                                    int tiles_per_wave, int waves_per_group, int nh,
                                                    int nkv, int hd, float scale, const void* kpool,
                                                    const void* vtpool, const int* page_table, int table_width,
                                                    int page_size, const int* positions, const int* tok_slot,
                                                    hipStream_t stream) {
    CPMCU_REQUIRE(n_tiles > 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention_prefill: bad shape tiles=%d heads=%d kv_heads=%d", n_tiles, nh, nkv);
    CPMCU_REQUIRE(hd >= 16 && hd <= 128 && hd % 16 == 0,
                  "attention_prefill: head_dim %d has no matrix-core kernel (16, 32, ... 128 have)", hd);
    CPMCU_REQUIRE(page_size % 32 == 0, "attention_prefill: a cache page of %d tokens is not a multiple of 32", page_size);
    const int G = nh / nkv;
    const int rpt = (G < 16 && 16 % G == 0) ? G : 16;
    const int tpt = 16 / rpt;
    const int HT = (G + 15) / 16;
    CPMCU_REQUIRE((long)nkv * HT <= 65535, "attention_prefill: too many head tiles");
    PagedView pv{page_table, table_width, page_size};
    dim3 grid(n_tiles, nkv * HT);
    const float sl = scale * 1.4426950408889634f;
    CPMCU_REQUIRE(tiles_per_wave == 2 || tiles_per_wave == 4, "attention_prefill: %d tiles a wavefront (2 or 4 are built)", tiles_per_wave);
    CPMCU_REQUIRE(waves_per_group == 1 || waves_per_group == 2 || waves_per_group == 4,
                  "attention_prefill: %d wavefronts a workgroup (1, 2 or 4 are built)", waves_per_group);
#define LAUNCH(HDv, Rv, NWv)                                                                                     \
    attention_prefill_mfma_kernel<HDv, Rv, NWv><<<grid, NWv * 64, 0, stream>>>(                                  \
        (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)kpool, (const bf16_t*)vtpool, pv, tiles, positions,       \
        tok_slot, nh, nkv, sl, rpt, tpt)
#define BY_R(HDv)                                                               \
    do {                                                                        \
        if (tiles_per_wave == 4 && waves_per_group == 4) LAUNCH(HDv, 4, 4);     \
        else if (tiles_per_wave == 4 && waves_per_group == 2) LAUNCH(HDv, 4, 2); \
        else if (tiles_per_wave == 4) LAUNCH(HDv, 4, 1);                        \
        else if (waves_per_group == 4) LAUNCH(HDv, 2, 4);                       \
        else if (waves_per_group == 2) LAUNCH(HDv, 2, 2);                       \
        else LAUNCH(HDv, 2, 1);                                                 \
    } while (0)
    switch (hd) {
        case 16: BY_R(16); break;
        case 32: BY_R(32); break;
        case 48: BY_R(48); break;
        case 64: BY_R(64); break;
        case 80: BY_R(80); break;
        case 96: BY_R(96); break;
        case 112: BY_R(112); break;
        default: BY_R(128); break;
    }
#undef BY_R
#undef LAUNCH
    CPMCU_LAUNCH_CHECK("attention_prefill_mfma");
    return nullptr;
}
