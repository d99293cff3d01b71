// Prefill attention over the paged cache on MFMA: portions of prompts (and, in a mixed
// step, single decoded tokens beside them) against everything their requests have cached,
// the portion's own keys included (they were written before this kernel runs).
//
// A wave owns 32 consecutive queries of one request and one query head: two column groups
// of 16 queries.  It walks the keys that any of its queries may read in blocks of 32:
//   S^T[keys x queries] = K[keys x hd] . Q^T          (A = K rows as they lie in the page)
//   O^T[hd x queries]  += V^T[hd x keys] . P^T        (A = value page, stored transposed)
// with the softmax running down the columns, as in the decode kernel.  The visibility rule
// (causal, chunk, window) is applied per element from the query's and the key's position.
// Waves do not talk to each other: no LDS, no barriers.  The waves of a workgroup are the
// query heads that share one kv head, on the same queries, so their K and V loads meet in
// the CU's cache.
// Scores, running maximum and sum, and the output are fp32; P is rounded to bf16 only as an
// MFMA operand.
#include "common.h"

template <int HD>
__global__ __launch_bounds__(512)
void attn_prefill_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages,
                         const bf16* __restrict__ v_pages, bf16* __restrict__ out,
                         const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                         const int* __restrict__ cu_seqlens, const int* __restrict__ block_table, int max_blocks,
                         const int* __restrict__ tile_start, int H, int G, int ps, int vis, int span,
                         float scale_log2e, int heads_per_wg) {
    constexpr int NC = HD / 32, ND = HD / 16;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, qd = lane >> 4;
    const int QH = H / G;
    const int rounds = (QH + heads_per_wg - 1) / heads_per_wg;
    const int g = blockIdx.y / rounds;
    const int hq = (blockIdx.y % rounds) * heads_per_wg + wave;      // head within the kv group
    if (hq >= QH) return;
    const int h = g * QH + hq;
    const int t0 = tile_start[blockIdx.x];
    const int seq = seq_of_token[t0];
    const int t_end = cu_seqlens[seq + 1];
    const int* bt = block_table + (size_t)seq * max_blocks;

    // this lane's two queries (column n of group 0 and of group 1)
    int pq[2], lo[2];
    bf16x8 qf[2][NC];
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int t = t0 + c * 16 + n;
        const bool live = t < t_end;
        pq[c] = live ? positions[t] : -1;
        lo[c] = live ? sp_first_visible(pq[c], vis, span) : 0;
#pragma unroll
        for (int cc = 0; cc < NC; ++cc)
            qf[c][cc] = live ? *(const bf16x8*)(q + ((size_t)t * H + h) * HD + cc * 32 + qd * 8) : zero8;
    }
    const int p_first = positions[t0];
    const int t_last = (t0 + 31 < t_end ? t0 + 31 : t_end - 1);
    const int p_last = positions[t_last];
    const int b_first = sp_first_visible(p_first, vis, span) / 32, b_last = p_last / 32;

    float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
    f32x4 o[2][ND];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int d = 0; d < ND; ++d) o[c][d] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int kb = b_first; kb <= b_last; ++kb) {
        const int key0 = kb * 32;
        const int page = bt[key0 / ps];
        const int off0 = key0 % ps;
        const size_t pg = (size_t)(page < 0 ? 0 : page) * G + g;
        const bf16* kbase = k_pages + (pg * ps + off0) * HD;
        const bf16* vbase = v_pages + pg * HD * ps + off0;
        bf16x8 kf[2][NC];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int cc = 0; cc < NC; ++cc)
                kf[tt][cc] = *(const bf16x8*)(kbase + (size_t)(tt * 16 + n) * HD + cc * 32 + qd * 8);
        bf16x8 vf[ND];
#pragma unroll
        for (int d = 0; d < ND; ++d) {
            const bf16x4 a = *(const bf16x4*)(vbase + (size_t)(d * 16 + n) * ps + qd * 4);
            const bf16x4 b = *(const bf16x4*)(vbase + (size_t)(d * 16 + n) * ps + 16 + qd * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) { vf[d][e] = a[e]; vf[d][4 + e] = b[e]; }
        }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            f32x4 s[2];
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                s[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int cc = 0; cc < NC; ++cc)
                    s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[tt][cc], qf[c][cc], s[tt], 0, 0, 0);
            }
            float mx = -INFINITY;
            bool ok[2][4];
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int j = key0 + tt * 16 + qd * 4 + i;
                    ok[tt][i] = j >= lo[c] && j <= pq[c];
                    const float v = ok[tt][i] ? (page < 0 ? NAN : s[tt][i] * scale_log2e) : -INFINITY;
                    s[tt][i] = v;
                    mx = fmaxf(mx, v);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run[c], mx);
            const float alpha = (m_run[c] == -INFINITY) ? 0.f : exp2f(m_run[c] - m_new);
            float sum = 0.f;
            bf16x8 pf;
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float e = ok[tt][i] ? exp2f(s[tt][i] - m_new) : 0.f;
                    sum += e;
                    pf[tt * 4 + i] = (bf16)e;
                }
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            l_run[c] = l_run[c] * alpha + sum;
            m_run[c] = m_new;
#pragma unroll
            for (int d = 0; d < ND; ++d) {
                o[c][d] = o[c][d] * alpha;
                o[c][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[d], pf, o[c][d], 0, 0, 0);
            }
        }
    }
    // o[c][d][i] of lane (n, qd): query t0 + c*16 + n, element d*16 + qd*4 + i
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int t = t0 + c * 16 + n;
        if (t >= t_end) continue;
        const float inv = 1.0f / fmaxf(l_run[c], 1e-30f);
        bf16* orow = out + ((size_t)t * H + h) * HD;
#pragma unroll
        for (int d = 0; d < ND; ++d) {
            bf16x4 w;
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = (bf16)(o[c][d][i] * inv);
            *(bf16x4*)(orow + d * 16 + qd * 4) = w;
        }
    }
}

// `tile_start[i]`: row of q of the first query of tile i; a tile is at most 32 consecutive
// queries of one request.
extern "C" int spite_attn_prefill(const void* q, const void* k_pages, const void* v_pages, void* out,
                                  const int* positions, const int* seq_of_token, const int* cu_seqlens,
                                  const int* block_table, int max_blocks, const int* tile_start, int n_tiles,
                                  int H, int G, int hd, int page_size, int vis, int span, float scale,
                                  hipStream_t st) {
    SP_REQUIRE(n_tiles >= 0 && H > 0 && G > 0 && H % G == 0, "attn_prefill: %d query heads over %d kv heads", H, G);
    SP_REQUIRE(hd == 64 || hd == 128, "attn_prefill: head size %d (this kernel has 64 and 128)", hd);
    SP_REQUIRE(page_size > 0 && page_size % 32 == 0, "attn_prefill: page size %d must be a multiple of 32", page_size);
    SP_REQUIRE(max_blocks > 0, "attn_prefill: bad table width");
    SP_REQUIRE(vis == SP_VIS_FULL || span > 0, "attn_prefill: chunk or window of %d", span);
    if (n_tiles == 0) return 0;
    const int QH = H / G;
    const int per_wg = QH < 8 ? QH : 8;
    const int rounds = (QH + per_wg - 1) / per_wg;
    SP_REQUIRE((long)G * rounds <= 65535, "attn_prefill: too many heads for one launch");
    const float sl = scale * 1.4426950408889634f;
    dim3 grid(n_tiles, G * rounds);
    if (hd == 128)
        attn_prefill_kernel<128><<<grid, per_wg * 64, 0, st>>>((const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages,
            (bf16*)out, positions, seq_of_token, cu_seqlens, block_table, max_blocks, tile_start, H, G, page_size,
            vis, span, sl, per_wg);
    else
        attn_prefill_kernel<64><<<grid, per_wg * 64, 0, st>>>((const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages,
            (bf16*)out, positions, seq_of_token, cu_seqlens, block_table, max_blocks, tile_start, H, G, page_size,
            vis, span, sl, per_wg);
    SP_LAUNCH_CHECK("attn_prefill");
    return 0;
}
