// Attention over the paged cache, one wave per (token, query head): the plain kernel of the
// true 32-bit path, and of bf16 for head sizes that the MFMA kernels refuse.
//
// The query at position p of its request reads the keys at [first_visible(p), p] through
// the request's block table.  Keys are walked in tiles of 64 that start at first_visible(p),
// so the order of every sum depends on p alone: a token gives the same bits whether it comes
// in a whole prompt, a portion or alone.  Scores, running maximum, running sum and the
// output are fp32; exp is the accurate one.  Options: a smooth cap on the scaled scores, and
// per-head slopes of a bias slope * (key position - query position) added before the cap.
#include "common.h"

#define ATT_MAX_D 8   // head sizes up to 512

template <typename T>
__global__ __launch_bounds__(64)
void attn_generic_kernel(const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                         T* __restrict__ out, const int* __restrict__ positions,
                         const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
                         int max_blocks, int H, int G, int hd, int ps, int vis, int span, float scale, float softcap, int kv_tiled,
                         const float* __restrict__ slopes) {
    extern __shared__ float smem[];
    float* q_sh = smem;                 // [hd]
    float* p_sh = smem + hd;            // [64]
    long long* row_sh = (long long*)(p_sh + 64);   // [64] first element of the kv head's part of each key's page, -1 = none
    int* off_sh = (int*)(row_sh + 64);             // [64] the key's offset in its page
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int g = h / (H / G);
    const int p = positions[t];
    const int* bt = block_table + (size_t)seq_of_token[t] * max_blocks;
    const int lo = sp_first_visible(p, vis, span);
    const float slope = slopes ? slopes[h] : 0.f;      // a bias slope * (key - query position) on the scaled score
    const T* qr = q + ((size_t)t * H + h) * hd;
    for (int c = lane; c < hd; c += 64) q_sh[c] = to_f32<T>(qr[c]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float o[ATT_MAX_D];
#pragma unroll
    for (int u = 0; u < ATT_MAX_D; ++u) o[u] = 0.f;

    for (int j0 = lo; j0 <= p; j0 += 64) {
        const int j = j0 + lane;
        float s = -INFINITY;
        long long row = -1;
        if (j <= p) {
            const int page = bt[j / ps];
            if (page < 0) {
                s = NAN;   // a page that was given back is asked for: poison the result
            } else {
                const long long pg = (long long)page * G + g;
                row = pg * hd * ps;
                const T* kr = k_pages + row;
                float acc = 0.f;
                for (int c = 0; c < hd; ++c) acc = fmaf(q_sh[c], to_f32<T>(kr[sp_k_index(j % ps, c, hd, kv_tiled)]), acc);
                s = acc * scale + slope * (float)(j - p);
                if (softcap > 0.f) s = softcap * tanhf(s / softcap);       // scores capped smoothly at +-softcap
            }
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float alpha = expf(m - m_new);
        const float pj = (j <= p) ? expf(s - m_new) : 0.f;
        l = l * alpha + wave_sum(pj);
        m = m_new;
        __syncthreads();
        p_sh[lane] = pj;
        row_sh[lane] = row;
        off_sh[lane] = j % ps;
        __syncthreads();
        const int n_valid = (p - j0 + 1) < 64 ? (p - j0 + 1) : 64;
#pragma unroll
        for (int u = 0; u < ATT_MAX_D; ++u) {
            const int c = lane + u * 64;
            if (c < hd) {
                float acc = o[u] * alpha;
                for (int jj = 0; jj < n_valid; ++jj) {
                    const long long r = row_sh[jj];
                    const float vv = r >= 0 ? to_f32<T>(v_pages[r + (long long)sp_v_index(c, off_sh[jj], hd, ps, kv_tiled)]) : 0.f;
                    acc = fmaf(p_sh[jj], vv, acc);
                }
                o[u] = acc;
            }
        }
    }
    const float inv = 1.0f / fmaxf(l, 1e-30f);
    T* orow = out + ((size_t)t * H + h) * hd;
#pragma unroll
    for (int u = 0; u < ATT_MAX_D; ++u) {
        const int c = lane + u * 64;
        if (c < hd) orow[c] = from_f32<T>(o[u] * inv);
    }
}

extern "C" int spite_attn_generic(const void* q, const void* k_pages, const void* v_pages, void* out, int dtype,
                                  const int* positions, const int* seq_of_token, const int* block_table,
                                  int max_blocks, int T, int H, int G, int hd, int page_size, int vis, int span,
                                  float scale, float softcap, const float* slopes, int kv_tiled, hipStream_t st) {
    SP_REQUIRE(softcap >= 0.f, "attention: score cap %g", softcap);
    SP_REQUIRE(T >= 0 && H > 0 && G > 0 && H % G == 0, "attention: %d query heads over %d kv heads", H, G);
    SP_REQUIRE(hd > 0 && hd <= 64 * ATT_MAX_D, "attention: head size %d, at most %d", hd, 64 * ATT_MAX_D);
    SP_REQUIRE(page_size > 0 && max_blocks > 0, "attention: bad page size %d or table width %d", page_size, max_blocks);
    SP_REQUIRE(vis >= 0 && vis < SP_VIS_COUNT && (!sp_vis_has_span(vis) || span > 0), "attention: chunk or window of %d", span);
    SP_REQUIRE(H <= 65535, "attention: too many heads");
    SP_REQUIRE(!kv_tiled || (dtype == SP_BF16 && hd % 32 == 0 && page_size % 32 == 0),
               "attention: pages in operand order are bfloat16 with head size %d and page size %d multiples of 32", hd, page_size);
    if (T == 0) return 0;
    dim3 grid(T, H);
    const size_t sh = (size_t)(hd + 64) * sizeof(float) + 64 * sizeof(long long) + 64 * sizeof(int) + 8;
    if (dtype == SP_F32)
        attn_generic_kernel<float><<<grid, 64, sh, st>>>((const float*)q, (const float*)k_pages, (const float*)v_pages,
            (float*)out, positions, seq_of_token, block_table, max_blocks, H, G, hd, page_size, vis, span, scale, softcap, kv_tiled, slopes);
    else if (dtype == SP_BF16)
        attn_generic_kernel<bf16><<<grid, 64, sh, st>>>((const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages,
            (bf16*)out, positions, seq_of_token, block_table, max_blocks, H, G, hd, page_size, vis, span, scale, softcap, kv_tiled, slopes);
    else return sp_fail("attention: unknown dtype %d", dtype);
    SP_LAUNCH_CHECK("attn_generic");
    return 0;
}
