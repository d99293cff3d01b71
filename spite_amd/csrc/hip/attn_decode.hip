// Decode attention over the paged cache on MFMA: one query token per request, the visible
// keys of a request split over workgroups ("split-KV"), partial (max, sum, output) per split
// in fp32, then a small kernel that combines the splits.  (Letting the workgroup that
// finishes last combine them was measured four times slower: making the partial results
// visible across the chip's L2 caches costs more than the second launch.)  With one split the
// output is written at once.
//
// A workgroup serves one token, one kv head and one split; the H/G query heads that share
// the kv head are the 16 columns of the MFMA tiles (unused columns are zero), so K and V are
// read once for all of them.  Its four waves take the split's 32-key blocks in turn.
//   S^T[keys x heads] = K[keys x hd] . Q^T            (A = K rows as they lie in the page)
//   O^T[hd x heads]  += V^T[hd x keys] . P^T          (A = value page, stored transposed)
// The softmax runs down the columns: a lane holds eight keys of one head, the other keys of
// that head sit in the lanes 16, 32 and 48 further on.  The first product leaves lane (n, qd)
// with rows qd*4 .. qd*4+3 of each of its two 16-row tiles, the second wants eight consecutive
// k indices per lane: the rows of the two tiles are therefore the keys qd*8 + i and
// qd*8 + 4 + i of the block (row r of tile tt is key (r/4)*8 + tt*4 + r%4), so that a lane's
// eight probabilities belong to eight consecutive keys and its V^T operand is one 16-byte
// read.  The pages hold keys and values in that operand order (see common.h), tile by tile, so
// that every load of a wave is one kilobyte in a row; the cache is read once, with
// non-temporal loads.
// Scores, running maximum and sum, and the output are fp32; P is rounded to bf16 only as an
// MFMA operand.
#include "common.h"
#include "no_alloc.h"

template <int HD>
__global__ __launch_bounds__(256)
void attn_decode_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages,
                        const bf16* __restrict__ v_pages, float* __restrict__ part, bf16* __restrict__ out,
                        const int* __restrict__ positions, const int* __restrict__ seq_of_token,
                        const int* __restrict__ block_table, int max_blocks, int H, int G, int ps, int vis,
                        int span, float scale_log2e, float cap_ratio, int n_splits,
                        const float* __restrict__ slopes, float inv_scale) {
    constexpr int NC = HD / 32;      // 32-wide chunks of the head for the score product
    constexpr int ND = HD / 16;      // 16-row tiles of the output
    constexpr int ROW = HD + 2;      // partial record: output, max, sum
    extern __shared__ float sm[];    // [4 waves][16 heads][ROW]
    const int split = blockIdx.x, g = blockIdx.y, t = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, qd = lane >> 4;
    const int QH = H / G;
    const int p = positions[t];
    const int lo = sp_first_visible(p, vis, span);
    const int* bt = block_table + (size_t)seq_of_token[t] * max_blocks;
    // a bias slope * (key - query position) on the scaled score of head n, as an addend of the raw score
    const float slope = (slopes && n < QH) ? slopes[g * QH + n] * inv_scale : 0.f;

    const int b_first = lo / 32, b_last = p / 32;
    const int nblk = b_last - b_first + 1;
    const int per = (nblk + n_splits - 1) / n_splits;
    const int rb = b_first + split * per;
    const int re = (rb + per < b_last + 1) ? rb + per : b_last + 1;

    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8 qf[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c)
        qf[c] = n < QH ? *(const bf16x8*)(q + ((size_t)t * H + g * QH + n) * HD + c * 32 + qd * 8) : zero8;

    float m_run = -INFINITY, l_run = 0.f;
    f32x4 o[ND];
#pragma unroll
    for (int d = 0; d < ND; ++d) o[d] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int kb = rb + wave; kb < re; kb += 4) {
        const int key0 = kb * 32;
        const int page = bt[key0 / ps];
        const int off0 = key0 % ps;
        const size_t pg = (size_t)(page < 0 ? 0 : page) * G + g;
        const int blk = off0 >> 5;                                   // the block of 32 keys inside the page
        const bf16* kbase = k_pages + pg * ps * HD + (size_t)blk * 2 * NC * 512 + lane * 8;
        const bf16* vbase = v_pages + pg * HD * ps + (size_t)blk * ND * 512 + lane * 8;
        bf16x8 kf[2][NC];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int c = 0; c < NC; ++c)
                kf[tt][c] = __builtin_nontemporal_load((const bf16x8*)(kbase + (tt * NC + c) * 512));
        bf16x8 vf[ND];
#pragma unroll
        for (int d = 0; d < ND; ++d) vf[d] = __builtin_nontemporal_load((const bf16x8*)(vbase + d * 512));
        if (key0 + 31 > p) {
            // the block that holds the query's own key: the rows behind it still hold what the
            // page's last owner left, and a probability of zero times a value that is not finite
            // is not zero; those values are taken as zero (this lane's keys are key0 + qd*8 + e)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const bool dead = key0 + qd * 8 + e > p;
#pragma unroll
                for (int d = 0; d < ND; ++d) vf[d][e] = dead ? (bf16)0.f : vf[d][e];
            }
        }

        f32x4 s[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
            s[tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NC; ++c)
                s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[tt][c], qf[c], s[tt], 0, 0, 0);
        }
        float mx = -INFINITY;
        bool ok[2][4];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = key0 + qd * 8 + tt * 4 + i;
                ok[tt][i] = j >= lo && j <= p;
                float raw = s[tt][i] + slope * (float)(j - p);
                // a cap on the scores: cap * tanh(score * scale / cap), with cap_ratio = scale / cap
                if (cap_ratio > 0.f) raw = tanhf(raw * cap_ratio) / cap_ratio;
                const float v = ok[tt][i] ? (page < 0 ? NAN : raw * scale_log2e) : -INFINITY;
                s[tt][i] = v;
                mx = fmaxf(mx, v);
            }
        mx = rows4_max(mx);
        const float m_new = fmaxf(m_run, mx);
        const float alpha = (m_run == -INFINITY) ? 0.f : exp2f(m_run - m_new);
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
        sum = rows4_sum(sum);
        l_run = l_run * alpha + sum;
        m_run = m_new;
#pragma unroll
        for (int d = 0; d < ND; ++d) {
            o[d] = o[d] * alpha;
            o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[d], pf, o[d], 0, 0, 0);
        }
    }

    // the four waves' partial results meet in LDS; o[d][i] of lane (n, qd) is O[head n][d*16 + qd*4 + i]
    float* mine = sm + ((size_t)wave * 16 + n) * ROW;
#pragma unroll
    for (int d = 0; d < ND; ++d)
#pragma unroll
        for (int i = 0; i < 4; ++i) mine[d * 16 + qd * 4 + i] = o[d][i];
    if (qd == 0) { mine[HD] = m_run; mine[HD + 1] = l_run; }
    __syncthreads();
    if (n_splits == 1) {                 // nothing to combine: the four waves' sums are the result
        for (int idx = threadIdx.x; idx < QH * HD; idx += 256) {
            const int hn = idx / HD, c = idx % HD;
            float M = -INFINITY;
#pragma unroll
            for (int w = 0; w < 4; ++w) M = fmaxf(M, sm[((size_t)w * 16 + hn) * ROW + HD]);
            float acc = 0.f, L = 0.f;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float mw = sm[((size_t)w * 16 + hn) * ROW + HD];
                const float f = (mw == -INFINITY) ? 0.f : exp2f(mw - M);
                acc += f * sm[((size_t)w * 16 + hn) * ROW + c];
                L += f * sm[((size_t)w * 16 + hn) * ROW + HD + 1];
            }
            out[((size_t)t * H + g * QH + hn) * HD + c] = (bf16)(acc * (1.0f / fmaxf(L, 1e-30f)));
        }
        return;
    }
    for (int idx = threadIdx.x; idx < QH * ROW; idx += 256) {
        const int hn = idx / ROW, c = idx % ROW;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) M = fmaxf(M, sm[((size_t)w * 16 + hn) * ROW + HD]);
        float acc = 0.f;
        if (c == HD) acc = M;
        else {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float mw = sm[((size_t)w * 16 + hn) * ROW + HD];
                const float f = (mw == -INFINITY) ? 0.f : exp2f(mw - M);
                acc += f * sm[((size_t)w * 16 + hn) * ROW + c];   // c == HD+1 sums the l's
            }
        }
        part[(((size_t)t * H + g * QH + hn) * n_splits + split) * ROW + c] = acc;
    }
}

template <int HD>
__global__ __launch_bounds__(HD)
void attn_decode_combine_kernel(const float* __restrict__ part, bf16* __restrict__ out, int H, int n_splits) {
    constexpr int ROW = HD + 2;
    __shared__ float wsh[256];          // weight of every split: exp2(m_s - M)
    __shared__ float linv;
    const int t = blockIdx.x, h = blockIdx.y, c = threadIdx.x;
    const float* rec = part + ((size_t)t * H + h) * n_splits * ROW;
    // the first wave turns the splits' maxima and sums into weights (up to 256 splits, 4 a lane)
    if (c < 64) {
        float ms[4], ls[4];
        float M = -INFINITY;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int s = c + u * 64;
            ms[u] = s < n_splits ? rec[(size_t)s * ROW + HD] : -INFINITY;
            ls[u] = s < n_splits ? rec[(size_t)s * ROW + HD + 1] : 0.f;
            M = fmaxf(M, ms[u]);
        }
        M = wave_max(M);
        float L = 0.f;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int s = c + u * 64;
            const float w = (ms[u] == -INFINITY) ? 0.f : exp2f(ms[u] - M);
            if (s < n_splits) wsh[s] = w;
            L += w * ls[u];
        }
        L = wave_sum(L);
        if (c == 0) linv = 1.0f / fmaxf(L, 1e-30f);
    }
    __syncthreads();
    float acc = 0.f;
#pragma unroll 8
    for (int s = 0; s < n_splits; ++s) acc += wsh[s] * rec[(size_t)s * ROW + c];
    out[((size_t)t * H + h) * HD + c] = (bf16)(acc * linv);
}

// Joins the splits' records [T][H][n_splits][hd + 2] (output not yet divided, maximum, sum) into
// the bf16 output [T][H][hd]; the prefill kernel's splits leave the same records.
int sp_attn_combine(const float* part, void* out, int T, int H, int hd, int n_splits, hipStream_t st) {
    SP_REQUIRE(T >= 0 && H > 0 && H <= 65535 && n_splits >= 1 && n_splits <= 256 && (hd == 64 || hd == 128),
               "attn_combine: T=%d H=%d hd=%d splits=%d", T, H, hd, n_splits);
    if (T == 0) return 0;
    if (hd == 128) attn_decode_combine_kernel<128><<<dim3(T, H), 128, 0, st>>>(part, (bf16*)out, H, n_splits);
    else attn_decode_combine_kernel<64><<<dim3(T, H), 64, 0, st>>>(part, (bf16*)out, H, n_splits);
    SP_LAUNCH_CHECK("attn_combine");
    return 0;
}

// Bytes of fp32 scratch that a call needs.
extern "C" size_t spite_attn_decode_workspace(int T, int H, int hd, int n_splits) {
    return (size_t)T * H * n_splits * (hd + 2) * sizeof(float);
}

extern "C" int spite_attn_decode(const void* q, const void* k_pages, const void* v_pages, void* out, void* workspace,
                                 const int* positions, const int* seq_of_token, const int* block_table,
                                 int max_blocks, int T, int H, int G, int hd, int page_size, int vis, int span,
                                 float scale, float softcap, const float* slopes, int n_splits, hipStream_t st) {
    SP_REQUIRE(softcap >= 0.f && scale > 0.f, "attn_decode: scale %g, score cap %g", scale, softcap);
    SP_REQUIRE(T >= 0 && H > 0 && G > 0 && H % G == 0, "attn_decode: %d query heads over %d kv heads", H, G);
    SP_REQUIRE(H / G <= 16, "attn_decode: %d query heads per kv head, at most 16", H / G);
    SP_REQUIRE(hd == 64 || hd == 128, "attn_decode: head size %d (this kernel has 64 and 128)", hd);
    SP_REQUIRE(page_size > 0 && page_size % 32 == 0, "attn_decode: page size %d must be a multiple of 32", page_size);
    SP_REQUIRE(max_blocks > 0 && n_splits >= 1 && n_splits <= 256, "attn_decode: bad table width, or %d splits (at most 256)", n_splits);
    SP_REQUIRE(vis >= 0 && vis < SP_VIS_COUNT && (!sp_vis_has_span(vis) || span > 0), "attn_decode: chunk or window of %d", span);
    SP_REQUIRE(G <= 65535 && T <= 65535, "attn_decode: too many heads or tokens for one launch");
    if (T == 0) return 0;
    const float sl = scale * 1.4426950408889634f, cr = softcap > 0.f ? scale / softcap : 0.f;
    dim3 grid(n_splits, G, T);
    const size_t sh = (size_t)4 * 16 * (hd + 2) * sizeof(float);
    if (hd == 128) {
        attn_decode_kernel<128><<<grid, 256, sh, st>>>((const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages,
            (float*)workspace, (bf16*)out, positions, seq_of_token, block_table, max_blocks, H, G, page_size, vis, span, sl, cr, n_splits, slopes, 1.0f / scale);
        SP_LAUNCH_CHECK("attn_decode");
        if (n_splits > 1)
            attn_decode_combine_kernel<128><<<dim3(T, H), 128, 0, st>>>((const float*)workspace, (bf16*)out, H, n_splits);
    } else {
        attn_decode_kernel<64><<<grid, 256, sh, st>>>((const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages,
            (float*)workspace, (bf16*)out, positions, seq_of_token, block_table, max_blocks, H, G, page_size, vis, span, sl, cr, n_splits, slopes, 1.0f / scale);
        SP_LAUNCH_CHECK("attn_decode");
        if (n_splits > 1)
            attn_decode_combine_kernel<64><<<dim3(T, H), 64, 0, st>>>((const float*)workspace, (bf16*)out, H, n_splits);
    }
    SP_LAUNCH_CHECK("attn_decode_combine");
    return 0;
}

// ---- the same call for callers that cannot allocate: the partial results go to an array of
// the library's own.  In host code `scratch` is only a handle for hipGetSymbolAddress; the
// address of each GPU's copy is looked up once per device and that pointer is what kernels get.
static __device__ __align__(256) float scratch[SPITE_ATTN_DECODE_STATIC_FLOATS];
enum { SP_MAX_DEVICES = 64 };
static float* g_scratch_ptr[SP_MAX_DEVICES];     // per device, null until its first call
static hipError_t scratch_of_current_device(float** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= SP_MAX_DEVICES) return hipErrorInvalidDevice;
    float* p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (p == nullptr) {
        e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);
    }
    *ptr = p;
    return hipSuccess;
}

extern "C" int spite_attn_decode_static(const void* q, const void* k_pages, const void* v_pages, void* out,
                                        const int* positions, const int* seq_of_token, const int* block_table,
                                        int max_blocks, int T, int H, int G, int hd, int page_size, int vis, int span,
                                        float scale, int n_splits, hipStream_t st) {
    SP_REQUIRE(T >= 0 && H > 0 && (hd == 64 || hd == 128) && n_splits >= 1 && n_splits <= 256,
               "attn_decode_static: T=%d H=%d hd=%d splits=%d", T, H, hd, n_splits);
    const size_t need = n_splits > 1 ? (size_t)T * H * n_splits * (hd + 2) : 0;
    SP_REQUIRE(need <= (size_t)SPITE_ATTN_DECODE_STATIC_FLOATS,
               "attn_decode_static: %zu floats of partial results (T=%d H=%d splits=%d hd=%d) exceed the library's %u; "
               "use fewer splits or spite_attn_decode with a workspace", need, T, H, n_splits, hd,
               (unsigned)SPITE_ATTN_DECODE_STATIC_FLOATS);
    float* ptr = nullptr;
    const hipError_t e = scratch_of_current_device(&ptr);
    SP_REQUIRE(e == hipSuccess && ptr != nullptr, "attn_decode_static: no address for the scratch array: %s",
               hipGetErrorString(e));
    return spite_attn_decode(q, k_pages, v_pages, out, ptr, positions, seq_of_token, block_table, max_blocks, T, H, G,
                             hd, page_size, vis, span, scale, 0.f, nullptr, n_splits, st);
}
