// Prefill attention over the paged cache on MFMA: portions of prompts (and, in a mixed
// step, single decoded tokens beside them) against everything their requests have cached,
// the portion's own keys included (they were written before this kernel runs).
//
// A workgroup of eight waves owns one kv head and a tile of consecutive queries of one
// request, as many as give at most 256 (query, query head) pairs over the H/G heads that
// share the kv head.  A pair is a column; a wave owns 32 columns, two MFMA column groups.
// The keys that any query of the tile may read are walked in blocks of 64.  A block's K rows
// and V^T rows are fetched from the pages once for the workgroup, by all threads together,
// into LDS (double-buffered: the block after the current one is in flight in registers while
// the current one is multiplied, and is stored to the other buffer behind the products; one
// barrier a block).  Every wave forms
//   S^T[keys x columns] = K[keys x hd] . Q^T          (A = K rows from LDS)
//   O^T[hd x columns]  += V^T[hd x keys] . P^T        (A = rows of the transposed value page)
// with the softmax running down the columns.  The visibility rule (causal, chunk, window) is
// applied per element from the column's position and the key's; blocks that every column of
// a wave sees whole skip the tests, blocks that none sees are skipped.
//
// KS = 2 (short prompts, where a tile's walk over its keys is the longest path and there are
// too few tiles to fill the chip): the tile has half the columns, waves 0-3 take them on the
// even blocks of 64 keys and waves 4-7 the same columns on the odd blocks; two blocks are staged
// per step, and at the end the two halves' (maximum, sum, output) meet in LDS.
//
// Order of keys.  The score product leaves lane (n, qd) with rows qd*4 .. qd*4+3 of each
// 16-row tile; the second product wants 8 consecutive k indices per lane.  The rows qd*4+i of
// the two tiles of a 32-key half are therefore the keys qd*8 + i and qd*8 + 4 + i: a lane's
// eight probabilities of a half belong to eight consecutive keys, and its V^T operand is one
// 16-byte read.  The pages hold keys and values in exactly these operand tiles (common.h), one
// kilobyte each in lane order; a block is copied to LDS as it lies, and a wave's operand read
// is 16 bytes per lane in a row, free of bank conflicts.
// Scores, running maximum and sum, and the output are fp32; P is rounded to bf16 only as an
// MFMA operand.
#include "common.h"

#define PF_COLS 256        // columns (query, head) per workgroup (divided by KS)
#define PF_KEYS 64         // keys per block

template <int HD, int KS>
__global__ __launch_bounds__(512)
void attn_prefill_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages,
                         const bf16* __restrict__ v_pages, bf16* __restrict__ out,
                         const int* __restrict__ positions, const int* __restrict__ cu_seqlens, int n_seqs,
                         const int* __restrict__ block_table, int max_blocks, int tile_q,
                         int H, int G, int ps, int vis, int span, float scale_log2e, float cap_ratio) {
    constexpr int NC = HD / 32, ND = HD / 16;
    constexpr int KCH = KS * PF_KEYS * HD / 8 / 512; // 16-byte chunks of the step's K blocks per thread
    constexpr int VCH = KCH;                         // and of its V^T blocks
    constexpr int KHALF = 2 * NC * 64;               // chunks of one 32-key half of a K block
    constexpr int VHALF = ND * 64;                   // and of a V^T block (the same number)
    constexpr int STEP = KS * PF_KEYS * HD;          // elements of the K (or V^T) blocks of one step
    extern __shared__ __attribute__((aligned(16))) bf16 sm[];
    bf16* Ks = sm;                                   // [2 buffers][KS blocks][half][tile tt][chunk cc][512]
    bf16* Vs = sm + 2 * STEP;                        // [2 buffers][KS blocks][half][tile d][512]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, qd = lane >> 4;
    const int QH = H / G, g = blockIdx.y;

    // which request and which of its queries: tiles are counted request by request; tiles
    // late in a request walk the most keys, so the grid starts from the end
    int tile = gridDim.x - 1 - blockIdx.x, seq = -1, t0 = 0, t_end = 0;
    for (int s = 0; s < n_seqs; ++s) {
        const int b = cu_seqlens[s], e = cu_seqlens[s + 1];
        const int nt = (e - b + tile_q - 1) / tile_q;
        if (tile < nt) { seq = s; t0 = b + tile * tile_q; t_end = (t0 + tile_q < e) ? t0 + tile_q : e; break; }
        tile -= nt;
    }
    if (seq < 0) return;
    const int* bt = block_table + (size_t)seq * max_blocks;
    const int p_first = positions[t0], p_last = positions[t_end - 1];
    const int b_first = sp_first_visible(p_first, vis, span) / PF_KEYS, b_last = p_last / PF_KEYS;
    const int wcol = KS == 2 ? (wave & 3) : wave;    // which 32 columns; with KS = 2 waves w and w+4 share them
    const int khalf = KS == 2 ? (wave >> 2) : 0;     // and take the even (0) or the odd (1) blocks

    // this lane's two columns
    int pq[2], lo[2], tok[2], head[2];
    bf16x8 qf[2][NC];
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    int pq_min = 0x7fffffff, pq_max = -1, lo_min = 0x7fffffff, lo_max = 0;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int col = wcol * 32 + c * 16 + n;
        const int tq = col / QH;
        tok[c] = t0 + tq;
        head[c] = g * QH + col % QH;
        const bool live = tok[c] < t_end;
        pq[c] = live ? positions[tok[c]] : -1;
        lo[c] = live ? sp_first_visible(pq[c], vis, span) : 0;
        if (live) {
            pq_min = min(pq_min, pq[c]); pq_max = max(pq_max, pq[c]);
            lo_min = min(lo_min, lo[c]); lo_max = max(lo_max, lo[c]);
        }
#pragma unroll
        for (int cc = 0; cc < NC; ++cc)
            qf[c][cc] = live ? *(const bf16x8*)(q + ((size_t)tok[c] * H + head[c]) * HD + cc * 32 + qd * 8) : zero8;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        pq_min = min(pq_min, __shfl_xor(pq_min, o, 64)); pq_max = max(pq_max, __shfl_xor(pq_max, o, 64));
        lo_min = min(lo_min, __shfl_xor(lo_min, o, 64)); lo_max = max(lo_max, __shfl_xor(lo_max, o, 64));
    }
    // uniform over the wave: scalar registers, so that the tests below are branches
    pq_min = __builtin_amdgcn_readfirstlane(pq_min); pq_max = __builtin_amdgcn_readfirstlane(pq_max);
    lo_min = __builtin_amdgcn_readfirstlane(lo_min); lo_max = __builtin_amdgcn_readfirstlane(lo_max);

    float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
    f32x4 o[2][ND];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int d = 0; d < ND; ++d) o[c][d] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto page_of = [&](int key) { const int i = key / ps; return i < max_blocks ? bt[i] : -1; };

    // ---- staging: thread's chunks of the block, pages -> registers -> LDS
    bf16x8 kreg[KCH], vreg[VCH];
    // step u stages the blocks u*KS .. u*KS + KS-1; every 32-key half comes from its own page
    auto stage_load = [&](int u) {
        size_t base[2 * KS];
#pragma unroll
        for (int h = 0; h < 2 * KS; ++h) {
            const int key = (u * KS) * PF_KEYS + h * 32;
            const int pg = page_of(key);
            // pages that are absent are read as page 0: their keys are masked, or poisoned below
            base[h] = ((size_t)(pg < 0 ? 0 : pg) * G + g) * (size_t)ps * HD + (size_t)((key % ps) >> 5) * (KHALF * 8);
        }
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            const int c = tid + 512 * i;
            const int h = c / KHALF;                 // which half of which block: a constant where KHALF >= 512
            size_t at = base[0];
#pragma unroll
            for (int hh = 1; hh < 2 * KS; ++hh) at = h == hh ? base[hh] : at;
            at += (size_t)(c - h * KHALF) * 8;
            kreg[i] = *(const bf16x8*)(k_pages + at);
            vreg[i] = *(const bf16x8*)(v_pages + at);      // V^T tiles of a half lie where its K tiles do
        }
    };
    auto stage_store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            *(bf16x8*)(Ks + buf * STEP + (tid + 512 * i) * 8) = kreg[i];
            *(bf16x8*)(Vs + buf * STEP + (tid + 512 * i) * 8) = vreg[i];
        }
    };

    // ---- one block of 64 keys out of LDS
    auto compute = [&](int kb, int buf) {
        if (kb < b_first || kb > b_last) return;
        const int key0 = kb * PF_KEYS;
        if (key0 > pq_max || key0 + PF_KEYS - 1 < lo_min) return;     // nothing here for this wave
        const bool whole = key0 >= lo_max && key0 + PF_KEYS - 1 <= pq_min;
        const bool absent0 = page_of(key0) < 0, absent1 = page_of(key0 + 32) < 0;
        const bf16* kb_ = Ks + buf * STEP + khalf * PF_KEYS * HD + lane * 8;
        const bf16* vb_ = Vs + buf * STEP + khalf * PF_KEYS * HD + lane * 8;
        f32x4 s[2][4];
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            bf16x8 kf[NC];
#pragma unroll
            for (int cc = 0; cc < NC; ++cc) kf[cc] = *(const bf16x8*)(kb_ + (tt * NC + cc) * 512);
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                s[c][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int cc = 0; cc < NC; ++cc)
                    s[c][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[cc], qf[c][cc], s[c][tt], 0, 0, 0);
            }
        }
        if (cap_ratio > 0.f) {
            // a cap on the scores: cap * tanh(score * scale / cap), with cap_ratio = scale / cap; the raw
            // score is replaced by the one that the scale below turns into the capped score
            const float inv = 1.0f / cap_ratio;
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) s[c][tt][i] = tanhf(s[c][tt][i] * cap_ratio) * inv;
        }
        bf16x8 pf[2][2];
        float alpha[2];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            // s[c][tt][i] is the key key0 + (tt/2)*32 + qd*8 + (tt%2)*4 + i; keys that the column
            // may not read become -inf, keys of a page that was given back NaN
            if (!(whole && !absent0 && !absent1)) {
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int j = key0 + (tt >> 1) * 32 + qd * 8 + (tt & 1) * 4 + i;
                        const bool ok = j >= lo[c] && j <= pq[c];
                        const bool absent = (tt >> 1) ? absent1 : absent0;
                        s[c][tt][i] = ok ? (absent ? NAN : s[c][tt][i]) : -INFINITY;
                    }
            }
            // the maximum of the raw scores; the scale (positive) goes into the exponent's fma
            float mx = -INFINITY;
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[c][tt][i]);
            mx = rows4_max(mx);
            const float m_new = fmaxf(m_run[c], mx * scale_log2e);
            // a column with nothing visible so far keeps m = -inf: its weights are zero, not NaN
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            alpha[c] = __builtin_amdgcn_exp2f(m_run[c] - m_safe);
            float sum = 0.f;
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float e = __builtin_amdgcn_exp2f(fmaf(s[c][tt][i], scale_log2e, -m_safe));
                    sum += e;
                    pf[c][tt >> 1][(tt & 1) * 4 + i] = (bf16)e;
                }
            sum = rows4_sum(sum);
            l_run[c] = l_run[c] * alpha[c] + sum;
            m_run[c] = m_new;
        }
        // the running maxima move in the first blocks and seldom after: the output is rescaled
        // only when some column of the wave needs it (alpha is exactly 1 otherwise)
        const bool rescale = __any(alpha[0] != 1.0f || alpha[1] != 1.0f);
        // keys behind the last query of the wave may lie behind the request's last position, where
        // the page still holds what its last owner left, and a half of the block whose page the
        // request has given back (the keys below a window's or a chunk's first visible one, where
        // a page is half a block) was read from a page that is somebody else's or nobody's; a
        // probability of zero times a value that is not finite is not zero, so those values are
        // taken as zero (the other keys below a column's first visible one are the request's own,
        // and finite)
        const bool stale = key0 + PF_KEYS - 1 > pq_max || absent0 || absent1;
#pragma unroll
        for (int d = 0; d < ND; ++d) {
            if (rescale) {
#pragma unroll
                for (int c = 0; c < 2; ++c) o[c][d] = o[c][d] * alpha[c];
            }
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                bf16x8 vf = *(const bf16x8*)(vb_ + (hh * ND + d) * 512);
                if (stale) {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        vf[e] = (key0 + hh * 32 + qd * 8 + e > pq_max || (hh ? absent1 : absent0)) ? (bf16)0.f : vf[e];
                }
#pragma unroll
                for (int c = 0; c < 2; ++c)
                    o[c][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[c][hh], o[c][d], 0, 0, 0);
            }
        }
    };

    const int u_first = b_first / KS, u_last = b_last / KS;
    stage_load(u_first);
    stage_store(0);
    __syncthreads();
    for (int u = u_first; u <= u_last; ++u) {
        const int buf = (u - u_first) & 1;
        if (u < u_last) stage_load(u + 1);
        compute(u * KS + khalf, buf);
        if (u < u_last) stage_store(buf ^ 1);
        __syncthreads();
    }

    if (KS == 2) {
        // the odd blocks' results join the even blocks': per lane 2 maxima, 2 sums and the output,
        // laid out [item][wave of the pair][lane] so that a wave's accesses run through the banks
        float* xs = (float*)sm;
        constexpr int ITEMS = 4 + 2 * ND * 4;
        float* mine = xs + ((size_t)wcol * 64 + lane);
        auto at = [&](int item) -> float& { return mine[(size_t)item * 256]; };
        if (khalf == 1) {
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                at(c) = m_run[c]; at(2 + c) = l_run[c];
#pragma unroll
                for (int d = 0; d < ND; ++d)
#pragma unroll
                    for (int i = 0; i < 4; ++i) at(4 + (c * ND + d) * 4 + i) = o[c][d][i];
            }
        }
        __syncthreads();
        if (khalf == 1) return;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const float mb = at(c), lb = at(2 + c);
            const float M = fmaxf(m_run[c], mb);
            const float fa = (m_run[c] == -INFINITY) ? 0.f : exp2f(m_run[c] - M);
            const float fb = (mb == -INFINITY) ? 0.f : exp2f(mb - M);
            l_run[c] = fa * l_run[c] + fb * lb;
#pragma unroll
            for (int d = 0; d < ND; ++d)
#pragma unroll
                for (int i = 0; i < 4; ++i) o[c][d][i] = fa * o[c][d][i] + fb * at(4 + (c * ND + d) * 4 + i);
        }
        (void)ITEMS;
    }

    // o[c][d][i] of lane (n, qd): column c*16 + n of the wave, element d*16 + qd*4 + i
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        if (tok[c] >= t_end) continue;
        const float inv = 1.0f / fmaxf(l_run[c], 1e-30f);
        bf16* orow = out + ((size_t)tok[c] * H + head[c]) * HD;
#pragma unroll
        for (int d = 0; d < ND; ++d) {
            bf16x4 w;
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = (bf16)(o[c][d][i] * inv);
            *(bf16x4*)(orow + d * 16 + qd * 4) = w;
        }
    }
}

template <int HD, int KS>
static int launch_prefill(const void* q, const void* k_pages, const void* v_pages, void* out, const int* positions,
                          const int* cu_seqlens, int n_seqs, const int* block_table, int max_blocks, int tile_q,
                          long n_tiles, int H, int G, int page_size, int vis, int span, float sl, float cr, hipStream_t st) {
    const size_t sh = (size_t)2 * 2 * KS * PF_KEYS * HD * sizeof(bf16);
    static bool allowed = false;          // one flag per instantiation: more LDS than the default limit
    if (!allowed) {
        hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_kernel<HD, KS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh);
        SP_REQUIRE(e == hipSuccess, "attn_prefill: %zu bytes of LDS refused: %s", sh, hipGetErrorString(e));
        allowed = true;
    }
    attn_prefill_kernel<HD, KS><<<dim3((unsigned)n_tiles, G), 512, sh, st>>>((const bf16*)q, (const bf16*)k_pages,
        (const bf16*)v_pages, (bf16*)out, positions, cu_seqlens, n_seqs, block_table, max_blocks, tile_q, H, G, page_size,
        vis, span, sl, cr);
    SP_LAUNCH_CHECK("attn_prefill");
    return 0;
}

// `counts` (host memory): the number of query tokens of each of the step's `n_seqs` requests,
// in the order of `cu_seqlens` (device), whose differences they are.  `key_split`: 0 lets the
// library choose, 1 or 2 force KS.
extern "C" int spite_attn_prefill(const void* q, const void* k_pages, const void* v_pages, void* out,
                                  const int* positions, const int* cu_seqlens, const int* counts, int n_seqs,
                                  const int* block_table, int max_blocks, int H, int G, int hd, int page_size,
                                  int vis, int span, float scale, float softcap, int key_split, hipStream_t st) {
    SP_REQUIRE(softcap >= 0.f && scale > 0.f, "attn_prefill: scale %g, score cap %g", scale, softcap);
    SP_REQUIRE(n_seqs >= 0 && H > 0 && G > 0 && H % G == 0, "attn_prefill: %d query heads over %d kv heads", H, G);
    SP_REQUIRE(H / G <= PF_COLS / 2, "attn_prefill: %d query heads per kv head, at most %d", H / G, PF_COLS / 2);
    SP_REQUIRE(hd == 64 || hd == 128, "attn_prefill: head size %d (this kernel has 64 and 128)", hd);
    SP_REQUIRE(page_size > 0 && page_size % 32 == 0, "attn_prefill: page size %d must be a multiple of 32", page_size);
    SP_REQUIRE(max_blocks > 0, "attn_prefill: bad table width");
    SP_REQUIRE(vis >= 0 && vis < SP_VIS_COUNT && (!sp_vis_has_span(vis) || span > 0), "attn_prefill: chunk or window of %d", span);
    SP_REQUIRE(G <= 65535, "attn_prefill: too many kv heads for one launch");
    SP_REQUIRE(key_split >= 0 && key_split <= 2, "attn_prefill: key split %d", key_split);
    long tiles[3] = {0, 0, 0};
    for (int ks = 1; ks <= 2; ++ks) {
        const int tile_q = PF_COLS / ks / (H / G);
        for (int s = 0; s < n_seqs; ++s) {
            SP_REQUIRE(counts[s] >= 0, "attn_prefill: request %d with %d tokens", s, counts[s]);
            tiles[ks] += (counts[s] + tile_q - 1) / tile_q;
        }
    }
    if (tiles[1] == 0) return 0;
    // few tiles: the longest tile's walk decides the time, so halve it
    if (key_split == 0) key_split = tiles[1] * G < 512 ? 2 : 1;
    SP_REQUIRE(tiles[key_split] <= 0x7fffffffL, "attn_prefill: too many tiles");
    const float sl = scale * 1.4426950408889634f, cr = softcap > 0.f ? scale / softcap : 0.f;
    const int tile_q = PF_COLS / key_split / (H / G);
#define SP_PF(HDV, KSV) launch_prefill<HDV, KSV>(q, k_pages, v_pages, out, positions, cu_seqlens, n_seqs, block_table, \
        max_blocks, tile_q, tiles[KSV], H, G, page_size, vis, span, sl, cr, st)
    if (hd == 128) return key_split == 2 ? SP_PF(128, 2) : SP_PF(128, 1);
    return key_split == 2 ? SP_PF(64, 2) : SP_PF(64, 1);
#undef SP_PF
}
