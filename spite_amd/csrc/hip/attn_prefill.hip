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

#define PF_COLS 256        // columns (query, head) per workgroup
#define PF_KEYS 64         // keys per block

template <int HD>
__global__ __launch_bounds__(512)
void attn_prefill_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages,
                         const bf16* __restrict__ v_pages, bf16* __restrict__ out,
                         const int* __restrict__ positions, const int* __restrict__ cu_seqlens, int n_seqs,
                         const int* __restrict__ block_table, int max_blocks, int tile_q,
                         int H, int G, int ps, int vis, int span, float scale_log2e) {
    constexpr int NC = HD / 32, ND = HD / 16;
    constexpr int KCH = PF_KEYS * HD / 8 / 512;      // 16-byte chunks of the K block per thread
    constexpr int VCH = HD * PF_KEYS / 8 / 512;      // and of the V^T block
    constexpr int KHALF = 2 * NC * 64;               // chunks of one 32-key half of a K block
    constexpr int VHALF = ND * 64;                   // and of a V^T block
    extern __shared__ __attribute__((aligned(16))) bf16 sm[];
    bf16* Ks = sm;                                   // [2][half][tile tt][chunk cc][512]
    bf16* Vs = sm + 2 * PF_KEYS * HD;                // [2][half][tile d][512]

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

    // this lane's two columns
    int pq[2], lo[2], tok[2], head[2];
    bf16x8 qf[2][NC];
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    int pq_min = 0x7fffffff, pq_max = -1, lo_min = 0x7fffffff, lo_max = 0;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int col = wave * 32 + c * 16 + n;
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
    auto stage_load = [&](int kb) {
        const int key0 = kb * PF_KEYS;
        const int pg0 = page_of(key0), pg1 = page_of(key0 + 32);
        const int blk0 = (key0 % ps) >> 5, blk1 = ((key0 + 32) % ps) >> 5;     // the 32-key blocks inside their pages
        // pages that are absent are read as page 0: their keys are masked, or poisoned below
        const size_t slab0 = ((size_t)(pg0 < 0 ? 0 : pg0) * G + g) * (size_t)ps * HD;
        const size_t slab1 = ((size_t)(pg1 < 0 ? 0 : pg1) * G + g) * (size_t)ps * HD;
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            const int c = tid + 512 * i;
            const size_t at = c < KHALF ? slab0 + ((size_t)blk0 * KHALF + c) * 8 : slab1 + ((size_t)blk1 * KHALF + (c - KHALF)) * 8;
            kreg[i] = *(const bf16x8*)(k_pages + at);
        }
#pragma unroll
        for (int i = 0; i < VCH; ++i) {
            const int c = tid + 512 * i;
            const size_t at = c < VHALF ? slab0 + ((size_t)blk0 * VHALF + c) * 8 : slab1 + ((size_t)blk1 * VHALF + (c - VHALF)) * 8;
            vreg[i] = *(const bf16x8*)(v_pages + at);
        }
    };
    auto stage_store = [&](int buf) {
#pragma unroll
        for (int i = 0; i < KCH; ++i) *(bf16x8*)(Ks + buf * PF_KEYS * HD + (tid + 512 * i) * 8) = kreg[i];
#pragma unroll
        for (int i = 0; i < VCH; ++i) *(bf16x8*)(Vs + buf * HD * PF_KEYS + (tid + 512 * i) * 8) = vreg[i];
    };

    // ---- one block of 64 keys out of LDS
    auto compute = [&](int kb, int buf) {
        const int key0 = kb * PF_KEYS;
        if (key0 > pq_max || key0 + PF_KEYS - 1 < lo_min) return;     // nothing here for this wave
        const bool whole = key0 >= lo_max && key0 + PF_KEYS - 1 <= pq_min;
        const bool absent0 = page_of(key0) < 0, absent1 = page_of(key0 + 32) < 0;
        const bf16* kb_ = Ks + buf * PF_KEYS * HD + lane * 8;
        const bf16* vb_ = Vs + buf * HD * PF_KEYS + lane * 8;
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
        bf16x8 pf[2][2];
        float alpha[2];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            float mx = -INFINITY;
            // s[c][tt][i] is the key key0 + (tt/2)*32 + qd*8 + (tt%2)*4 + i
            if (whole && !absent0 && !absent1) {
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) { s[c][tt][i] *= scale_log2e; mx = fmaxf(mx, s[c][tt][i]); }
            } else {
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int j = key0 + (tt >> 1) * 32 + qd * 8 + (tt & 1) * 4 + i;
                        const bool ok = j >= lo[c] && j <= pq[c];
                        const bool absent = (tt >> 1) ? absent1 : absent0;
                        const float v = ok ? (absent ? NAN : s[c][tt][i] * scale_log2e) : -INFINITY;
                        s[c][tt][i] = v;
                        mx = fmaxf(mx, v);
                    }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run[c], mx);
            // a column with nothing visible so far keeps m = -inf: its weights are zero, not NaN
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            alpha[c] = exp2f(m_run[c] - m_safe);
            float sum = 0.f;
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float e = exp2f(s[c][tt][i] - m_safe);
                    sum += e;
                    pf[c][tt >> 1][(tt & 1) * 4 + i] = (bf16)e;
                }
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            l_run[c] = l_run[c] * alpha[c] + sum;
            m_run[c] = m_new;
        }
#pragma unroll
        for (int d = 0; d < ND; ++d) {
#pragma unroll
            for (int c = 0; c < 2; ++c) o[c][d] = o[c][d] * alpha[c];
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const bf16x8 vf = *(const bf16x8*)(vb_ + (hh * ND + d) * 512);
#pragma unroll
                for (int c = 0; c < 2; ++c)
                    o[c][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[c][hh], o[c][d], 0, 0, 0);
            }
        }
    };

    stage_load(b_first);
    stage_store(0);
    __syncthreads();
    for (int kb = b_first; kb <= b_last; ++kb) {
        const int buf = (kb - b_first) & 1;
        if (kb < b_last) stage_load(kb + 1);
        compute(kb, buf);
        if (kb < b_last) stage_store(buf ^ 1);
        __syncthreads();
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

// `counts` (host memory): the number of query tokens of each of the step's `n_seqs` requests,
// in the order of `cu_seqlens` (device), whose differences they are.
extern "C" int spite_attn_prefill(const void* q, const void* k_pages, const void* v_pages, void* out,
                                  const int* positions, const int* cu_seqlens, const int* counts, int n_seqs,
                                  const int* block_table, int max_blocks, int H, int G, int hd, int page_size,
                                  int vis, int span, float scale, hipStream_t st) {
    SP_REQUIRE(n_seqs >= 0 && H > 0 && G > 0 && H % G == 0, "attn_prefill: %d query heads over %d kv heads", H, G);
    SP_REQUIRE(H / G <= PF_COLS, "attn_prefill: %d query heads per kv head, at most %d", H / G, PF_COLS);
    SP_REQUIRE(hd == 64 || hd == 128, "attn_prefill: head size %d (this kernel has 64 and 128)", hd);
    SP_REQUIRE(page_size > 0 && page_size % 32 == 0, "attn_prefill: page size %d must be a multiple of 32", page_size);
    SP_REQUIRE(max_blocks > 0, "attn_prefill: bad table width");
    SP_REQUIRE(vis == SP_VIS_FULL || span > 0, "attn_prefill: chunk or window of %d", span);
    SP_REQUIRE(G <= 65535, "attn_prefill: too many kv heads for one launch");
    const int tile_q = PF_COLS / (H / G);
    long n_tiles = 0;
    for (int s = 0; s < n_seqs; ++s) {
        SP_REQUIRE(counts[s] >= 0, "attn_prefill: request %d with %d tokens", s, counts[s]);
        n_tiles += (counts[s] + tile_q - 1) / tile_q;
    }
    if (n_tiles == 0) return 0;
    SP_REQUIRE(n_tiles <= 0x7fffffffL, "attn_prefill: too many tiles");
    const float sl = scale * 1.4426950408889634f;
    dim3 grid((unsigned)n_tiles, G);
    const size_t sh = (size_t)2 * 2 * PF_KEYS * hd * sizeof(bf16);
    static bool allowed[2] = {false, false};     // the kernels ask for more LDS than the default limit
    if (hd == 128) {
        if (!allowed[0]) {
            hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh);
            SP_REQUIRE(e == hipSuccess, "attn_prefill: %zu bytes of LDS refused: %s", sh, hipGetErrorString(e));
            allowed[0] = true;
        }
        attn_prefill_kernel<128><<<grid, 512, sh, st>>>((const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages,
            (bf16*)out, positions, cu_seqlens, n_seqs, block_table, max_blocks, tile_q, H, G, page_size, vis, span, sl);
    } else {
        if (!allowed[1]) {
            hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_kernel<64>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh);
            SP_REQUIRE(e == hipSuccess, "attn_prefill: %zu bytes of LDS refused: %s", sh, hipGetErrorString(e));
            allowed[1] = true;
        }
        attn_prefill_kernel<64><<<grid, 512, sh, st>>>((const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages,
            (bf16*)out, positions, cu_seqlens, n_seqs, block_table, max_blocks, tile_q, H, G, page_size, vis, span, sl);
    }
    SP_LAUNCH_CHECK("attn_prefill");
    return 0;
}
