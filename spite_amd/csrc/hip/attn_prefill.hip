// Prefill attention over the paged cache on MFMA: portions of prompts (and, in a mixed
// step, single decoded tokens beside them) against everything their requests have cached,
// the portion's own keys included (they were written before this kernel runs).
//
// A workgroup of eight waves owns one kv head and a tile of consecutive queries of one
// request, as many as give at most 256 (query, query head) pairs over the H/G heads that
// share the kv head.  A pair is a column; a wave owns 32 columns, the N side of the
// 32x32x16 MFMA.  The keys that any query of the tile may read are walked in steps of 128.
// A step's K tiles and V^T tiles go from the pages straight into LDS (loads that write
// LDS, no trip through registers), double-buffered: the step after the current one is in
// flight while the current one is multiplied; one barrier a step.  Every wave takes the
// step's four runs of 32 keys in turn and forms
//   S^T[keys x columns] = K[keys x hd] . Q^T          (A = K rows from LDS, B = Q in registers)
//   O^T[hd x columns]  += V^T[hd x keys] . P^T        (A = rows of the transposed value page)
// with the softmax running down the columns: lanes l and l+32 hold a column, 16 keys of a
// run each.
//
// Three kinds of runs, chosen per wave by branches on wave-uniform values:
//   * runs that every column of the wave reads whole (most of a long context): no tests
//     per element, the cheapest path;
//   * runs at an edge (the causal diagonal, the first visible key of a chunk or a window,
//     the end of the request's keys, a page that was given back): the visibility rule is
//     applied per element, values that the request does not own are taken as zero;
//   * runs that no column of the wave reads: skipped.
// Optional per-head slopes (a score bias slope * (key - query position)) and a smooth cap on
// the scores take the per-element path in an instantiation of their own.
//
// Splits.  When the tiles are too few to fill the chip, or fill it unevenly (a long context
// behind a short portion: every tile walks the same many keys, and 328 tiles on 256 compute
// units take two rounds where 1.3 would do), a tile's steps are dealt to `n_splits`
// workgroups; each leaves (output, maximum, sum) of its part in fp32 and a second kernel
// joins them.
//
// Order of keys.  The pages hold keys and values in operand tiles of one kilobyte (common.h):
// a K tile is 16 rows x 32 head elements, row r of tile tt of a 32-key run being the key
// (r/4)*8 + tt*4 + r%4; a V^T tile is 16 head elements x 32 keys.  The 32x32x16 product takes
// two such tiles as its 32 rows.  Its result leaves lane (n, hh) with rows 8j + 4hh + i
// (j, i = 0..3) of column n, which are the keys (hh + 2(j&1))*8 + (j>>1)*4 + i of the run: a
// lane's values j = 0, 2 are the eight consecutive keys 8hh.. of the run's first 16 keys, its
// values j = 1, 3 those of the second 16: exactly the B operand (8 consecutive k per lane) of
// the two products with V^T, with no exchange between lanes.
// Scores, running maximum and sum, and the output are fp32; P is rounded to bf16 only as an
// MFMA operand.
#include "common.h"
#include <type_traits>

#define PF_COLS 256        // columns (query, head) per workgroup
#define PF_KEYS 128        // keys per step
#define PF_RUNS (PF_KEYS / 32)

// EXTRA: score slopes or a cap are in use (every run takes the per-element path)
template <int HD, bool EXTRA>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attn_prefill_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages,
                         const bf16* __restrict__ v_pages, bf16* __restrict__ out, float* __restrict__ part,
                         const int* __restrict__ positions, const int* __restrict__ cu_seqlens, int n_seqs,
                         const int* __restrict__ block_table, int max_blocks, int tile_q,
                         int H, int G, int ps, int vis, int span, float scale_log2e, float cap_ratio,
                         const float* __restrict__ slopes, float inv_scale, int n_splits) {
    constexpr int NS = HD / 16;                      // steps of 16 head elements in the score product
    constexpr int NDT = HD / 32;                     // 32-row tiles of the output
    constexpr int NC = HD / 32;                      // chunks of a K tile row
    constexpr int TPR = HD / 16;                     // one-kilobyte tiles of a 32-key run (keys, or values)
    constexpr int RUN = 32 * HD;                     // elements of a run
    constexpr int STEP = PF_KEYS * HD;               // elements of the K (or V^T) tiles of one step
    extern __shared__ __attribute__((aligned(16))) bf16 sm[];
    bf16* Ks = sm;                                   // [2 buffers][PF_RUNS runs][TPR tiles][512]
    bf16* Vs = sm + 2 * STEP;                        // the same for V^T

    // (the wave's number is the same in all of its lanes: saying so keeps what follows from it in scalar registers)
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, hh = lane >> 5;
    const int QH = H / G;
    // consecutive workgroups take the kv heads in turn: with as many kv heads as the chip has
    // dies, a head's keys and values stay in one die's L2
    const int g = blockIdx.x % G;
    const int split = (blockIdx.x / G) % n_splits;

    // which request and which of its queries: tiles are counted request by request; tiles
    // late in a request walk the most keys, so the grid starts from the end
    const int n_tiles = gridDim.x / (G * n_splits);
    int tile = n_tiles - 1 - (int)(blockIdx.x / (G * n_splits)), seq = -1, t0 = 0, t_end = 0;
    for (int s = 0; s < n_seqs; ++s) {
        const int b = cu_seqlens[s], e = cu_seqlens[s + 1];
        const int nt = (e - b + tile_q - 1) / tile_q;
        if (tile < nt) { seq = s; t0 = b + tile * tile_q; t_end = (t0 + tile_q < e) ? t0 + tile_q : e; break; }
        tile -= nt;
    }
    if (seq < 0) return;
    const int* bt = block_table + (size_t)seq * max_blocks;
    const int p_first = positions[t0], p_last = positions[t_end - 1];
    const int u_first = sp_first_visible(p_first, vis, span) / PF_KEYS, u_last = p_last / PF_KEYS;

    // this lane's column (lanes l and l+32 share it)
    const int col = wave * 32 + n;
    const int tok = t0 + col / QH, head = g * QH + col % QH;
    const bool live = tok < t_end;
    const int pq = live ? positions[tok] : -1;
    const int lo = live ? sp_first_visible(pq, vis, span) : 0;
    const float slope = (EXTRA && slopes && live) ? slopes[head] * inv_scale : 0.f;
    bf16x8 qf[NS];
    {
        const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
        const bf16* qrow = q + ((size_t)(live ? tok : t0) * H + (live ? head : 0)) * HD + hh * 8;
#pragma unroll
        for (int st = 0; st < NS; ++st) qf[st] = live ? *(const bf16x8*)(qrow + st * 16) : zero8;
    }
    int pq_min = live ? pq : 0x7fffffff, pq_max = pq, lo_min = live ? lo : 0x7fffffff, lo_max = lo;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        pq_min = min(pq_min, __shfl_xor(pq_min, o, 64)); pq_max = max(pq_max, __shfl_xor(pq_max, o, 64));
        lo_min = min(lo_min, __shfl_xor(lo_min, o, 64)); lo_max = max(lo_max, __shfl_xor(lo_max, o, 64));
    }
    // uniform over the wave: scalar registers, so that the tests below are branches
    pq_min = __builtin_amdgcn_readfirstlane(pq_min); pq_max = __builtin_amdgcn_readfirstlane(pq_max);
    lo_min = __builtin_amdgcn_readfirstlane(lo_min); lo_max = __builtin_amdgcn_readfirstlane(lo_max);

    // m_run: the running maximum of the scaled scores (in the exponent's units); l_run: this
    // lane's part of the running sum (the two lanes of a column meet at the end)
    float m_run = -INFINITY, l_run = 0.f;
    f32x16 o[NDT];
#pragma unroll
    for (int d = 0; d < NDT; ++d)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[d][i] = 0.f;

    auto page_of = [&](int key) { const int i = key / ps; return i < max_blocks ? bt[i] : -1; };

    // ---- staging: every wave sends its share of the step's tiles from the pages into LDS.  A
    // step has PF_RUNS runs of keys and as many of values, each TPR tiles of one kilobyte that
    // lie in a row in its page; a wave sends one run's keys or values, a tile a load (16 bytes a lane).
    static_assert(PF_RUNS == 4, "eight waves send four runs of keys and four of values");
    const int hx = wave >> 1, is_v = wave & 1;
    auto stage = [&](int u, int buf) __attribute__((always_inline)) {
        const int key = u * PF_KEYS + hx * 32;
        int pg = page_of(key);
        // a page that is absent is read as page 0: its keys are masked or poisoned below, its
        // values taken as zero
        pg = pg < 0 ? 0 : pg;
        const size_t at = ((size_t)pg * G + g) * (size_t)ps * HD + (size_t)((key % ps) >> 5) * RUN + lane * 8;
        const bf16* src = (is_v ? v_pages : k_pages) + at;
        bf16* dst = (is_v ? Vs : Ks) + buf * STEP + hx * RUN;
#pragma unroll
        for (int i = 0; i < TPR; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + i * 512),
                                             (__attribute__((address_space(3))) void*)(dst + i * 512), 16, 0, 0);
    };

    // this lane's part of the operand addresses: row r of tile tt, the lane's half of the k run
    const int tt = (lane >> 4) & 1, r = lane & 15;
    const int k_lane = tt * NC * 512 + hh * 128 + r * 8;
    const int v_lane = tt * 512 + hh * 128 + r * 8;

    // ---- one run (32 keys, from key0) out of LDS, its tiles `at` elements into the buffers.
    // MASKED: tests per element.
    auto run32 = [&](int key0, int at, auto masked_tag) __attribute__((always_inline)) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        const bf16* kb_ = Ks + at + k_lane;
        const bf16* vb_ = Vs + at + v_lane;
        f32x16 s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.f;
        {
            bf16x8 kf[NS];
#pragma unroll
            for (int st = 0; st < NS; ++st) kf[st] = *(const bf16x8*)(kb_ + (st >> 1) * 512 + (st & 1) * 256);
#pragma unroll
            for (int st = 0; st < NS; ++st) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[st], qf[st], s, 0, 0, 0);
            // all of the run's K operands are asked for before the first product waits for one
            __builtin_amdgcn_sched_group_barrier(0x100, NS, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, NS, 0);
        }
        // (nothing of what follows moves up between them: the reads of V^T below would otherwise be
        // counted among the eight reads above, and the K operands they displace be read one by one,
        // each product waiting for its own)
        __builtin_amdgcn_sched_barrier(0);
        // on the cheap path the run's V^T operands are asked for before the softmax, whose arithmetic
        // hides their way
        bf16x8 vf[NDT][2];
        if (!MASKED) {
#pragma unroll
            for (int d = 0; d < NDT; ++d)
#pragma unroll
                for (int kg = 0; kg < 2; ++kg) vf[d][kg] = *(const bf16x8*)(vb_ + (2 * d) * 512 + kg * 256);
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * NDT, 0);
        }
        bool absent = false;
        if (MASKED) {
            absent = page_of(key0) < 0;
            // s[4j+i] is the key key0 + (hh + 2(j&1))*8 + (j>>1)*4 + i; keys that the column may not
            // read become -inf, keys of a page that was given back NaN
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = key0 + (hh + 2 * (j & 1)) * 8 + (j >> 1) * 4 + i;
                    float v = s[4 * j + i];
                    if (EXTRA) {
                        v += slope * (float)(key - pq);
                        // a cap on the scores: cap * tanh(score * scale / cap), with cap_ratio = scale / cap;
                        // the raw score is replaced by the one that the scale turns into the capped score
                        if (cap_ratio > 0.f) v = tanhf(v * cap_ratio) / cap_ratio;
                    }
                    const bool ok = key >= lo && key <= pq;
                    s[4 * j + i] = ok ? (absent ? NAN : v) : -INFINITY;
                }
        }
        // the maximum of the raw scores; the scale (positive) goes into the exponent's fma
        float mx = fmaxf(s[0], s[1]);
#pragma unroll
        for (int i = 2; i < 16; i += 2) mx = fmaxf(fmaxf(mx, s[i]), s[i + 1]);
        {
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
            mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
        }
        const float m_new = fmaxf(m_run, mx * scale_log2e);
        // a column with nothing visible so far keeps m = -inf: its weights are zero, not NaN
        const float m_safe = (MASKED && m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
        float sum = 0.f;
        bf16x8 pf[2];                                // P, as the second product's B operands
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = __builtin_amdgcn_exp2f(fmaf(s[4 * j + i], scale_log2e, -m_safe));
                sum += e;
                pf[j & 1][(j >> 1) * 4 + i] = (bf16)e;
            }
        l_run = l_run * alpha + sum;
        m_run = m_new;
        // the running maxima move in the first runs and seldom after: the output is rescaled
        // only when some column of the wave needs it (alpha is exactly 1 otherwise)
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int d = 0; d < NDT; ++d) o[d] = o[d] * alpha;
        }
        if (!MASKED) {
#pragma unroll
            for (int d = 0; d < NDT; ++d)
#pragma unroll
                for (int kg = 0; kg < 2; ++kg)
                    o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[d][kg], pf[kg], o[d], 0, 0, 0);
            return;
        }
        // Values that the request does not own must not meet even a probability of zero (zero times
        // a value that is not finite is not zero): the keys behind the last query of the wave may
        // lie behind the request's last position, where the page holds what its last owner left,
        // and a run whose page the request has given back was read from some other page.  Those
        // values are taken as zero.  (The other keys below a column's first visible one are the
        // request's own, and finite.)
        const bool stale = key0 + 31 > pq_max || absent;
#pragma unroll
        for (int d = 0; d < NDT; ++d)
#pragma unroll
            for (int kg = 0; kg < 2; ++kg) {
                bf16x8 v = *(const bf16x8*)(vb_ + (2 * d) * 512 + kg * 256);
                if (stale) {
                    // this lane's keys of the fragment: key0 + 16kg + 8hh + e
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        v[e] = (absent || key0 + kg * 16 + hh * 8 + e > pq_max) ? (bf16)0.f : v[e];
                }
                o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v, pf[kg], o[d], 0, 0, 0);
            }
    };
    // a step at an edge: every wave chooses its path run by run
    auto edge_step = [&](int u, int buf) __attribute__((always_inline)) {
        for (int h = 0; h < PF_RUNS; ++h) {
            const int key0 = u * PF_KEYS + h * 32;
            if (key0 > pq_max || key0 + 31 < lo_min) continue;            // nothing here for this wave
            const bool whole = !EXTRA && key0 >= lo_max && key0 + 31 <= pq_min && page_of(key0) >= 0;
            if (whole) run32(key0, buf * STEP + h * RUN, std::false_type{});
            else run32(key0, buf * STEP + h * RUN, std::true_type{});
        }
    };

    // The steps u_first .. u_last fall into three runs: a few at the lower edge (a chunk's or a
    // window's first keys), those that every query of the tile reads whole, and a few at the
    // upper edge (the causal diagonal).  The softmax does not care for the order of the keys,
    // so the edges come first, in a loop whose waves choose their path run by run, and the
    // whole steps after them in a loop that holds the cheap path and nothing else (one loop with
    // both paths makes the compiler merge their ends, at the price of moving the operands of
    // either into common registers in every run).  A split takes its share of that order.
    int uA = u_last + 1, uB = u_last + 1;
    if (!EXTRA) {
        uA = max(u_first, (sp_first_visible(p_last, vis, span) + PF_KEYS - 1) / PF_KEYS);
        uB = min(u_last + 1, (p_first + 1) / PF_KEYS);
        if (uA >= uB) uA = uB = u_last + 1;
    }
    const int n_steps = u_last + 1 - u_first, n_low = uA - u_first, n_edge = n_steps - (uB - uA);
    auto step_at = [&](int i) { return i < n_low ? u_first + i : (i < n_edge ? uB + (i - n_low) : uA + (i - n_edge)); };
    const int i_begin = (int)((long)n_steps * split / n_splits), i_end = (int)((long)n_steps * (split + 1) / n_splits);
    bool poison = false;          // a whole step met a page that is not there
    if (i_begin < i_end) {
        stage(step_at(i_begin), 0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
    int i = i_begin, buf = 0;
    for (; i < i_end && i < n_edge; ++i, buf ^= 1) {
        if (i + 1 < i_end) stage(step_at(i + 1), buf ^ 1);
        edge_step(step_at(i), buf);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
    if (i < i_end && pq_max >= 0) {
        // every query of the tile reads the keys of the steps that follow: a page that is missing
        // poisons them all.  The pages are looked up here, 64 at a time, not run by run in the loop
        // (a table entry per run is a scalar load that the next run's reads of LDS would wait for).
        const int k_lo = (uA + (i - n_edge)) * PF_KEYS, k_hi = (uA + (i_end - n_edge)) * PF_KEYS;
        bool bad = false;
        for (int pg = k_lo / ps + lane; pg <= (k_hi - 1) / ps; pg += 64) bad |= pg >= max_blocks || bt[pg] < 0;
        poison = __any(bad);
    }
    for (; i < i_end; ++i, buf ^= 1) {
        const int u = uA + (i - n_edge);
        if (i + 1 < i_end) stage(u + 1, buf ^ 1);
        if (pq_max >= 0) {
#pragma unroll
            for (int h = 0; h < PF_RUNS; ++h) run32(u * PF_KEYS + h * 32, buf * STEP + h * RUN, std::false_type{});
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    // the two lanes of a column add their parts of the sum
    {
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run), __float_as_uint(l_run), false, false);
        l_run = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
    }
    // o[d][4j+i] of lane (n, hh): column n of the wave, head element 32d + 8j + 4hh + i
    if (!live) return;
    if (n_splits > 1) {
        // This split's part of the tile, as it lies in the registers: a wave's stores are runs of
        // one kilobyte (a layout by columns would scatter them in pieces of 32 bytes).  The kernel
        // below reads it back the same way.
        float* rec = part + ((size_t)blockIdx.x * 8 + wave) * (32 * HD + 64);
#pragma unroll
        for (int d = 0; d < NDT; ++d)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                f32x4 w;
#pragma unroll
                for (int i2 = 0; i2 < 4; ++i2) w[i2] = poison ? NAN : o[d][4 * j + i2];
                *(f32x4*)(rec + ((d * 4 + j) * 64 + lane) * 4) = w;
            }
        rec[32 * HD + lane] = hh == 0 ? m_run : (poison ? NAN : l_run);
        return;
    }
    const float inv = poison ? NAN : 1.0f / fmaxf(l_run, 1e-30f);
    bf16* orow = out + ((size_t)tok * H + head) * HD;
#pragma unroll
    for (int d = 0; d < NDT; ++d)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            bf16x4 w;
#pragma unroll
            for (int i2 = 0; i2 < 4; ++i2) w[i2] = (bf16)(o[d][4 * j + i2] * inv);
            *(bf16x4*)(orow + d * 32 + j * 8 + hh * 4) = w;
        }
}

// Joins the splits of every tile: workgroup (tile, kv head) reads the records that its splits'
// workgroups left, in the registers' own layout, weighs them by their maxima and writes the
// output as the unsplit kernel does.
template <int HD>
__global__ __launch_bounds__(512)
void attn_prefill_join_kernel(const float* __restrict__ part, bf16* __restrict__ out, const int* __restrict__ cu_seqlens,
                              int n_seqs, int tile_q, int H, int G, int n_splits) {
    constexpr int NDT = HD / 32;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 31, hh = lane >> 5;
    const int QH = H / G, g = blockIdx.x % G;
    const int n_tiles = gridDim.x / G;
    int tile = n_tiles - 1 - (int)(blockIdx.x / G), t0 = -1, t_end = 0;
    for (int s = 0; s < n_seqs; ++s) {
        const int b = cu_seqlens[s], e = cu_seqlens[s + 1];
        const int nt = (e - b + tile_q - 1) / tile_q;
        if (tile < nt) { t0 = b + tile * tile_q; t_end = (t0 + tile_q < e) ? t0 + tile_q : e; break; }
        tile -= nt;
    }
    if (t0 < 0) return;
    const int col = wave * 32 + n;
    const int tok = t0 + col / QH, head = g * QH + col % QH;
    if (tok >= t_end) return;
    // the splits of this tile and kv head are the workgroups (blockIdx.x / G) * n_splits + s of the first kernel
    const size_t wg0 = ((size_t)(blockIdx.x / G) * n_splits) * G + g;
    auto rec_of = [&](int s) { return part + ((wg0 + (size_t)s * G) * 8 + wave) * (32 * HD + 64); };
    float M = -INFINITY;
    for (int s = 0; s < n_splits; ++s) M = fmaxf(M, rec_of(s)[32 * HD + n]);
    float L = 0.f;
    f32x4 acc[NDT][4];
#pragma unroll
    for (int d = 0; d < NDT; ++d)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[d][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < n_splits; ++s) {
        const float* rec = rec_of(s);
        const float m = rec[32 * HD + n], l = rec[32 * HD + 32 + n];
        if (m == -INFINITY) continue;                    // a split with no keys for this column
        const float w = exp2f(m - M);
        L += w * l;
#pragma unroll
        for (int d = 0; d < NDT; ++d)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[d][j] += w * *(const f32x4*)(rec + ((d * 4 + j) * 64 + lane) * 4);
    }
    const float inv = 1.0f / fmaxf(L, 1e-30f);
    bf16* orow = out + ((size_t)tok * H + head) * HD;
#pragma unroll
    for (int d = 0; d < NDT; ++d)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            bf16x4 w;
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = (bf16)(acc[d][j][i] * (L != L ? NAN : inv));
            *(bf16x4*)(orow + d * 32 + j * 8 + hh * 4) = w;
        }
}

template <int HD, bool EXTRA>
static int launch_prefill(const void* q, const void* k_pages, const void* v_pages, void* out, float* part, const int* positions,
                          const int* cu_seqlens, int n_seqs, const int* block_table, int max_blocks, int tile_q,
                          long n_tiles, int H, int G, int page_size, int vis, int span, float sl, float cr,
                          const float* slopes, float inv_scale, int n_splits, hipStream_t st) {
    const size_t sh = (size_t)2 * 2 * PF_KEYS * HD * sizeof(bf16);
    static bool allowed = false;          // one flag per instantiation: more LDS than the default limit
    if (!allowed) {
        hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_kernel<HD, EXTRA>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh);
        SP_REQUIRE(e == hipSuccess, "attn_prefill: %zu bytes of LDS refused: %s", sh, hipGetErrorString(e));
        allowed = true;
    }
    attn_prefill_kernel<HD, EXTRA><<<dim3((unsigned)(n_tiles * G * n_splits)), 512, sh, st>>>((const bf16*)q, (const bf16*)k_pages,
        (const bf16*)v_pages, (bf16*)out, part, positions, cu_seqlens, n_seqs, block_table, max_blocks, tile_q, H, G, page_size,
        vis, span, sl, cr, slopes, inv_scale, n_splits);
    SP_LAUNCH_CHECK("attn_prefill");
    return 0;
}

static long prefill_tiles(const int* counts, int n_seqs, int tile_q) {
    long tiles = 0;
    for (int s = 0; s < n_seqs; ++s) tiles += (counts[s] + tile_q - 1) / tile_q;
    return tiles;
}

// Into how many splits a step's tiles should be cut, for `max_keys` keys that the longest walk
// of a tile covers.  Splitting costs a record of (hd + 2) floats per column and split, written
// and read once; it pays where the walks are long and the tiles fill the compute units badly:
// the fewest splits (up to 8) that bring the last round of workgroups to nine tenths full, each
// split keeping at least 16 steps.
extern "C" int spite_attn_prefill_splits(const int* counts, int n_seqs, int H, int G, long max_keys) {
    if (n_seqs <= 0 || H <= 0 || G <= 0 || H % G || H / G > PF_COLS) return 1;
    const long tiles = prefill_tiles(counts, n_seqs, PF_COLS / (H / G)) * G;
    const long cus = sp_cu_count(), steps = (max_keys + PF_KEYS - 1) / PF_KEYS;
    if (tiles <= 0 || tiles >= 4 * cus) return 1;
    int best = 1;
    double best_fill = (double)tiles / (double)(((tiles + cus - 1) / cus) * cus);
    for (int n = 2; n <= 8 && steps / n >= 16 && best_fill < 0.9; ++n) {
        const long w = tiles * n;
        const double fill = (double)w / (double)(((w + cus - 1) / cus) * cus);
        if (fill > best_fill + 0.03) { best = n; best_fill = fill; }
    }
    return best;
}

// `counts` (host memory): the number of query tokens of each of the step's `n_seqs` requests,
// in the order of `cu_seqlens` (device), whose differences they are.  `n_splits` > 1: every
// tile's keys are dealt to that many workgroups, whose partial results go to `workspace`
// (spite_attn_prefill_workspace bytes) and are joined by a second kernel.  `slopes` (device,
// fp32 [H], or null): a bias slopes[head] * (key position - query position) added to the scaled
// scores before the cap.
extern "C" int spite_attn_prefill(const void* q, const void* k_pages, const void* v_pages, void* out, void* workspace,
                                  const int* positions, const int* cu_seqlens, const int* counts, int n_seqs,
                                  const int* block_table, int max_blocks, int H, int G, int hd, int page_size,
                                  int vis, int span, float scale, float softcap, const float* slopes, int n_splits,
                                  hipStream_t st) {
    SP_REQUIRE(softcap >= 0.f && scale > 0.f, "attn_prefill: scale %g, score cap %g", scale, softcap);
    SP_REQUIRE(n_seqs >= 0 && H > 0 && G > 0 && H % G == 0, "attn_prefill: %d query heads over %d kv heads", H, G);
    SP_REQUIRE(H / G <= PF_COLS, "attn_prefill: %d query heads per kv head, at most %d", H / G, PF_COLS);
    SP_REQUIRE(hd == 64 || hd == 128, "attn_prefill: head size %d (this kernel has 64 and 128)", hd);
    SP_REQUIRE(page_size > 0 && page_size % 32 == 0, "attn_prefill: page size %d must be a multiple of 32", page_size);
    SP_REQUIRE(max_blocks > 0, "attn_prefill: bad table width");
    SP_REQUIRE(vis >= 0 && vis < SP_VIS_COUNT && (!sp_vis_has_span(vis) || span > 0), "attn_prefill: chunk or window of %d", span);
    SP_REQUIRE(n_splits >= 1 && n_splits <= 256 && (n_splits == 1 || workspace), "attn_prefill: %d splits (1 to 256; more than one need a workspace)", n_splits);
    long T = 0;
    for (int s = 0; s < n_seqs; ++s) {
        SP_REQUIRE(counts[s] >= 0, "attn_prefill: request %d with %d tokens", s, counts[s]);
        T += counts[s];
    }
    const int tile_q = PF_COLS / (H / G);
    const long tiles = prefill_tiles(counts, n_seqs, tile_q);
    if (tiles == 0) return 0;
    SP_REQUIRE(tiles * G * n_splits <= 0x7fffffffL && T <= 0x7fffffffL, "attn_prefill: too many tiles");
    const float sl = scale * 1.4426950408889634f, cr = softcap > 0.f ? scale / softcap : 0.f;
    const bool extra = cr > 0.f || slopes != nullptr;
#define SP_PF(HDV, EX) launch_prefill<HDV, EX>(q, k_pages, v_pages, out, (float*)workspace, positions, cu_seqlens, n_seqs, \
        block_table, max_blocks, tile_q, tiles, H, G, page_size, vis, span, sl, cr, slopes, 1.0f / scale, n_splits, st)
    const int rc = hd == 128 ? (extra ? SP_PF(128, true) : SP_PF(128, false)) : (extra ? SP_PF(64, true) : SP_PF(64, false));
#undef SP_PF
    if (rc != 0 || n_splits == 1) return rc;
    if (hd == 128)
        attn_prefill_join_kernel<128><<<dim3((unsigned)(tiles * G)), 512, 0, st>>>((const float*)workspace, (bf16*)out, cu_seqlens,
                                                                                  n_seqs, tile_q, H, G, n_splits);
    else
        attn_prefill_join_kernel<64><<<dim3((unsigned)(tiles * G)), 512, 0, st>>>((const float*)workspace, (bf16*)out, cu_seqlens,
                                                                                 n_seqs, tile_q, H, G, n_splits);
    SP_LAUNCH_CHECK("attn_prefill_join");
    return 0;
}

// Bytes of fp32 scratch that a call with `n_splits` > 1 needs: one record of 256 columns per
// tile, kv head and split.
extern "C" size_t spite_attn_prefill_workspace(const int* counts, int n_seqs, int H, int G, int hd, int n_splits) {
    if (n_splits <= 1 || n_seqs <= 0 || H <= 0 || G <= 0 || H % G || H / G > PF_COLS) return 0;
    return (size_t)prefill_tiles(counts, n_seqs, PF_COLS / (H / G)) * G * n_splits * 8 * (32 * (size_t)hd + 64) * sizeof(float);
}
