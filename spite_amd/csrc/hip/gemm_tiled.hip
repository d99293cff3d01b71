// Tiled bf16 product for many rows (prefill) over weights stored in MFMA operand order:
// Y[M,N] = X[M,K] . W[N,K]^T, fp32 accumulation on MFMA 16x16x32.
//
// "Operand order" of W[N,K] (N % 16 == 0, K % 64 == 0): the matrix is cut into tiles of 16
// rows x 32 k; tile (i, j) lies at ((i * K/32) + j) * 512 elements, and inside it the eight
// elements W[16i + r][32j + 8q .. 8q+7] lie at ((q*16 + r) * 8): exactly what lane q*16 + r of
// a wave holds as the MFMA "A" operand.  A wave's load of a tile is one kilobyte in a row,
// eight whole cache lines, where the same load from a row-major matrix touches sixteen half
// lines; the path from L2 into the registers carries about half again as much that way, and
// that path, not the MFMA units or LDS, is what bounds this kernel.  The tiles of one row
// band follow each other in k, so a wave streams its four bands.
//
// A workgroup of eight waves owns 16*NB*WM rows of X ("slots") and 64*WN rows of W
// (WN * WM = 8); a wave owns 64 rows of W and 16*NB slots: 4 x NB accumulator tiles (NB = 8;
// 10 where the registers of the third W set go to the accumulators; 4 for short prompts, where
// the accumulators' registers go to more W sets).
//  * W never touches LDS: three rotating sets of operand registers, loaded two steps of 32 k
//    ahead of the products (NB = 10: two sets, one step ahead; NB = 4: six sets, five ahead).
//    NTW: W is read with non-temporal loads (where a band of W meets few row tiles it is read
//    once, and such a stream runs faster past the caches).
//  * X is the "B" operand, shared by the waves: tiles of 64 k go through LDS, fetched with
//    eight lanes a row (whole cache lines), rows padded by 16 bytes against bank conflicts,
//    double-buffered, one barrier per 64 k.
//  * Tiles are handed out so that the workgroups running on one XCD (one L2) at a time share
//    W bands and walk K together.
//  * k_splits > 1: a tile's sum over k is cut into runs, each a workgroup of its own that
//    writes partial sums (plain products over few tiles; the caller adds the runs).
// Grouped form (experts) and GLU as in gemm_generic.hip; with GLU a wave's bands are two of
// gate rows and the two matching of up rows.
#include "common.h"

#define TLD 72             // padded row of the X tile in LDS, in elements (64 k + 8)

// GROUPED: the grouped form (row lists per group); apart from what it leaves out of the plain
// product's code, it gives the two forms names of their own in a trace.
template <int WN, int WM, int NB, bool GLU, typename TY, bool NTW, bool GROUPED>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_tiled_kernel(const bf16* __restrict__ X, int ldx, const bf16* __restrict__ W, long w_group_stride,
                       TY* __restrict__ Y, int ldy, int M, int N, int K,
                       const int* __restrict__ offsets, int n_groups, const int* __restrict__ a_rows,
                       const float* __restrict__ a_scale, const int* __restrict__ y_rows, int m_tiles, int n_tiles,
                       int k_splits, size_t split_stride) {
    static_assert(WN * WM == 8, "eight waves");
    constexpr int WS = 16 * NB;                     // slots of a wave: NB slot tiles
    constexpr int BM = WS * WM, BN = 64 * WN;
    constexpr int NCOLS = GLU ? BN / 2 : BN;        // output columns per workgroup
    extern __shared__ __attribute__((aligned(16))) bf16 Xs[];     // [2][BM * TLD]

    // Which tile.  Workgroups go to the eight XCDs in turn, each with an L2 of its own: XCD x
    // takes the x-th eighth of the tiles, ordered with the row tile running fastest.
    // With k_splits > 1 a tile's sum over k is cut into that many runs, each a workgroup of its
    // own that writes its partial sums to Y + run * split_stride (the caller adds them up).
    const int units = m_tiles * n_tiles * k_splits;
    const int per_xcd = (units + 7) / 8;
    const int unit_id = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (unit_id >= units) return;
    const int ks = unit_id % k_splits, tile_id = unit_id / k_splits;
    const int tile_m = tile_id % m_tiles, tile_n = tile_id / m_tiles;
    int g = 0, row0, row_end = M;
    if (GROUPED) {
        if (!sp_find_tile(offsets, n_groups, BM, tile_m, g, row0, row_end)) return;
    } else {
        row0 = tile_m * BM;
        if (row0 >= M) return;
    }
    const int n0 = tile_n * NCOLS;
    const bf16* Wg = W + (size_t)g * w_group_stride;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave % WN, wm = wave / WN;
    const int r = lane & 15, q = lane >> 4;

    // ---- X: global -> registers -> LDS; thread loads 16-byte chunk (tid % 8) of rows tid/8 + 64*i
    constexpr int XL = (BM + 63) / 64;
    const int lrow = tid >> 3, lchunk = tid & 7;
    const bf16* xsrc[XL];
#pragma unroll
    for (int i = 0; i < XL; ++i) {
        // rows past the group read its last row again: no load of the main loop carries a
        // condition, and what such rows produce is never stored
        int s = row0 + lrow + 64 * i;
        s = s < row_end ? s : row_end - 1;
        xsrc[i] = X + (size_t)(a_rows ? a_rows[s] : s) * ldx + lchunk * 8;
    }
    // ---- W: the wave's four row bands
    //      plain: rows n0 + wn*64 + a*16; GLU: bands 0, 1 gate rows n0 + wn*32 + ..., bands 2, 3 the up rows N + ...
    constexpr int TG = GLU ? 2 : 4;          // bands that name distinct output columns
    const int kt_all = K / 32;               // tiles in a band
    const bf16* wsrc[4];
    int ncol[4];                             // output column of the band's first row
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int n = n0 + wn * 16 * TG + (a % TG) * 16;
        int band = n / 16;
        band = band < N / 16 ? band : N / 16 - 1;        // bands past N read the last band again
        if (GLU && a >= TG) band += N / 16;
        ncol[a] = n;
        wsrc[a] = Wg + (size_t)band * kt_all * 512 + lane * 8;
    }
    // this workgroup's run of 64-k steps
    const int nu_all = K / 64, per_run = (nu_all + k_splits - 1) / k_splits;
    const int u_first = ks * per_run;
    const int nu = (u_first + per_run < nu_all ? u_first + per_run : nu_all) - u_first;     // > 0 by the caller's choice of k_splits
#pragma unroll
    for (int i = 0; i < XL; ++i) xsrc[i] += (size_t)u_first * 64;
#pragma unroll
    for (int a = 0; a < 4; ++a) wsrc[a] += (size_t)u_first * 2 * 512;
    Y += (size_t)ks * split_stride;
    auto load_x = [&](bf16x8 (&xr)[XL], int u) {
        const int k0 = (u < nu ? u : nu - 1) * 64;
#pragma unroll
        for (int i = 0; i < XL; ++i)
            if (64 * (i + 1) <= BM || lrow + 64 * i < BM) xr[i] = *(const bf16x8*)(xsrc[i] + k0);   // (whole waves)
    };
    auto store_x = [&](bf16x8 (&xr)[XL], int buf) {
#pragma unroll
        for (int i = 0; i < XL; ++i)
            if (64 * (i + 1) <= BM || lrow + 64 * i < BM)
                *(bf16x8*)(Xs + buf * (BM * TLD) + (lrow + 64 * i) * TLD + lchunk * 8) = xr[i];
    };
    const int kt = 2 * nu;                   // 32-k tiles of the run
    auto load_w = [&](bf16x8 (&ws)[4], int t) {
        const size_t at = (size_t)(t < kt ? t : kt - 1) * 512;
#pragma unroll
        for (int a = 0; a < 4; ++a)
            ws[a] = NTW ? __builtin_nontemporal_load((const bf16x8*)(wsrc[a] + at)) : *(const bf16x8*)(wsrc[a] + at);
    };

    f32x4 acc[4][NB];          // [W band a][slot tile b]
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
    auto mul = [&](bf16x8 (&ws)[4], int buf, int kk) {
        const bf16* xs = Xs + buf * (BM * TLD) + (wm * WS + r) * TLD + kk * 32 + q * 8;
        constexpr int NX = 4;                        // slot tiles read from LDS at a time
#pragma unroll
        for (int b0 = 0; b0 < NB; b0 += NX) {
            bf16x8 xf[NX];
#pragma unroll
            for (int b = 0; b < NX; ++b)
                if (b0 + b < NB) xf[b] = *(const bf16x8*)(xs + (b0 + b) * 16 * TLD);
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < NX; ++b)
                    if (b0 + b < NB)
                        acc[a][b0 + b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ws[a], xf[b], acc[a][b0 + b], 0, 0, 0);
        }
    };

    // Step u covers 64 k: two half steps t = 2u, 2u+1.  Half step t multiplies W set t % 3
    // with the X tile in LDS buffer u % 2 while W tile t+2 is asked for into set (t+2) % 3.
    // X tile u+1 is asked for at the start of step u and stored to the other LDS buffer at
    // its end.  Three steps bring every name back.  The loop runs whole rounds of three with
    // no condition inside; up to two steps follow it.  Loads past the end fetch the last tile
    // again and are never used.
    bf16x8 w0[4], w1[4], w2[4], xr[XL];
    auto step = [&](bf16x8 (&wa)[4], bf16x8 (&wb)[4], bf16x8 (&wc)[4], int u) {
        // wa: set of half step 2u, wb: of 2u+1, wc: of 2u+2; wa is loaded again for 2u+3
        load_x(xr, u + 1);
        load_w(wc, 2 * u + 2);
        __builtin_amdgcn_sched_barrier(0);
        mul(wa, u & 1, 0);
        load_w(wa, 2 * u + 3);
        __builtin_amdgcn_sched_barrier(0);
        mul(wb, u & 1, 1);
        store_x(xr, (u + 1) & 1);
        __syncthreads();
    };
    if constexpr (NB == 8) {
        load_x(xr, 0);
        load_w(w0, 0);
        load_w(w1, 1);
        store_x(xr, 0);
        __syncthreads();
        int u = 0;
        for (; u + 3 <= nu; u += 3) {
            step(w0, w1, w2, u);            // half steps 0, 1: use w0, w1; load w2 (t=2), w0 (t=3)
            step(w2, w0, w1, u + 1);        // half steps 2, 3: use w2, w0; load w1 (t=4), w2 (t=5)
            step(w1, w2, w0, u + 2);        // half steps 4, 5: use w1, w2; load w0 (t=6), w1 (t=7)
        }
        if (u < nu) {
            step(w0, w1, w2, u);
            if (u + 1 < nu) step(w2, w0, w1, u + 1);
        }
    } else if constexpr (NB == 4) {
        // few slots a wave (short prompts, where the time is the stream of W from memory): the
        // accumulators' registers go to six sets of W, each asked for again as soon as its
        // products are issued, five half steps ahead of its use: three times the bytes in flight
        bf16x8 w3[4], w4[4], w5[4];
        auto step6 = [&](bf16x8 (&wa)[4], bf16x8 (&wb)[4], int u) {
            load_x(xr, u + 1);
            __builtin_amdgcn_sched_barrier(0);
            mul(wa, u & 1, 0);
            load_w(wa, 2 * u + 6);
            __builtin_amdgcn_sched_barrier(0);
            mul(wb, u & 1, 1);
            load_w(wb, 2 * u + 7);
            store_x(xr, (u + 1) & 1);
            __syncthreads();
        };
        load_x(xr, 0);
        load_w(w0, 0); load_w(w1, 1); load_w(w2, 2); load_w(w3, 3); load_w(w4, 4); load_w(w5, 5);
        store_x(xr, 0);
        __syncthreads();
        int u = 0;
        for (; u + 3 <= nu; u += 3) {
            step6(w0, w1, u);
            step6(w2, w3, u + 1);
            step6(w4, w5, u + 2);
        }
        if (u < nu) {
            step6(w0, w1, u);
            if (u + 1 < nu) step6(w2, w3, u + 1);
        }
    } else {
        // more slot tiles a wave: the registers of the third set go to the accumulators, and a
        // set is asked for again as soon as its products are issued, one half step ahead
        load_x(xr, 0);
        load_w(w0, 0);
        load_w(w1, 1);
        store_x(xr, 0);
        __syncthreads();
        for (int u = 0; u < nu; ++u) {
            load_x(xr, u + 1);
            __builtin_amdgcn_sched_barrier(0);
            mul(w0, u & 1, 0);
            load_w(w0, 2 * u + 2);
            __builtin_amdgcn_sched_barrier(0);
            mul(w1, u & 1, 1);
            load_w(w1, 2 * u + 3);
            store_x(xr, (u + 1) & 1);
            __syncthreads();
        }
    }

    // acc[a][b][i] of lane (r, q): column ncol[a] + q*4 + i, slot row0 + wm*WS + b*16 + r.  A lane's four
    // columns go out in one store (8 bytes of bf16, 16 of fp32) where the row's address allows it.
    const bool vec_ok = (ldy & 3) == 0 && (((uintptr_t)Y) & 15) == 0 && (N & 3) == 0;
    auto put4 = [&](TY* dst, int n, const float (&v)[4]) {
        if (vec_ok && n + 3 < N) {
            if constexpr (sizeof(TY) == 2) {
                bf16x4 o;
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = (bf16)v[i];
                *(bf16x4*)(dst + n) = o;
            } else {
                *(f32x4*)(dst + n) = f32x4{v[0], v[1], v[2], v[3]};
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n + i < N) dst[n + i] = from_f32<TY>(v[i]);
        }
    };
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int s = row0 + wm * WS + b * 16 + r;
        if (s >= row_end) continue;
        const float sc = a_scale ? a_scale[s] : 1.0f;
        const size_t yr = y_rows ? (size_t)y_rows[s] : (size_t)s;
        TY* yrow = Y + yr * ldy;
        if (GLU) {
#pragma unroll
            for (int a = 0; a < TG; ++a) {
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float gv = acc[a][b][i] * sc, uv = acc[a + TG][b][i] * sc;
                    v[i] = gv / (1.0f + __expf(-gv)) * uv;
                }
                put4(yrow, ncol[a] + q * 4, v);
            }
        } else {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = acc[a][b][i] * sc;
                put4(yrow, ncol[a] + q * 4, v);
            }
        }
    }
}

template <int WN, int WM, int NB, bool GLU, typename TY, bool NTW = false>
static int launch_tiled_kernel(const void* X, int ldx, const void* W, long w_group_stride, void* Y, int ldy, int M, int N,
                               int K, const int* offsets, int n_groups, const int* a_rows, const float* a_scale,
                               const int* y_rows, int k_splits, size_t split_stride, hipStream_t st) {
    constexpr int BM = 16 * NB * WM, BN = 64 * WN;
    // row tiles: a group with rows has 1 + (rows - 1) / tile of them, so groups with rows + M / tile bounds them
    const int m_tiles = offsets ? M / BM + (n_groups < M ? n_groups : M) : (M + BM - 1) / BM;
    const int ncols = GLU ? BN / 2 : BN;
    const int n_tiles = (N + ncols - 1) / ncols;
    SP_REQUIRE((long)m_tiles * n_tiles * k_splits < (1L << 30), "gemm_tiled: too many tiles");
    const size_t sh = (size_t)2 * BM * TLD * sizeof(bf16);
    static bool allowed = false;        // one flag per instantiation; more LDS than the default limit for WM = 2
    if (!allowed) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_tiled_kernel<WN, WM, NB, GLU, TY, NTW, true>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void*)gemm_tiled_kernel<WN, WM, NB, GLU, TY, NTW, false>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh);
        SP_REQUIRE(e == hipSuccess, "gemm_tiled: %zu bytes of LDS refused: %s", sh, hipGetErrorString(e));
        allowed = true;
    }
    const dim3 grid((m_tiles * n_tiles * k_splits + 7) / 8 * 8);
    if (offsets)
        gemm_tiled_kernel<WN, WM, NB, GLU, TY, NTW, true><<<grid, 512, sh, st>>>(
            (const bf16*)X, ldx, (const bf16*)W, w_group_stride, (TY*)Y, ldy, M, N, K, offsets, n_groups, a_rows, a_scale,
            y_rows, m_tiles, n_tiles, k_splits, split_stride);
    else
        gemm_tiled_kernel<WN, WM, NB, GLU, TY, NTW, false><<<grid, 512, sh, st>>>(
            (const bf16*)X, ldx, (const bf16*)W, w_group_stride, (TY*)Y, ldy, M, N, K, offsets, n_groups, a_rows, a_scale,
            y_rows, m_tiles, n_tiles, k_splits, split_stride);
    SP_LAUNCH_CHECK("gemm_tiled");
    return 0;
}

template <int WN, int WM, int NB>
static int launch_tiled(const void* X, int ldx, const void* W, long w_group_stride, void* Y, int y_dtype, int ldy, int M,
                        int N, int K, const int* offsets, int n_groups, const int* a_rows, const float* a_scale,
                        const int* y_rows, int glu, hipStream_t st) {
    // Few row tiles a band of W (a short prompt): W is read once, and a stream that is read
    // once runs faster with non-temporal loads (7.1 against 6.3 TB/s); with many row tiles the
    // bands are read again from L2, which such loads would bypass.
    const bool once = NB == 8 && WM == 1 && M / (offsets ? n_groups : 1) <= 128;
#define SP_TL(GLUV, TY, NTV) launch_tiled_kernel<WN, WM, NB, GLUV, TY, NTV>(X, ldx, W, w_group_stride, Y, ldy, M, N, K, offsets, \
                                                                        n_groups, a_rows, a_scale, y_rows, 1, 0, st)
    if constexpr (NB == 8 && WM == 1) {
        if (once) {
            if (glu) return y_dtype == SP_BF16 ? SP_TL(true, bf16, true) : SP_TL(true, float, true);
            return y_dtype == SP_BF16 ? SP_TL(false, bf16, true) : SP_TL(false, float, true);
        }
    }
    if (glu) return y_dtype == SP_BF16 ? SP_TL(true, bf16, false) : SP_TL(true, float, false);
    return y_dtype == SP_BF16 ? SP_TL(false, bf16, false) : SP_TL(false, float, false);
#undef SP_TL
}

// Sum of the partial products of a split call: out[m][n] = sum over runs of part[run][m][n].
template <typename TY>
__global__ void add_runs_kernel(const float* __restrict__ part, int runs, size_t stride, TY* __restrict__ out, int ldy, int M, int N) {
    const size_t total = (size_t)M * N;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        float v = 0.f;
        for (int r = 0; r < runs; ++r) v += part[(size_t)r * stride + i];
        out[(i / N) * ldy + i % N] = from_f32<TY>(v);
    }
}

// A plain product (no groups, no row lists, no GLU) over few tiles, the sum over k cut into
// `k_splits` runs so that the chip is filled: `workspace` holds k_splits * M * N floats.
extern "C" int spite_gemm_tiled_split(const void* X, int ldx, const void* W, void* Y, int y_dtype, int ldy, int M, int N,
                                      int K, int k_splits, void* workspace, hipStream_t st) {
    SP_REQUIRE(M > 0 && N > 0 && K > 0 && ldx >= K && ldy >= N, "gemm_tiled: bad sizes M=%d N=%d K=%d", M, N, K);
    SP_REQUIRE(K % 64 == 0 && N % 16 == 0, "gemm_tiled: operand order needs K=%d a multiple of 64 and N=%d of 16", K, N);
    SP_REQUIRE(ldx % 8 == 0, "gemm_tiled: the row stride %d must be a multiple of 8", ldx);
    SP_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_tiled: operands must be 16-byte aligned");
    SP_REQUIRE(y_dtype == SP_BF16 || y_dtype == SP_F32, "gemm_tiled: output dtype %d", y_dtype);
    const int nu = K / 64;
    SP_REQUIRE(k_splits >= 2 && workspace, "gemm_tiled: a split call needs at least two runs and a workspace");
    SP_REQUIRE(((nu + k_splits - 1) / k_splits) * (k_splits - 1) < nu, "gemm_tiled: %d runs over %d steps leave a run empty", k_splits, nu);
    const size_t stride = (size_t)M * N;
    int rc = launch_tiled_kernel<8, 1, 8, false, float, true>(X, ldx, W, 0, workspace, N, M, N, K, nullptr, 1, nullptr, nullptr, nullptr,
                                                        k_splits, stride, st);
    if (rc) return rc;
    const size_t blocks = (stride + 255) / 256;
    const int grid = (int)(blocks < 8192 ? blocks : 8192);
    if (y_dtype == SP_BF16) add_runs_kernel<bf16><<<grid, 256, 0, st>>>((const float*)workspace, k_splits, stride, (bf16*)Y, ldy, M, N);
    else add_runs_kernel<float><<<grid, 256, 0, st>>>((const float*)workspace, k_splits, stride, (float*)Y, ldy, M, N);
    SP_LAUNCH_CHECK("add_runs");
    return 0;
}

// W in operand order (see above), every group N (2N with GLU) rows of K.
// `shape`: 0 lets the library choose; 1 = 512 W rows x 128 slots a workgroup, 2 = 256 x 256,
// 3 = 512 x 160 (for groups of a little over 128 rows, which would need a second tile of 128),
// 4 and 5 = 512 x 64 with W asked for five half steps ahead (short prompts: the stream of W from
// memory is the time; 4 reads W with non-temporal loads, 5 with plain ones), 6 = 512 x 96 (plain
// products only).
extern "C" int spite_gemm_tiled(const void* X, int ldx, const void* W, long w_group_stride, void* Y, int y_dtype,
                                int ldy, int M, int N, int K, const int* offsets, int n_groups, const int* a_rows,
                                const float* a_scale, const int* y_rows, int glu, int shape, hipStream_t st) {
    SP_REQUIRE(M >= 0 && N > 0 && K > 0 && ldx >= K && ldy >= N, "gemm_tiled: bad sizes M=%d N=%d K=%d", M, N, K);
    SP_REQUIRE(K % 64 == 0 && N % 16 == 0, "gemm_tiled: operand order needs K=%d a multiple of 64 and N=%d of 16", K, N);
    SP_REQUIRE(ldx % 8 == 0, "gemm_tiled: the row stride %d must be a multiple of 8", ldx);
    SP_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_tiled: operands must be 16-byte aligned");
    SP_REQUIRE(y_dtype == SP_BF16 || y_dtype == SP_F32, "gemm_tiled: output dtype %d", y_dtype);
    SP_REQUIRE(!offsets || n_groups > 0, "gemm_tiled: grouped call without groups");
    SP_REQUIRE(shape >= 0 && shape <= 6, "gemm_tiled: tile shape %d", shape);
    if (M == 0) return 0;
    if (shape == 0) {
        // Tiles come in whole numbers per CU: a plain product whose 128-row tiles leave many of the
        // CUs without one (2,048 x 5,120 on 256 CUs: 160 tiles) takes 96-row tiles when those need no
        // further round (220 tiles).  A tile's time is a fixed part (W's stream, start and end) and a
        // part per 16 rows, measured as 38 and 8.5 us at K = 5,120 on an MI355X; only their ratio
        // counts here, and both parts grow with K alike.  The sum over k runs in the same order in
        // both, so a row's result does not depend on the choice.
        constexpr double TILE_FIXED = 38.0, TILE_PER_16_ROWS = 8.5;
        shape = 1;
        if (!offsets && !glu) {
            const long cus = sp_cu_count(), cols = (N + 511) / 512;
            const long rounds8 = (((M + 127) / 128) * cols + cus - 1) / cus, rounds6 = (((M + 95) / 96) * cols + cus - 1) / cus;
            if (rounds6 * (TILE_FIXED + TILE_PER_16_ROWS * 6) < rounds8 * (TILE_FIXED + TILE_PER_16_ROWS * 8)) shape = 6;
        }
    }
    if (shape == 6) {
        SP_REQUIRE(!offsets && !glu, "gemm_tiled: the 96-row tile is for plain products");
        return y_dtype == SP_BF16
            ? launch_tiled_kernel<8, 1, 6, false, bf16, false>(X, ldx, W, w_group_stride, Y, ldy, M, N, K, nullptr, 1, a_rows, a_scale, y_rows, 1, 0, st)
            : launch_tiled_kernel<8, 1, 6, false, float, false>(X, ldx, W, w_group_stride, Y, ldy, M, N, K, nullptr, 1, a_rows, a_scale, y_rows, 1, 0, st);
    }
    if (shape == 1)
        return launch_tiled<8, 1, 8>(X, ldx, W, w_group_stride, Y, y_dtype, ldy, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, st);
    if (shape == 4 || shape == 5) {
        // 512 x 64, six W sets ahead: 4 streams W with non-temporal loads, 5 with plain ones
#define SP_T4(GLUV, TY, NTV) launch_tiled_kernel<8, 1, 4, GLUV, TY, NTV>(X, ldx, W, w_group_stride, Y, ldy, M, N, K, offsets, \
                                                                     n_groups, a_rows, a_scale, y_rows, 1, 0, st)
        if (shape == 4) {
            if (glu) return y_dtype == SP_BF16 ? SP_T4(true, bf16, true) : SP_T4(true, float, true);
            return y_dtype == SP_BF16 ? SP_T4(false, bf16, true) : SP_T4(false, float, true);
        }
        if (glu) return y_dtype == SP_BF16 ? SP_T4(true, bf16, false) : SP_T4(true, float, false);
        return y_dtype == SP_BF16 ? SP_T4(false, bf16, false) : SP_T4(false, float, false);
#undef SP_T4
    }
    if (shape == 3)
        return launch_tiled<8, 1, 10>(X, ldx, W, w_group_stride, Y, y_dtype, ldy, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, st);
    return launch_tiled<4, 2, 8>(X, ldx, W, w_group_stride, Y, y_dtype, ldy, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, st);
}
