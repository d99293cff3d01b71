// Tiled bf16 product for many rows (prefill): Y[M,N] = X[M,K] . W[N,K]^T on MFMA 16x16x32 with
// fp32 accumulation.  A workgroup of eight waves owns 128*WM rows of X ("slots") and 64*WN
// rows of W (WN * WM = 8); a wave owns 64 rows of W and 128 slots: 4 x 8 accumulator tiles,
// so that a byte read from LDS or from the cache feeds as many products as the registers
// allow.
//
//  * W is the MFMA "A" operand and never touches LDS: a wave reads its own rows from global
//    memory straight into the operand layout (lane (r, q): 16 bytes of row r), two k steps
//    ahead of the products, in three rotating sets of registers.  Where few rows meet a
//    weight (experts), the kernel is a stream of W, like the decode kernel.
//  * X is the "B" operand, shared by the waves: its tiles of 32 k go through LDS (rows padded
//    by 16 bytes, so that the 16-byte operand reads of sixteen rows fall into different bank
//    groups), double-buffered, one barrier per tile; they too are fetched two steps ahead.
//  * A lane ends with four consecutive columns n of one row m of Y.
//  * Tiles are handed out so that the workgroups running on one XCD (one L2) at a time share
//    W tiles and walk K together.
//
// Grouped form (experts) and GLU as in gemm_generic.hip: a workgroup's slots lie inside one
// group; a slot's scale multiplies the fp32 sums; with GLU a wave's W rows are half gate rows
// and half the matching up rows.
#include "common.h"

#define MBK 32
#define MLD (MBK + 8)      // padded row of the X tile in LDS, in elements
#define MTA 4              // W row tiles per wave
#define MTB 8              // slot tiles per wave

template <int WN, int WM, bool GLU, bool EXACT, typename TY>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_mfma_kernel(const bf16* __restrict__ X, int ldx, const bf16* __restrict__ W, long w_group_stride,
                      TY* __restrict__ Y, int ldy, int M, int N, int K,
                      const int* __restrict__ offsets, int n_groups, const int* __restrict__ a_rows,
                      const float* __restrict__ a_scale, const int* __restrict__ y_rows, int m_tiles, int n_tiles) {
    static_assert(WN * WM == 8, "eight waves");
    constexpr int BM = 128 * WM, BN = 64 * WN;
    constexpr int NCOLS = GLU ? BN / 2 : BN;        // output columns per workgroup
    __shared__ __attribute__((aligned(16))) bf16 Xs[2][BM * MLD];

    // Which tile.  Workgroups go to the eight XCDs in turn, each with an L2 of its own: XCD x
    // takes the x-th eighth of the tiles, ordered with the row tile running fastest.
    const int per_xcd = (m_tiles * n_tiles + 7) / 8;
    const int tile_id = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (tile_id >= m_tiles * n_tiles) return;
    const int tile_m = tile_id % m_tiles, tile_n = tile_id / m_tiles;
    int g = 0, row0, row_end = M;
    if (offsets) {
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

    // ---- X: global -> registers -> LDS; thread loads 16-byte chunk (tid % 4) of rows tid/4 + 128*i
    constexpr int XL = WM;
    const int lrow = tid >> 2, lchunk = tid & 3;
    const bf16* xsrc[XL];
#pragma unroll
    for (int i = 0; i < XL; ++i) {
        // rows past the group read its last row again: the loads of the main loop carry no
        // condition (a select on a loaded value would make the wave wait for it at once), and
        // what such rows produce is never stored
        int s = row0 + lrow + 128 * i;
        s = s < row_end ? s : row_end - 1;
        xsrc[i] = X + (size_t)(a_rows ? a_rows[s] : s) * ldx + lchunk * 8;
    }
    // ---- W: the wave's four row tiles; lane (r, q) reads row r of each
    //      plain: rows n0 + wn*64 + a*16; GLU: tiles 0, 1 gate rows n0 + wn*32 + ..., tiles 2, 3 the up rows N + ...
    constexpr int TG = GLU ? MTA / 2 : MTA;    // tiles that name distinct output columns
    const bf16* wsrc[MTA];
    int ncol[MTA];           // output column of the tile's first row
#pragma unroll
    for (int a = 0; a < MTA; ++a) {
        const int n = n0 + wn * 16 * TG + (a % TG) * 16;
        const int nr = (n + r) < N ? n + r : N - 1;
        const size_t grow = ((GLU && a >= TG) ? (size_t)N : 0) + nr;
        ncol[a] = n;
        wsrc[a] = Wg + grow * K + q * 8;
    }
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const int nt = (K + MBK - 1) / MBK;
    // EXACT: K is a multiple of the tile and no load carries a condition; tiles past the end
    // load the last tile again (never used).  Otherwise chunks past K are zero (K is a
    // multiple of 8); that form is slower and only serves odd widths.
    auto load_x = [&](bf16x8 (&xr)[XL], int t) {
        const int k0 = (t < nt ? t : nt - 1) * MBK;
#pragma unroll
        for (int i = 0; i < XL; ++i)
            xr[i] = (EXACT || k0 + lchunk * 8 < K) ? *(const bf16x8*)(xsrc[i] + k0) : zero;
    };
    auto store_x = [&](bf16x8 (&xr)[XL], int buf) {
#pragma unroll
        for (int i = 0; i < XL; ++i) *(bf16x8*)(Xs[buf] + (lrow + 128 * i) * MLD + lchunk * 8) = xr[i];
    };
    auto load_w = [&](bf16x8 (&ws)[MTA], int t) {
        const int k0 = (t < nt ? t : nt - 1) * MBK;
#pragma unroll
        for (int a = 0; a < MTA; ++a) ws[a] = (EXACT || k0 + q * 8 < K) ? *(const bf16x8*)(wsrc[a] + k0) : zero;
    };

    f32x4 acc[MTA][MTB];       // [W row tile a][slot tile b]
#pragma unroll
    for (int a = 0; a < MTA; ++a)
#pragma unroll
        for (int b = 0; b < MTB; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
    auto mul = [&](bf16x8 (&ws)[MTA], int buf) {
        const bf16* xs = Xs[buf] + (wm * 128 + r) * MLD + q * 8;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            bf16x8 xf[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) xf[b] = *(const bf16x8*)(xs + (half * 4 + b) * 16 * MLD);
#pragma unroll
            for (int a = 0; a < MTA; ++a)
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    acc[a][half * 4 + b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ws[a], xf[b], acc[a][half * 4 + b], 0, 0, 0);
        }
    };

    // Step t multiplies tile t out of LDS buffer t % 2 and W set t % 3, while tile t+2 is asked
    // for (W into set (t+2) % 3, X into registers) and tile t+1's X, which arrived during the
    // step before, is stored to the other LDS buffer.  Six steps bring every name back; the loop
    // has one way out (leaving it from the middle made the compiler spill the accumulators).
    bf16x8 w0[MTA], w1[MTA], w2[MTA], xa[XL], xb[XL];
    auto step = [&](bf16x8 (&w_use)[MTA], bf16x8 (&w_load)[MTA], bf16x8 (&x_load)[XL], bf16x8 (&x_store)[XL], int t) {
        load_x(x_load, t + 2);
        load_w(w_load, t + 2);
        __builtin_amdgcn_sched_barrier(0);
        if (t < nt) mul(w_use, t & 1);       // the last round of six may run past the end: only its loads happen
        store_x(x_store, (t + 1) & 1);
        __syncthreads();
    };
    load_x(xa, 0); load_w(w0, 0);
    load_x(xb, 1); load_w(w1, 1);
    store_x(xa, 0);
    __syncthreads();
    for (int t = 0; t < nt; t += 6) {
        step(w0, w2, xa, xb, t);
        step(w1, w0, xb, xa, t + 1);
        step(w2, w1, xa, xb, t + 2);
        step(w0, w2, xb, xa, t + 3);
        step(w1, w0, xa, xb, t + 4);
        step(w2, w1, xb, xa, t + 5);
    }

    // acc[a][b][i] of lane (r, q): column ncol[a] + q*4 + i, slot row0 + wm*128 + b*16 + r
#pragma unroll
    for (int b = 0; b < MTB; ++b) {
        const int s = row0 + wm * 128 + b * 16 + r;
        if (s >= row_end) continue;
        const float sc = a_scale ? a_scale[s] : 1.0f;
        const size_t yr = y_rows ? (size_t)y_rows[s] : (size_t)s;
        TY* yrow = Y + yr * ldy;
        if (GLU) {
#pragma unroll
            for (int a = 0; a < TG; ++a) {
                const int n = ncol[a] + q * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (n + i < N) {
                        const float gv = acc[a][b][i] * sc, uv = acc[a + TG][b][i] * sc;
                        yrow[n + i] = from_f32<TY>(gv / (1.0f + __expf(-gv)) * uv);
                    }
                }
            }
        } else {
#pragma unroll
            for (int a = 0; a < MTA; ++a) {
                const int n = ncol[a] + q * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) yrow[n + i] = from_f32<TY>(acc[a][b][i] * sc);
            }
        }
    }
}

template <int WN, int WM>
static int launch_mfma(const void* X, int ldx, const void* W, long w_group_stride, void* Y, int y_dtype, int ldy, int M,
                       int N, int K, const int* offsets, int n_groups, const int* a_rows, const float* a_scale,
                       const int* y_rows, int glu, hipStream_t st) {
    constexpr int BM = 128 * WM, BN = 64 * WN;
    // row tiles: a group with rows has 1 + (rows - 1) / tile of them, so groups with rows + M / tile bounds them
    const int m_tiles = offsets ? M / BM + (n_groups < M ? n_groups : M) : (M + BM - 1) / BM;
    const int ncols = glu ? BN / 2 : BN;
    const int n_tiles = (N + ncols - 1) / ncols;
    SP_REQUIRE((long)m_tiles * n_tiles < (1L << 30), "gemm_mfma: too many tiles");
    dim3 grid((m_tiles * n_tiles + 7) / 8 * 8);
#define SP_MM(GLUV, TY) do { if (K % MBK == 0) gemm_mfma_kernel<WN, WM, GLUV, true, TY><<<grid, 512, 0, st>>>((const bf16*)X, ldx, \
        (const bf16*)W, w_group_stride, (TY*)Y, ldy, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, m_tiles, n_tiles); \
    else gemm_mfma_kernel<WN, WM, GLUV, false, TY><<<grid, 512, 0, st>>>((const bf16*)X, ldx, (const bf16*)W, \
        w_group_stride, (TY*)Y, ldy, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, m_tiles, n_tiles); } while (0)
    if (glu) { if (y_dtype == SP_BF16) SP_MM(true, bf16); else SP_MM(true, float); }
    else { if (y_dtype == SP_BF16) SP_MM(false, bf16); else SP_MM(false, float); }
#undef SP_MM
    SP_LAUNCH_CHECK("gemm_mfma");
    return 0;
}

// `shape`: 0 lets the library choose; 1 = 512 W rows x 128 slots a workgroup, 2 = 256 x 256.
extern "C" int spite_gemm_mfma(const void* X, int ldx, const void* W, long w_group_stride, void* Y, int y_dtype,
                               int ldy, int M, int N, int K, const int* offsets, int n_groups, const int* a_rows,
                               const float* a_scale, const int* y_rows, int glu, int shape, hipStream_t st) {
    SP_REQUIRE(M >= 0 && N > 0 && K > 0 && ldx >= K && ldy >= N, "gemm_mfma: bad sizes M=%d N=%d K=%d", M, N, K);
    SP_REQUIRE(K % 8 == 0 && ldx % 8 == 0, "gemm_mfma: K=%d and the row stride %d must be multiples of 8", K, ldx);
    SP_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_mfma: operands must be 16-byte aligned");
    SP_REQUIRE(y_dtype == SP_BF16 || y_dtype == SP_F32, "gemm_mfma: output dtype %d", y_dtype);
    SP_REQUIRE(!offsets || n_groups > 0, "gemm_mfma: grouped call without groups");
    SP_REQUIRE(shape >= 0 && shape <= 2, "gemm_mfma: tile shape %d", shape);
    if (M == 0) return 0;
    if (shape == 0) shape = (offsets || M <= 128) ? 1 : 2;
    if (shape == 1)
        return launch_mfma<8, 1>(X, ldx, W, w_group_stride, Y, y_dtype, ldy, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, st);
    return launch_mfma<4, 2>(X, ldx, W, w_group_stride, Y, y_dtype, ldy, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, st);
}
