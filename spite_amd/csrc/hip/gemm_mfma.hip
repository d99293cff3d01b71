// Tiled bf16 product for many rows (prefill): Y[M,N] = X[M,K] . W[N,K]^T on MFMA 16x16x32 with
// fp32 accumulation.  A workgroup of NW waves owns 128 rows of X (slots) and 256 rows of W;
// each wave owns 256/NW of the W rows and all 128 slots.
//
//  * W is the MFMA "A" operand and never touches LDS: a wave reads its own rows from global
//    memory straight into the operand layout (lane (r, q): 16 bytes of row r), the tile after
//    the current one already in flight in a second set of registers.  Where few rows meet a
//    weight (experts), the kernel is a stream of W at HBM speed, like the decode kernel.
//  * X is the "B" operand, shared by the four waves: its 128 x 64 tiles go through LDS (rows
//    padded by 16 bytes, so that the 16-byte operand reads of sixteen rows fall into sixteen
//    different bank groups), double-buffered, one barrier per tile.
//  * A lane ends with four consecutive columns n of one row m of Y.
//
// Grouped form (experts) and GLU as in gemm_generic.hip: a workgroup's slots lie inside one
// group; a slot's scale multiplies the fp32 sums; with GLU a wave's W rows are half gate rows
// and half the matching up rows.
#include "common.h"

#define MBM 128            // slots per workgroup
#define MBN 256            // W rows per workgroup
#define MBK 64
#define MLD (MBK + 8)      // padded row of the X tile in LDS, in elements

template <int NW, bool GLU, bool EXACT, typename TY>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_mfma_kernel(const bf16* __restrict__ X, int ldx, const bf16* __restrict__ W, long w_group_stride,
                      TY* __restrict__ Y, int ldy, int M, int N, int K,
                      const int* __restrict__ offsets, int n_groups, const int* __restrict__ a_rows,
                      const float* __restrict__ a_scale, const int* __restrict__ y_rows) {
    __shared__ __attribute__((aligned(16))) bf16 Xs[2][MBM * MLD];
    constexpr int NCOLS = GLU ? MBN / 2 : MBN;      // output columns per workgroup

    int g = 0, row0, row_end = M;
    if (offsets) {
        int mt = blockIdx.y, acc = 0;
        g = -1;
        for (int e = 0; e < n_groups; ++e) {
            const int b = offsets[e], en = offsets[e + 1];
            const int nt = (en - b + MBM - 1) / MBM;
            if (mt < acc + nt) { g = e; row0 = b + (mt - acc) * MBM; row_end = en; break; }
            acc += nt;
        }
        if (g < 0) return;
    } else {
        row0 = blockIdx.y * MBM;
        if (row0 >= M) return;
    }
    const int n0 = blockIdx.x * NCOLS;
    const bf16* Wg = W + (size_t)g * w_group_stride;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, q = lane >> 4;

    constexpr int TA = MBN / (NW * 16);      // W row tiles per wave
    constexpr int XL = 1024 / (NW * 64);     // 16-byte chunks of the X tile per thread
    constexpr int XR = NW * 8;               // rows of the X tile that one pass of the threads covers
    // ---- X: global -> registers -> LDS; thread loads 16-byte chunk (tid % 8) of rows tid/8 + XR*i
    const int lrow = tid >> 3, lchunk = tid & 7;
    const bf16* xsrc[XL];
#pragma unroll
    for (int i = 0; i < XL; ++i) {
        // rows past the group read its last row again: the loads of the main loop carry no
        // condition (a select on a loaded value would make the wave wait for it at once), and
        // what such rows produce is never stored
        int s = row0 + lrow + XR * i;
        s = s < row_end ? s : row_end - 1;
        xsrc[i] = X + (size_t)(a_rows ? a_rows[s] : s) * ldx;
    }
    // ---- W: the wave's TA row tiles; lane (r, q) reads row r of each
    //      plain: rows n0 + wave*16*TA + a*16; GLU: the first TA/2 tiles gate rows, the others the up rows N + ...
    constexpr int TG = GLU ? TA / 2 : TA;    // tiles that name distinct output columns
    const bf16* wsrc[TA];
    int ncol[TA];           // output column of the tile's first row
#pragma unroll
    for (int a = 0; a < TA; ++a) {
        const int n = n0 + wave * 16 * TG + (a % TG) * 16;
        const int nr = (n + r) < N ? n + r : N - 1;
        const size_t grow = ((GLU && a >= TG) ? (size_t)N : 0) + nr;
        ncol[a] = n;
        wsrc[a] = Wg + grow * K;
    }
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8 xr[XL];
    bf16x8 w0[TA][2], w1[TA][2];     // W operands of the even and of the odd tiles: [row tile][32-wide k step]
    // EXACT: K is a multiple of the tile, no load carries a condition.  Otherwise chunks past
    // K are zero (K is a multiple of 8); that form is slower and only serves odd widths.
    auto load_x = [&](int k0) {
        const int k = k0 + lchunk * 8;
#pragma unroll
        for (int i = 0; i < XL; ++i) xr[i] = (EXACT || k < K) ? *(const bf16x8*)(xsrc[i] + k) : zero;
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int i = 0; i < XL; ++i) *(bf16x8*)(Xs[buf] + (lrow + XR * i) * MLD + lchunk * 8) = xr[i];
    };
    auto load_w = [&](bf16x8 (&ws)[TA][2], int k0) {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const int k = k0 + kk * 32 + q * 8;
#pragma unroll
            for (int a = 0; a < TA; ++a) ws[a][kk] = (EXACT || k < K) ? *(const bf16x8*)(wsrc[a] + k) : zero;
        }
    };

    f32x4 acc[TA][8];       // [W row tile a][slot tile b]
#pragma unroll
    for (int a = 0; a < TA; ++a)
#pragma unroll
        for (int b = 0; b < 8; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
    auto mul = [&](bf16x8 (&ws)[TA][2], int buf) {
        const bf16* xs = Xs[buf];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                bf16x8 xf[4];
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    xf[b] = *(const bf16x8*)(xs + ((half * 4 + b) * 16 + r) * MLD + kk * 32 + q * 8);
#pragma unroll
                for (int a = 0; a < TA; ++a)
#pragma unroll
                    for (int b = 0; b < 4; ++b)
                        acc[a][half * 4 + b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ws[a][kk], xf[b], acc[a][half * 4 + b], 0, 0, 0);
            }
        }
    };

    // Tile t is multiplied out of Xs[t & 1] and w0 (t even) or w1 (t odd) while tile t+1 is
    // in flight: its X chunks into registers (stored to the other LDS buffer after the
    // products), its W operands into the other register set.
    const int nt = (K + MBK - 1) / MBK;
    load_x(0);
    load_w(w0, 0);
    store_x(0);
    __syncthreads();
    int t = 0;
    for (; t + 2 < nt; t += 2) {                 // steady state: no condition inside
        load_x((t + 1) * MBK); load_w(w1, (t + 1) * MBK);
        __builtin_amdgcn_sched_barrier(0);
        mul(w0, 0);
        store_x(1);
        __syncthreads();
        load_x((t + 2) * MBK); load_w(w0, (t + 2) * MBK);
        __builtin_amdgcn_sched_barrier(0);
        mul(w1, 1);
        store_x(0);
        __syncthreads();
    }
    if (t + 1 < nt) {                            // two tiles left
        load_x((t + 1) * MBK); load_w(w1, (t + 1) * MBK);
        __builtin_amdgcn_sched_barrier(0);
        mul(w0, 0);
        store_x(1);
        __syncthreads();
        mul(w1, 1);
    } else {                                     // one tile left
        mul(w0, 0);
    }

    // acc[a][b][i] of lane (r, q): column ncol[a] + q*4 + i, slot row0 + b*16 + r
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const int s = row0 + b * 16 + r;
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
            for (int a = 0; a < TA; ++a) {
                const int n = ncol[a] + q * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) yrow[n + i] = from_f32<TY>(acc[a][b][i] * sc);
            }
        }
    }
}

extern "C" int spite_gemm_mfma(const void* X, int ldx, const void* W, long w_group_stride, void* Y, int y_dtype,
                               int ldy, int M, int N, int K, const int* offsets, int n_groups, const int* a_rows,
                               const float* a_scale, const int* y_rows, int glu, hipStream_t st) {
    SP_REQUIRE(M >= 0 && N > 0 && K > 0 && ldx >= K && ldy >= N, "gemm_mfma: bad sizes M=%d N=%d K=%d", M, N, K);
    SP_REQUIRE(K % 8 == 0 && ldx % 8 == 0, "gemm_mfma: K=%d and the row stride %d must be multiples of 8", K, ldx);
    SP_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_mfma: operands must be 16-byte aligned");
    SP_REQUIRE(y_dtype == SP_BF16 || y_dtype == SP_F32, "gemm_mfma: output dtype %d", y_dtype);
    SP_REQUIRE(!offsets || n_groups > 0, "gemm_mfma: grouped call without groups");
    if (M == 0) return 0;
    const int m_tiles = (M + MBM - 1) / MBM + (offsets ? n_groups : 0);
    SP_REQUIRE(m_tiles <= 65535, "gemm_mfma: too many row tiles (%d)", m_tiles);
    const int ncols = glu ? MBN / 2 : MBN;
    dim3 grid((N + ncols - 1) / ncols, m_tiles);
#define SP_MM(GLUV, TY) do { if (K % MBK == 0) gemm_mfma_kernel<8, GLUV, true, TY><<<grid, 512, 0, st>>>((const bf16*)X, ldx, \
        (const bf16*)W, w_group_stride, (TY*)Y, ldy, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows); \
    else gemm_mfma_kernel<8, GLUV, false, TY><<<grid, 512, 0, st>>>((const bf16*)X, ldx, (const bf16*)W, \
        w_group_stride, (TY*)Y, ldy, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows); } while (0)
    if (glu) { if (y_dtype == SP_BF16) SP_MM(true, bf16); else SP_MM(true, float); }
    else { if (y_dtype == SP_BF16) SP_MM(false, bf16); else SP_MM(false, float); }
#undef SP_MM
    SP_LAUNCH_CHECK("gemm_mfma");
    return 0;
}
