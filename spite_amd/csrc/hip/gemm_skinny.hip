// Weight-streaming product for few rows (decode): Y[M,N] = X[M,K] . W[N,K]^T, bf16 in, fp32
// accumulate on MFMA 16x16x32, for M up to a few dozen.  The time goes into reading W once
// at HBM speed, so the shape of the kernel is the shape of that stream:
//
//  * A workgroup owns 16*R rows of W (R MFMA tiles) and all of K; its NW waves take the
//    128-element blocks of K in turn (wave w: blocks w, w+NW, ...) and their partial sums
//    meet in LDS.  Small N times large K still gives thousands of waves, each with several
//    16-byte loads per lane in flight.
//  * W is the MFMA "A" operand (rows of W = rows of the tile), X the "B" operand (tokens =
//    columns).  MFMA does not care in which order k runs as long as both operands agree, so
//    lane (row r, quarter q) reads 8*S consecutive elements W[r][kb + q*8S ..]: every row is
//    read in runs of 64*S bytes.  (Plain loads: a 128-byte line is shared by two load
//    instructions, and non-temporal loads were measured to fetch it twice.  In operand order,
//    where a load instruction takes whole lines, non-temporal loads are used: the stream of W
//    is read once and runs a tenth faster when it does not displace what the caches hold.)
//  * Grouped form (experts): see gemm_generic.hip.  A slot's scale multiplies the fp32 sums
//    (W.(s x) = s (W.x)), so the scaled input is never rounded.  With GLU the workgroup also
//    owns the matching "up" rows N+n and writes silu(gate) * up.
//
//  * TILED: W lies in MFMA operand order (see gemm_tiled.hip: tiles of 16 rows x 32 k, each
//    one kilobyte in lane order).  A lane's loads are then the tile's 16 bytes at lane * 16,
//    and k runs q*8 .. q*8+7 inside every 32: X is read to match.
//
// Within one instantiation a row's sum runs over k in an order that does not depend on M or on
// the other rows.  The caller picks the instantiation (S, and above 64 rows another kernel) from
// the number of rows, so across step sizes a bfloat16 product agrees only to rounding; the
// 32-bit path's products (gemm_generic.hip) give the same bits for every batch.
#include "common.h"

template <int R, int G, int S, int NW, bool GLU, bool TILED, typename TY>
__global__ __launch_bounds__(NW * 64)
void gemm_skinny_kernel(const bf16* __restrict__ X, int ldx, const bf16* __restrict__ W, long w_group_stride,
                        TY* __restrict__ Y, int ldy, int M, int N, int K,
                        const int* __restrict__ offsets, int n_groups, const int* __restrict__ a_rows,
                        const float* __restrict__ a_scale, const int* __restrict__ y_rows) {
    constexpr int RA = GLU ? 2 * R : R;        // A tiles per wave
    constexpr int KB = 32 * S;                 // k elements per block
    constexpr int J = RA * G * 4;              // partial sums per lane
    constexpr int MT = 16 * G;                 // slots per workgroup
    extern __shared__ float red[];             // [NW][J][64]

    int g = 0, row0, row_end = M;
    if (offsets) {
        if (!sp_find_tile(offsets, n_groups, MT, blockIdx.y, g, row0, row_end)) return;
    } else {
        row0 = blockIdx.y * MT;
        if (row0 >= M) return;
    }
    const int n0 = blockIdx.x * (16 * R);
    const bf16* Wg = W + (size_t)g * w_group_stride;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, q = lane >> 4;

    const bf16* wp[RA];
#pragma unroll
    for (int a = 0; a < RA; ++a) {
        // rows past N read row N-1 again, slots past the group its last slot: the loads of
        // the main loop carry no condition (a select on a loaded value would make the wave
        // wait for it at once), lanes with one address are served by one request, and what
        // such rows produce is never stored
        int n = n0 + (a % R) * 16 + r;
        n = n < N ? n : N - 1;
        const size_t row = (GLU && a >= R) ? (size_t)N + n : (size_t)n;
        if (TILED) wp[a] = Wg + (row / 16) * (size_t)(K / 32) * 512 + lane * 8;     // the row's band; N % 16 == 0
        else wp[a] = Wg + row * K;
    }
    const bf16* xp[G];
#pragma unroll
    for (int b = 0; b < G; ++b) {
        int s = row0 + b * 16 + r;
        s = s < row_end ? s : row_end - 1;
        xp[b] = X + (size_t)(a_rows ? a_rows[s] : s) * ldx;
    }

    f32x4 acc[RA][G];
#pragma unroll
    for (int a = 0; a < RA; ++a)
#pragma unroll
        for (int b = 0; b < G; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    // Two register buffers, named apart so that every index is a constant: block i+1 is in
    // flight while block i is multiplied.
    bf16x8 wa0[RA][S], xb0[G][S], wa1[RA][S], xb1[G][S];
    auto load = [&](bf16x8 (&wa)[RA][S], bf16x8 (&xb)[G][S], int kb) {
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const int k = TILED ? kb + s * 32 + q * 8 : kb + q * (8 * S) + s * 8;
            const size_t kw = TILED ? (size_t)(kb / 32 + s) * 512 : (size_t)k;
#pragma unroll
            for (int a = 0; a < RA; ++a) wa[a][s] = TILED ? __builtin_nontemporal_load((const bf16x8*)(wp[a] + kw)) : *(const bf16x8*)(wp[a] + kw);
#pragma unroll
            for (int b = 0; b < G; ++b) xb[b][s] = *(const bf16x8*)(xp[b] + k);
        }
    };
    // the last block when K is no multiple of the block: chunks past K are zero (K % 8 == 0)
    auto load_tail = [&](bf16x8 (&wa)[RA][S], bf16x8 (&xb)[G][S], int kb) {
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const int k = TILED ? kb + s * 32 + q * 8 : kb + q * (8 * S) + s * 8;
            const size_t kw = TILED ? (size_t)(kb / 32 + s) * 512 : (size_t)k;
#pragma unroll
            for (int a = 0; a < RA; ++a) wa[a][s] = k < K ? *(const bf16x8*)(wp[a] + kw) : zero;
#pragma unroll
            for (int b = 0; b < G; ++b) xb[b][s] = k < K ? *(const bf16x8*)(xp[b] + k) : zero;
        }
    };
    auto mul = [&](bf16x8 (&wa)[RA][S], bf16x8 (&xb)[G][S]) {
#pragma unroll
        for (int s = 0; s < S; ++s)
#pragma unroll
            for (int a = 0; a < RA; ++a)
#pragma unroll
                for (int b = 0; b < G; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[a][s], xb[b][s], acc[a][b], 0, 0, 0);
    };
    constexpr int STEP = NW * KB;
    const int k_full = K / KB * KB;            // whole blocks end here
    int kb = wave * KB;
    if (kb < k_full) load(wa0, xb0, kb);
    while (kb < k_full) {
        if (kb + STEP < k_full) load(wa1, xb1, kb + STEP);
        mul(wa0, xb0);
        kb += STEP;
        if (kb >= k_full) break;
        if (kb + STEP < k_full) load(wa0, xb0, kb + STEP);
        mul(wa1, xb1);
        kb += STEP;
    }
    if (k_full < K && wave == (k_full / KB) % NW) {   // the partial block goes to the wave whose turn it is
        load_tail(wa0, xb0, k_full);
        mul(wa0, xb0);
    }

    // partial sums of the waves meet in LDS: red[wave][j][lane]
#pragma unroll
    for (int a = 0; a < RA; ++a)
#pragma unroll
        for (int b = 0; b < G; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                red[(wave * J + (a * G + b) * 4 + i) * 64 + lane] = acc[a][b][i];
    __syncthreads();
    // acc[a][b][i] of lane (r, q) is the element (row n0 + a*16 + q*4 + i, slot row0 + b*16 + r)
    constexpr int JO = R * G * 4;              // outputs per lane position (gate and up fold into one)
    for (int o = threadIdx.x; o < JO * 64; o += NW * 64) {
        const int j = o >> 6, l = o & 63;
        const int a = j / (G * 4), b = (j / 4) % G, i = j & 3;
        const int n = n0 + a * 16 + (l >> 4) * 4 + i;
        const int s = row0 + b * 16 + (l & 15);
        if (n >= N || s >= row_end) continue;
        float v = 0.f, u = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            v += red[(w * J + j) * 64 + l];
            if (GLU) u += red[(w * J + j + JO) * 64 + l];
        }
        if (a_scale) { const float sc = a_scale[s]; v *= sc; u *= sc; }
        if (GLU) v = v / (1.0f + __expf(-v)) * u;
        const size_t yr = y_rows ? (size_t)y_rows[s] : (size_t)s;
        Y[yr * ldy + n] = from_f32<TY>(v);
    }
}

template <int R, int G, int S, int NW>
static int launch_skinny(const void* X, int ldx, const void* W, long wgs, void* Y, int y_dtype, int ldy, int M, int N,
                         int K, const int* offsets, int n_groups, const int* a_rows, const float* a_scale,
                         const int* y_rows, int glu, int tiled, int live_groups, hipStream_t st) {
    const int MT = 16 * G;
    // row tiles: a group with rows has 1 + (rows - 1) / MT of them, so (groups with rows) + M / MT bounds them.
    // A workgroup of a tile that does not exist leaves at once, but only after it was given its registers:
    // with 128 groups of which 2 hold rows those were two thirds of the kernel's time.
    int live = n_groups < M ? n_groups : M;
    if (live_groups > 0 && live_groups < live) live = live_groups;
    const int m_tiles = offsets ? M / MT + live : (M + MT - 1) / MT;
    SP_REQUIRE(m_tiles <= 65535, "gemm_skinny: too many row tiles (%d)", m_tiles);
    dim3 grid((N + 16 * R - 1) / (16 * R), m_tiles);
    const size_t sh = (size_t)NW * (glu ? 2 : 1) * R * G * 4 * 64 * sizeof(float);
#define SP_SK(GLUV, TY) do { \
        auto kern = tiled ? gemm_skinny_kernel<R, G, S, NW, GLUV, true, TY> : gemm_skinny_kernel<R, G, S, NW, GLUV, false, TY>; \
        if (sh > 48 * 1024) { hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh); \
            if (e != hipSuccess) return sp_fail("gemm_skinny: cannot get %zu bytes of LDS: %s", sh, hipGetErrorString(e)); } \
        kern<<<grid, NW * 64, sh, st>>>((const bf16*)X, ldx, (const bf16*)W, wgs, (TY*)Y, ldy, M, N, K, offsets, \
                                        n_groups, a_rows, a_scale, y_rows); } while (0)
    if (glu) { if (y_dtype == SP_BF16) SP_SK(true, bf16); else SP_SK(true, float); }
    else { if (y_dtype == SP_BF16) SP_SK(false, bf16); else SP_SK(false, float); }
#undef SP_SK
    SP_LAUNCH_CHECK("gemm_skinny");
    return 0;
}

// `max_rows`: the most rows any group brings (M itself for a plain product); picks how many
// token columns a workgroup carries.  `live_groups`: the caller's promise that no more groups than
// this hold rows (0: no promise); the grid is cut to the row tiles that can exist.
extern "C" int spite_gemm_skinny(const void* X, int ldx, const void* W, long w_group_stride, void* Y, int y_dtype,
                                 int ldy, int M, int N, int K, const int* offsets, int n_groups, const int* a_rows,
                                 const float* a_scale, const int* y_rows, int glu, int max_rows, int variant,
                                 int w_tiled, int live_groups, hipStream_t st) {
    SP_REQUIRE(M >= 0 && N > 0 && K > 0 && ldx >= K && ldy >= N, "gemm_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
    SP_REQUIRE(K % 8 == 0 && ldx % 8 == 0, "gemm_skinny: K=%d and the row stride %d must be multiples of 8", K, ldx);
    SP_REQUIRE(((uintptr_t)X & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_skinny: operands must be 16-byte aligned");
    SP_REQUIRE(y_dtype == SP_BF16 || y_dtype == SP_F32, "gemm_skinny: output dtype %d", y_dtype);
    SP_REQUIRE(!offsets || n_groups > 0, "gemm_skinny: grouped call without groups");
    SP_REQUIRE(!w_tiled || (K % 32 == 0 && N % 16 == 0), "gemm_skinny: operand order needs K=%d a multiple of 32 and N=%d of 16", K, N);
    if (M == 0) return 0;
#define SP_ARGS X, ldx, W, w_group_stride, Y, y_dtype, ldy, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows, glu, w_tiled, live_groups, st
    // measured on MI355X (GB/s of W at Llama 4 Scout's shapes): one row tile per workgroup for
    // the experts' grouped stream, two for the dense projections, four for the output matrix
    if (variant == 0) {
        // (with one or two tokens only a few groups have rows at all: more rows of W a workgroup)
        if (max_rows <= 16) {
            if (offsets) variant = glu ? 8 : (max_rows <= 2 ? 7 : 6);
            else if ((size_t)N * K >= ((size_t)1 << 28)) variant = max_rows <= 8 ? 4 : 7;
            else variant = 8;
        }
        else if (max_rows <= 32) variant = !offsets && (size_t)N * K >= ((size_t)1 << 28) ? 10 : 2;
        // (groups of experts at 33 to 64 tokens hold a few rows each, only the shared one all:
        // 32 columns a workgroup and a second row tile for that group beat 64 columns for all)
        else if (offsets) variant = glu ? 2 : 10;
        // (a plain product's time grows with the tokens, whose rows every workgroup reads from
        // L2 beside its rows of W: from about 50 tokens on, 64 rows of W a workgroup with two row
        // tiles of 32 columns beat 32 rows of W with all 64 columns)
        else variant = max_rows > 48 ? 10 : 9;
    }
    switch (variant) {
        case 2: return launch_skinny<2, 2, 2, 8>(SP_ARGS);
        case 3: return launch_skinny<2, 4, 2, 4>(SP_ARGS);
        case 4: return launch_skinny<2, 1, 4, 8>(SP_ARGS);
        case 6: return launch_skinny<1, 1, 2, 8>(SP_ARGS);
        case 7: return launch_skinny<4, 1, 2, 8>(SP_ARGS);
        case 8: return launch_skinny<2, 1, 2, 8>(SP_ARGS);
        case 9: return launch_skinny<2, 4, 2, 8>(SP_ARGS);
        case 10: return launch_skinny<4, 2, 2, 8>(SP_ARGS);
        default: return sp_fail("gemm_skinny: unknown variant %d", variant);
    }
#undef SP_ARGS
}
