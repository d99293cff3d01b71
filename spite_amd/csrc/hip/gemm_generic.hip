// Plain tiled matrix product, Y = A . W^T, fp32 FMA with fp32 accumulation in ascending k:
// the true 32-bit path of every projection, and the bf16 path for shapes that the MFMA
// kernels refuse.  Each output element is one thread's private sum, so a row's result does
// not depend on which other rows share the call.
//
// Grouped form (experts): the rows of the call are `slots`; group g owns the slots
// [offsets[g], offsets[g+1]) and multiplies them with W + g*w_group_stride.  A slot reads
// row a_rows[s] of A (times a_scale[s], in fp32, before the product) and writes row
// y_rows[s] of Y.  With `glu` the group's W holds 2N rows, gate rows first, and the kernel
// writes silu(gate) * up.
#include "common.h"

#define GBM 64
#define GBN 64
#define GBK 16

template <typename T, typename TY, int GLU>
__global__ __launch_bounds__(256)
void gemm_generic_kernel(const T* __restrict__ A, int lda, const T* __restrict__ W, long w_group_stride,
                         TY* __restrict__ Y, int ldy, int M, int N, int K,
                         const int* __restrict__ offsets, int n_groups,
                         const int* __restrict__ a_rows, const float* __restrict__ a_scale,
                         const int* __restrict__ y_rows) {
    __shared__ float As[GBK][GBM + 1];
    __shared__ float Ws[GLU ? 2 : 1][GBK][GBN + 1];
    // ---- which group and which of its row tiles
    int g = 0, row0 = 0, row_end = M;
    if (offsets) {
        if (!sp_find_tile(offsets, n_groups, GBM, blockIdx.y, g, row0, row_end)) return;
    } else {
        row0 = blockIdx.y * GBM;
        if (row0 >= M) return;
    }
    const int n0 = blockIdx.x * GBN;
    const T* Wg = W + (size_t)g * w_group_stride;
    const int tid = threadIdx.x;
    const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
    float acc_g[4][4] = {}, acc_u[4][4] = {};

    const int lk = tid % GBK, lr = tid / GBK;   // loader: k index and first row (step 16)
    int a_src[4]; float a_sc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int s = row0 + lr + i * 16;
        if (s < row_end) { a_src[i] = a_rows ? a_rows[s] : s; a_sc[i] = a_scale ? a_scale[s] : 1.0f; }
        else { a_src[i] = -1; a_sc[i] = 0.f; }
    }
    for (int k0 = 0; k0 < K; k0 += GBK) {
        const int k = k0 + lk;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = lr + i * 16;
            float v = 0.f;
            if (a_src[i] >= 0 && k < K) v = to_f32<T>(A[(size_t)a_src[i] * lda + k]) * a_sc[i];
            As[lk][m] = v;
            const int n = n0 + m;
            float wv = 0.f, wu = 0.f;
            if (n < N && k < K) {
                wv = to_f32<T>(Wg[(size_t)n * K + k]);
                if (GLU) wu = to_f32<T>(Wg[(size_t)(N + n) * K + k]);
            }
            Ws[0][lk][m] = wv;
            if (GLU) Ws[1][lk][m] = wu;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GBK; ++kk) {
            float a[4], b[4], c[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[kk][tm + i]; b[i] = Ws[0][kk][tn + i]; if (GLU) c[i] = Ws[1][kk][tn + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc_g[i][j] = fmaf(a[i], b[j], acc_g[i][j]);
                    if (GLU) acc_u[i][j] = fmaf(a[i], c[j], acc_u[i][j]);
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int s = row0 + tm + i;
        if (s >= row_end) continue;
        const size_t yr = y_rows ? (size_t)y_rows[s] : (size_t)s;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tn + j;
            if (n >= N) continue;
            float v = acc_g[i][j];
            if (GLU) v = v / (1.0f + expf(-v)) * acc_u[i][j];
            Y[yr * ldy + n] = from_f32<TY>(v);
        }
    }
}

extern "C" int spite_gemm_generic(const void* A, int lda, const void* W, long w_group_stride, int dtype,
                                  void* Y, int y_dtype, int ldy, int M, int N, int K,
                                  const int* offsets, int n_groups, const int* a_rows,
                                  const float* a_scale, const int* y_rows, int glu, hipStream_t st) {
    SP_REQUIRE(M >= 0 && N > 0 && K > 0 && lda >= K && ldy >= N, "gemm: bad sizes M=%d N=%d K=%d lda=%d ldy=%d",
               M, N, K, lda, ldy);
    SP_REQUIRE(!offsets || n_groups > 0, "gemm: grouped call without groups");
    if (M == 0) return 0;
    // row tiles: a group with rows has 1 + (rows - 1) / tile of them, so groups with rows + M / tile bounds them
    const int m_tiles = offsets ? M / GBM + (n_groups < M ? n_groups : M) : (M + GBM - 1) / GBM;
    SP_REQUIRE(m_tiles <= 65535, "gemm: too many row tiles (%d)", m_tiles);
    dim3 grid((N + GBN - 1) / GBN, m_tiles);
#define SP_GEMM_LAUNCH(T, TY, GLU) gemm_generic_kernel<T, TY, GLU><<<grid, 256, 0, st>>>( \
        (const T*)A, lda, (const T*)W, w_group_stride, (TY*)Y, ldy, M, N, K, offsets, n_groups, a_rows, a_scale, y_rows)
    if (dtype == SP_F32 && y_dtype == SP_F32) { if (glu) SP_GEMM_LAUNCH(float, float, 1); else SP_GEMM_LAUNCH(float, float, 0); }
    else if (dtype == SP_BF16 && y_dtype == SP_BF16) { if (glu) SP_GEMM_LAUNCH(bf16, bf16, 1); else SP_GEMM_LAUNCH(bf16, bf16, 0); }
    else if (dtype == SP_BF16 && y_dtype == SP_F32) { if (glu) SP_GEMM_LAUNCH(bf16, float, 1); else SP_GEMM_LAUNCH(bf16, float, 0); }
    else return sp_fail("gemm: unsupported dtypes in=%d out=%d", dtype, y_dtype);
#undef SP_GEMM_LAUNCH
    SP_LAUNCH_CHECK("gemm_generic");
    return 0;
}
