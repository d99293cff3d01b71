// Shared declarations of the gfx950 kernel library: element types, error reporting,
// wave-level reductions.  Everything here is written for 64-wide wavefronts.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

typedef __bf16 bf16;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

enum { SP_F32 = 0, SP_BF16 = 1 };
// Which keys a query may read besides the causal rule j <= p: shared with the cache manager.
#define SP_VIS_FN __device__ __host__ __forceinline__
#include "../visibility.h"

#define SP_WAVE 64

// ---- error reporting: every entry point returns 0 or a negative code, and the text of the
// last failure of the calling thread is kept for spite_hip_last_error().
int sp_fail(const char* fmt, ...);
#define SP_REQUIRE(cond, ...) do { if (!(cond)) return sp_fail(__VA_ARGS__); } while (0)
// Compute units of the current device (asked once per device): what tile counts are weighed against.
int sp_cu_count();
// attn_decode.hip: joins the records that split attention leaves (see there).
int sp_attn_combine(const float* part, void* out, int T, int H, int hd, int n_splits, hipStream_t st);
#define SP_LAUNCH_CHECK(name) do { hipError_t e_ = hipGetLastError(); \
    if (e_ != hipSuccess) return sp_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); } while (0)


// ---- layouts of one kv head's part of a cache page.
// Row-major: keys [page_size][hd], values transposed [hd][page_size].
// Operand order (bf16, hd % 32 == 0, page_size % 32 == 0): the MFMA attention kernels' operand
// tiles, each one kilobyte in lane order, so that a wave's load is a run of whole cache lines.
//   keys:   blocks of 32 keys; block b holds two tiles tt of 16 rows, row r of tile tt being the
//           key (r/4)*8 + tt*4 + r%4 of the block, each tile cut into hd/32 chunks cc of 32
//           elements: tile (b, tt, cc) at ((b*2 + tt) * hd/32 + cc) * 512, inside it element
//           8q+e of row r at (q*16 + r)*8 + e.
//   values: block b, 16 head elements dt*16 .. dt*16+15 as rows, the block's 32 keys as k:
//           tile (b, dt) at (b * hd/16 + dt) * 512, inside it key 8q+e of row r at (q*16 + r)*8 + e.
__device__ __forceinline__ size_t sp_k_index(int off, int c, int hd, bool tiled) {
    if (!tiled) return (size_t)off * hd + c;
    const int b = off >> 5, w = off & 31;
    const int r = ((w >> 3) << 2) | (w & 3), tt = (w >> 2) & 1;
    return ((size_t)(b * 2 + tt) * (hd >> 5) + (c >> 5)) * 512 + (size_t)(((((c & 31) >> 3) << 4) + r) << 3) + (c & 7);
}
__device__ __forceinline__ size_t sp_v_index(int c, int off, int hd, int ps, bool tiled) {
    if (!tiled) return (size_t)c * ps + off;
    const int b = off >> 5, w = off & 31;
    return ((size_t)b * (hd >> 4) + (c >> 4)) * 512 + (size_t)((((w >> 3) << 4) + (c & 15)) << 3) + (w & 7);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Which group and which rows the row tile `mt` of a grouped product covers.  Groups are walked
// in order, group e bringing ceil((offsets[e+1] - offsets[e]) / MT) tiles of MT rows.  A wave
// looks at 64 groups at a time (a prefix sum over its lanes), so that hundreds of groups cost a
// few steps; every lane of the wave must call it and gets the same answer.  False: mt lies
// past the last tile.
__device__ __forceinline__ bool sp_find_tile(const int* offsets, int n_groups, int MT, int mt,
                                             int& g, int& row0, int& row_end) {
    const int lane = threadIdx.x & 63;
    int base = 0;
    for (int c = 0; c < n_groups; c += 64) {
        const int e = c + lane;
        int b = 0, en = 0;
        if (e < n_groups) { b = offsets[e]; en = offsets[e + 1]; }
        const int nt = (en - b + MT - 1) / MT;
        int incl = nt;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { const int v = __shfl_up(incl, o, 64); if (lane >= o) incl += v; }
        const int total = __shfl(incl, 63, 64);
        if (mt < base + total) {
            const bool mine = mt >= base + incl - nt && mt < base + incl;
            const int src = __ffsll((unsigned long long)__ballot(mine)) - 1;
            // the same in every lane: say so, to keep them in scalar registers
            g = __builtin_amdgcn_readfirstlane(c + src);
            row0 = __builtin_amdgcn_readfirstlane(__shfl(b, src, 64) + (mt - base - __shfl(incl - nt, src, 64)) * MT);
            row_end = __builtin_amdgcn_readfirstlane(__shfl(en, src, 64));
            return true;
        }
        base += total;
    }
    return false;
}

// Maximum / sum over the four lanes n, n+16, n+32, n+48 of a wave (the four rows of 16 lanes that
// hold one MFMA column), the result in all four.  The row swaps are vector instructions: no
// trip through the LDS crossbar as a shuffle across rows takes.
__device__ __forceinline__ float rows4_max(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float rows4_sum(float v) {
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Sum over a workgroup of NT threads (NT a multiple of 64, at most 1024); every thread
// gets the result.  `red` is shared scratch of at least NT/64 floats; two barriers.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NT / 64; ++i) t += red[i];
    __syncthreads();
    return t;
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16>(bf16 v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return (bf16)v; }
