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
// Which keys a query may read besides the causal rule j <= p.
enum { SP_VIS_FULL = 0, SP_VIS_CHUNK = 1, SP_VIS_WINDOW = 2 };

#define SP_WAVE 64

// ---- error reporting: every entry point returns 0 or a negative code, and the text of the
// last failure of the calling thread is kept for spite_hip_last_error().
int sp_fail(const char* fmt, ...);
#define SP_REQUIRE(cond, ...) do { if (!(cond)) return sp_fail(__VA_ARGS__); } while (0)
#define SP_LAUNCH_CHECK(name) do { hipError_t e_ = hipGetLastError(); \
    if (e_ != hipSuccess) return sp_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); } while (0)

// First position a query at p may read (the last is p itself).
__device__ __forceinline__ int sp_first_visible(int p, int vis, int span) {
    if (vis == SP_VIS_CHUNK) return (p / span) * span;
    if (vis == SP_VIS_WINDOW) return p - span + 1 > 0 ? p - span + 1 : 0;
    return 0;
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
