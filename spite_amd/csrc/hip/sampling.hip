// Token choice from fp32 logits rows: arg-max (the lowest index wins a tie) and the
// inverse-CDF draw of crates/spite-sampling/src/lib.rs:247-265 (m = max, total = sum
// exp(l-m), the first index whose running sum reaches u*total, arg-max if rounding leaves
// none).  One workgroup per row; each thread owns one contiguous slice of the row, so the
// running sum walks the row in index order.
#include "common.h"

#define SAMP_NT 1024

__device__ __forceinline__ void argmax_combine(float& v, int& i, float ov, int oi) {
    if (oi >= 0 && (i < 0 || ov > v || (ov == v && oi < i))) { v = ov; i = oi; }
}

// Block-wide arg-max of (v, i) pairs; i < 0 means "nothing".  Result valid in every thread.
__device__ void block_argmax(float& v, int& i, float* sv, int* si) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o, 64);
        const int oi = __shfl_xor(i, o, 64);
        argmax_combine(v, i, ov, oi);
    }
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { sv[w] = v; si[w] = i; }
    __syncthreads();
    v = sv[0]; i = si[0];
    for (int k = 1; k < SAMP_NT / 64; ++k) argmax_combine(v, i, sv[k], si[k]);
    __syncthreads();
}

__global__ __launch_bounds__(SAMP_NT)
void sample_rows_kernel(const float* __restrict__ logits, int ld, int V, const float* __restrict__ temperature,
                        const float* __restrict__ uniform, int* __restrict__ out) {
    __shared__ float sv[SAMP_NT / 64];
    __shared__ int si[SAMP_NT / 64];
    __shared__ float part[SAMP_NT];
    __shared__ int found;
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)r * ld;
    const float temp = temperature ? temperature[r] : 0.f;
    const int per = (V + SAMP_NT - 1) / SAMP_NT;
    const int b = tid * per, e = (b + per < V) ? b + per : V;

    // arg-max: neighbouring threads read neighbouring elements; a thread meets its indices in
    // rising order, so "greater than" keeps the lowest index of equal values
    float bv = 0.f; int bi = -1;
    for (int i = tid; i < V; i += SAMP_NT) {
        const float x = row[i];
        if (bi < 0 || x > bv) { bv = x; bi = i; }
    }
    block_argmax(bv, bi, sv, si);
    if (temp <= 0.f) { if (tid == 0) out[r] = bi; return; }

    // masses relative to the maximum of l/temperature
    const float mx = bv / temp;
    float s = 0.f;
    for (int i = b; i < e; ++i) s += expf(row[i] / temp - mx);
    part[tid] = s;
    if (tid == 0) found = 0x7fffffff;
    __syncthreads();
    float excl = 0.f, total = 0.f;
    for (int k = 0; k < SAMP_NT; ++k) { if (k == tid) excl = total; total += part[k]; }
    const float target = uniform[r] * total;
    // Every slice that starts below the target walks on from the sum of the slices before
    // it; the lowest index that reaches the target is the answer.
    if (b < e && (tid == 0 || excl < target)) {
        float cum = excl;
        for (int i = b; i < e; ++i) {
            cum += expf(row[i] / temp - mx);
            if (cum >= target) { atomicMin(&found, i); break; }
        }
    }
    __syncthreads();
    if (tid == 0) out[r] = found != 0x7fffffff ? found : bi;
}

// Arg-max in two stages when no row draws: the row is cut into slices, a workgroup finds the
// best of its slice, a second kernel the best of the slices (lowest index among equals).
#define ARG_SLICES 32
__global__ __launch_bounds__(256)
void argmax_slices_kernel(const float* __restrict__ logits, int ld, int V, float* __restrict__ pv, int* __restrict__ pi) {
    __shared__ float sv[4];
    __shared__ int si[4];
    const int r = blockIdx.y, sl = blockIdx.x, tid = threadIdx.x;
    const int per = (V + ARG_SLICES - 1) / ARG_SLICES;
    const int b = sl * per, e = (b + per < V) ? b + per : V;
    const float* row = logits + (size_t)r * ld;
    float bv = 0.f; int bi = -1;
#pragma unroll 4
    for (int i = b + tid; i < e; i += 256) {
        const float x = row[i];
        if (bi < 0 || x > bv) { bv = x; bi = i; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        argmax_combine(bv, bi, ov, oi);
    }
    if ((tid & 63) == 0) { sv[tid >> 6] = bv; si[tid >> 6] = bi; }
    __syncthreads();
    if (tid == 0) {
        for (int k = 1; k < 4; ++k) argmax_combine(bv, bi, sv[k], si[k]);
        pv[r * ARG_SLICES + sl] = bv; pi[r * ARG_SLICES + sl] = bi;
    }
}
__global__ void argmax_final_kernel(const float* __restrict__ pv, const int* __restrict__ pi, int* __restrict__ out) {
    const int r = blockIdx.x;
    float bv = pv[r * ARG_SLICES + threadIdx.x]; int bi = pi[r * ARG_SLICES + threadIdx.x];
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        argmax_combine(bv, bi, ov, oi);
    }
    if (threadIdx.x == 0) out[r] = bi;
}

// `scratch`: n_rows * 32 floats and as many ints, for the two-stage arg-max (may be null:
// then one workgroup walks each row).
extern "C" int spite_argmax_rows(const float* logits, int ld, int n_rows, int V, float* scratch_v, int* scratch_i,
                                 int* out, hipStream_t st) {
    SP_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "argmax: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
    SP_REQUIRE(n_rows <= 65535, "argmax: too many rows");
    if (n_rows == 0) return 0;
    argmax_slices_kernel<<<dim3(ARG_SLICES, n_rows), 256, 0, st>>>(logits, ld, V, scratch_v, scratch_i);
    SP_LAUNCH_CHECK("argmax_slices");
    argmax_final_kernel<<<n_rows, ARG_SLICES, 0, st>>>(scratch_v, scratch_i, out);
    SP_LAUNCH_CHECK("argmax_final");
    return 0;
}

extern "C" int spite_sample_rows(const float* logits, int ld, int n_rows, int V, const float* temperature,
                                 const float* uniform, int* out, hipStream_t st) {
    SP_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "sample: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
    SP_REQUIRE(!temperature || uniform, "sample: temperatures without uniform draws");
    if (n_rows == 0) return 0;
    sample_rows_kernel<<<n_rows, SAMP_NT, 0, st>>>(logits, ld, V, temperature, uniform, out);
    SP_LAUNCH_CHECK("sample_rows");
    return 0;
}
