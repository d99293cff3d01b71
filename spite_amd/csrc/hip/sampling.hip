// Token choice from fp32 logits rows: arg-max (the lowest index wins a tie) and the
// inverse-CDF draw of crates/spite-sampling/src/lib.rs:247-265 (m = max, total = sum
// exp(l-m), the first index whose running sum reaches u*total, arg-max if rounding leaves
// none).  One workgroup per row.
#include "common.h"
#include <type_traits>

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

// The draw: masses exp(l/T - max) are summed over spans of SAMP_SPAN consecutive elements, a
// span by one wave (sixteen loads of 64 neighbouring elements, one sum across the lanes), the
// spans in index order; the first span, then the first run of 64 in it, then the first element
// at which the running sum reaches u * total is the answer.
#define SAMP_SPAN 1024
__global__ __launch_bounds__(SAMP_NT)
void sample_rows_kernel(const float* __restrict__ logits, int ld, int V, const float* __restrict__ temperature,
                        const float* __restrict__ uniform, int* __restrict__ out) {
    __shared__ float sv[SAMP_NT / 64];
    __shared__ int si[SAMP_NT / 64];
    __shared__ int at_span;
    __shared__ float before, goal;
    extern __shared__ float span_sum[];             // [spans]
    const int r = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float* row = logits + (size_t)r * ld;
    const float temp = temperature ? temperature[r] : 0.f;

    // arg-max: neighbouring threads read neighbouring elements; a thread meets its indices in
    // rising order, so "greater than" keeps the lowest index of equal values
    float bv = 0.f; int bi = -1;
    for (int base = tid; base < V; base += 16 * SAMP_NT) {       // sixteen loads in flight
        float x[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int i = base + u * SAMP_NT;
            x[u] = i < V ? row[i] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            const int i = base + u * SAMP_NT;
            if (i < V && (bi < 0 || x[u] > bv)) { bv = x[u]; bi = i; }
        }
    }
    block_argmax(bv, bi, sv, si);
    if (temp <= 0.f) { if (tid == 0) out[r] = bi; return; }

    const float mx = bv / temp;
    const int n_spans = (V + SAMP_SPAN - 1) / SAMP_SPAN;
    for (int sp = wave; sp < n_spans; sp += SAMP_NT / 64) {
        float x[SAMP_SPAN / 64];
#pragma unroll
        for (int u = 0; u < SAMP_SPAN / 64; ++u) {
            const int i = sp * SAMP_SPAN + u * 64 + lane;
            x[u] = i < V ? row[i] : -INFINITY;
        }
        float s = 0.f;
#pragma unroll
        for (int u = 0; u < SAMP_SPAN / 64; ++u) s += expf(x[u] / temp - mx);      // (exp(-inf) = 0 past the end)
        s = wave_sum(s);
        if (lane == 0) span_sum[sp] = s;
    }
    __syncthreads();
    if (tid == 0) {
        float total = 0.f;
        for (int sp = 0; sp < n_spans; ++sp) total += span_sum[sp];
        const float target = uniform[r] * total;
        float cum = 0.f;
        int sp = 0;
        while (sp < n_spans - 1 && cum + span_sum[sp] < target) cum += span_sum[sp++];
        at_span = sp; before = cum; goal = target;
    }
    __syncthreads();
    if (wave == 0) {
        // inside the span: run by run, the running sum over a run's lanes in index order
        float cum = before;
        int found = -1;
        for (int u = 0; u < SAMP_SPAN / 64 && found < 0; ++u) {
            const int i = at_span * SAMP_SPAN + u * 64 + lane;
            float c = i < V ? expf(row[i] / temp - mx) : 0.f;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const float v = __shfl_up(c, o, 64);
                if (lane >= o) c += v;
            }
            const unsigned long long hit = __ballot(i < V && cum + c >= goal);
            if (hit) found = at_span * SAMP_SPAN + u * 64 + (__ffsll((long long)hit) - 1);
            cum += __shfl(c, 63, 64);
        }
        if (lane == 0) out[r] = found >= 0 ? found : bi;
    }
}

// ------------------------------------------------------------------ filters before the draw
// The reference's pipeline on a row of logits, in place (crates/spite-sampling/src/lib.rs:
// 273-296): repetition penalty over a list of distinct ids (l > 0 ? l / pen : l * pen,
// :206-232), division by the temperature (:116-125), min-p (drop l < max + ln(min_p),
// :186-197), top-k (keep l >= the k-th largest, :128-144), top-p (sorted by falling logit,
// equal ones by index, the shortest prefix whose share of sum exp(l - max) reaches p, at least
// one; :147-180).  Dropped logits become -inf.  One workgroup per row; nothing is sorted:
// the k-th largest value and the value at which the mass reaches p are found digit by digit
// (four bits a pass) over an order-preserving integer image of the floats, with counts, or
// masses in 64-bit floating point, per digit.  Every thread owns the same elements of the row
// in all passes, and all sums run in a fixed order.
// `params` is [6][n_rows] doubles: on (0 = leave the row alone), temperature, ln(min_p)
// (-inf = off), top_k (0 = off), top_p (>= 1 = off), penalty.
#define FILT_NT 1024
#define TP_BINS 128        // top-p: bins of the first look, a quarter wide, the last one open
#define TP_LIST 8192       // top-p: the most candidates that are sorted in LDS

__device__ __forceinline__ uint32_t float_key(float x) {
    const uint32_t b = __float_as_uint(x);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key_float(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// f(i, row[i]) for the thread's elements tid, tid + NT, ..., the same ones in every pass over a
// row; sixteen loads are in flight at a time.  (16-byte loads of four neighbours were measured
// slower: the passes are bound by their arithmetic and LDS traffic on the one CU, not by loads.)
template <typename F>
__device__ __forceinline__ void each_of_mine(const float* row, int V, F f) {
    constexpr int U = 16;
    for (int base = threadIdx.x; base < V; base += U * FILT_NT) {
        float x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = base + u * FILT_NT;
            x[u] = i < V ? row[i] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = base + u * FILT_NT;
            if (i < V) f(i, x[u]);
        }
    }
}

// Sums of 16 per-thread values over the workgroup, the same in every thread afterwards.
template <typename A>
__device__ void block_sum16(A (&v)[16], A* sh /* [FILT_NT/64][16] */) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        A x = v[j];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
        if (lane == 0) sh[w * 16 + j] = x;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        A t = 0;
        for (int k = 0; k < FILT_NT / 64; ++k) t += sh[k * 16 + j];
        v[j] = t;
    }
    __syncthreads();
}
template <typename A>
__device__ A block_sum1(A x, A* sh) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
    if (lane == 0) sh[w] = x;
    __syncthreads();
    A t = 0;
    for (int k = 0; k < FILT_NT / 64; ++k) t += sh[k];
    __syncthreads();
    return t;
}

// Bitonic sort of list[0, n) (n a power of two) in LDS by the whole workgroup, largest first.
__device__ void sort_falling(unsigned long long* list, int n) {
    for (int k = 2; k <= n; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int t = threadIdx.x; t < n; t += FILT_NT) {
                const int o = t ^ j;
                if (o > t) {
                    const unsigned long long a = list[t], b = list[o];
                    const bool falling = (t & k) == 0;
                    if (falling ? a < b : a > b) { list[t] = b; list[o] = a; }
                }
            }
            __syncthreads();
        }
}

// ---- where a row's elements lie below its maximum: bins of a quarter (the last one open), and,
// inside a run of those bins that holds too many elements to sort, 127 finer bins.
struct Bins {
    int lo0, hi0;          // the quarter bins of the candidates
    bool fine;             // whether the finer bins cut the candidates down further
    int lo1, hi1;          // then: the finer bins of the candidates
    float s1;              // finer bins per quarter bin of the run
};
__device__ __forceinline__ int bin_coarse(float mx, float x) { return (int)fminf((mx - x) * 4.0f, (float)(TP_BINS - 1)); }
__device__ __forceinline__ int bin_fine(float mx, float x, int lo0, float s1) {
    return (int)fminf(fmaxf(((mx - x) * 4.0f - (float)lo0) * s1, 0.f), (float)(TP_BINS - 2));
}
// 0: above the candidates (it stays for certain), 1: a candidate, 2: below them
__device__ __forceinline__ int bin_class(const Bins& b, float mx, float x) {
    const int c = bin_coarse(mx, x);
    if (c < b.lo0) return 0;
    if (c > b.hi0) return 2;
    if (!b.fine) return 1;
    const int f = bin_fine(mx, x, b.lo0, b.s1);
    return f < b.lo1 ? 0 : (f > b.hi1 ? 2 : 1);
}

// The largest key t such that weight(keys >= t) reaches the goal, where an element weighs 1
// (MASS = false: goal = k, the k-th largest key) or exp(l - mx) (MASS = true: goal = p as a
// share of `total`).  `above` returns the weight of the keys greater than the result.
template <bool MASS>
__device__ uint32_t select_key(const float* row, int V, float mx, double total, double goal, double& above_out, double* sh,
                               double* buckets /* [16][FILT_NT] */) {
    typedef typename std::conditional<MASS, double, int>::type A;
    uint32_t prefix = 0;
    A above = 0;
    for (int shift = 28; shift >= 0; shift -= 4) {
        // the thread's sixteen sums lie in LDS, [digit][thread]: indexing registers by the digit
        // would cost sixteen selects an element
        A* mine = (A*)buckets + threadIdx.x;
#pragma unroll
        for (int j = 0; j < 16; ++j) mine[j * FILT_NT] = 0;
        each_of_mine(row, V, [&](int, float x) {
            const uint32_t key = float_key(x);
            if (shift == 28 || ((key ^ prefix) >> (shift + 4)) == 0) {
                const int d = (key >> shift) & 15;
                mine[d * FILT_NT] += MASS ? (A)expf(x - mx) : (A)1;
            }
        });
        A w[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) w[j] = mine[j * FILT_NT];
        block_sum16<A>(w, (A*)sh);
        int d = 15;
        A run = above;
        for (; d > 0; --d) {
            const A with = run + w[d];
            if (MASS ? ((double)with / total >= goal) : ((double)with >= goal)) break;
            run = with;
        }
        prefix |= (uint32_t)d << shift;
        above = run;
    }
    above_out = (double)above;
    return prefix;
}

__global__ __launch_bounds__(FILT_NT)
void filter_rows_kernel(float* __restrict__ work, int ld, int V, int n_rows, const double* __restrict__ params,
                        const int* __restrict__ pen_ids, const int* __restrict__ pen_offsets) {
    __shared__ double sh[FILT_NT / 64 * 16];
    __shared__ int cut;
    extern __shared__ __attribute__((aligned(16))) double buckets[];      // [16][FILT_NT]
    const int r = blockIdx.x, tid = threadIdx.x;
    if (params[r] == 0.0) return;
    float* row = work + (size_t)r * ld;
    const float temp = (float)params[n_rows + r], ln_min_p = (float)params[2 * n_rows + r];
    const int top_k = (int)params[3 * n_rows + r];
    const double top_p = params[4 * n_rows + r];
    const float pen = (float)params[5 * n_rows + r];

    for (int j = pen_offsets[r] + tid; j < pen_offsets[r + 1]; j += FILT_NT) {       // distinct ids
        const int id = pen_ids[j];
        const float v = row[id];
        row[id] = v > 0.f ? v / pen : v * pen;
    }
    __syncthreads();
    // temperature and the maximum
    float mx = -INFINITY;
    each_of_mine(row, V, [&](int i, float x) {
        if (temp > 0.f) { x = x / temp; row[i] = x; }
        mx = fmaxf(mx, x);
    });
    mx = wave_max(mx);
    {
        float* shf = (float*)sh;
        if ((tid & 63) == 0) shf[tid >> 6] = mx;
        __syncthreads();
        for (int k = 0; k < FILT_NT / 64; ++k) mx = fmaxf(mx, shf[k]);
        __syncthreads();
    }
    if (ln_min_p > -INFINITY) {
        const float thresh = mx + ln_min_p;
        each_of_mine(row, V, [&](int i, float x) { if (x < thresh) row[i] = -INFINITY; });
    }
    if (top_k > 0 && top_k < V) {
        // counts by distance from the maximum name the bin of the k-th largest element (if that
        // bin is crowded, finer bins inside it do); its elements are sorted in LDS
        int* hist_n = (int*)buckets;                                       // [TP_BINS]
        unsigned long long* list = (unsigned long long*)buckets + TP_BINS; // [TP_LIST]
        for (int j = tid; j < TP_BINS; j += FILT_NT) hist_n[j] = 0;
        if (tid == 0) cut = 0;
        __syncthreads();
        each_of_mine(row, V, [&](int, float x) {
            const int bin = bin_coarse(mx, x);
            if (bin < TP_BINS - 1 || x > -INFINITY) atomicAdd(&hist_n[bin], 1);     // the open bin counts what is finite
        });
        __syncthreads();
        Bins b = {-1, -1, false, 0, 0, 0.f};
        int before = 0;
        for (int j = 0; j < TP_BINS - 1; ++j) {
            if (before + hist_n[j] >= top_k) { b.lo0 = b.hi0 = j; break; }
            before += hist_n[j];
        }
        const bool all_stay = b.lo0 < 0 && before + hist_n[TP_BINS - 1] < top_k;   // fewer than k finite values
        int n_cand = b.lo0 >= 0 ? hist_n[b.lo0] : 0;
        __syncthreads();
        if (b.lo0 >= 0 && n_cand > TP_LIST) {
            b.s1 = (float)(TP_BINS - 1);
            for (int j = tid; j < TP_BINS; j += FILT_NT) hist_n[j] = 0;
            __syncthreads();
            each_of_mine(row, V, [&](int, float x) {
                if (bin_coarse(mx, x) == b.lo0) atomicAdd(&hist_n[bin_fine(mx, x, b.lo0, b.s1)], 1);
            });
            __syncthreads();
            for (int j = 0; j < TP_BINS - 1; ++j) {
                if (before + hist_n[j] >= top_k) { b.fine = true; b.lo1 = b.hi1 = j; n_cand = hist_n[j]; break; }
                before += hist_n[j];
            }
            __syncthreads();
        }
        float thresh;
        if (all_stay) {
            thresh = -INFINITY;
        } else if (b.lo0 >= 0 && n_cand <= TP_LIST) {
            int n_pad = 64;
            while (n_pad < n_cand) n_pad <<= 1;
            for (int j = tid; j < n_pad; j += FILT_NT) list[j] = 0;
            __syncthreads();
            each_of_mine(row, V, [&](int, float x) {
                if (bin_class(b, mx, x) == 1) list[atomicAdd(&cut, 1)] = float_key(x);
            });
            __syncthreads();
            sort_falling(list, n_pad);
            thresh = key_float((uint32_t)list[top_k - before - 1]);
            __syncthreads();
        } else {
            double above;
            thresh = key_float(select_key<false>(row, V, mx, 1.0, (double)top_k, above, sh, buckets));
        }
        each_of_mine(row, V, [&](int i, float x) { if (x < thresh) row[i] = -INFINITY; });
    }
    if (top_p < 1.0) {
        // An element is (key, index) in one 64-bit number that falls as the reference's stable
        // sort runs: `bound` is the last element kept, and every element not below it stays.
        auto composite = [](float x, int i) { return ((unsigned long long)float_key(x) << 32) | (0xffffffffu - (uint32_t)i); };
        unsigned long long bound;

        // The total mass, and a first look at where it lies: masses (fixed point, so that their
        // sums do not depend on the order of the atomic adds) and counts by distance from the
        // maximum, in bins of a quarter.  They tell in which bins the boundary can lie: the
        // elements above those bins stay for certain, the ones below go, and the elements of
        // the bins themselves are sorted in LDS; if they are too many for that, finer bins
        // inside those bins cut them down first.
        unsigned long long* hist_m = (unsigned long long*)buckets;        // [TP_BINS]
        int* hist_n = (int*)(hist_m + TP_BINS);                            // [TP_BINS]
        unsigned long long* list = hist_m + 2 * TP_BINS;                   // [TP_LIST]
        const double FIX = 1099511627776.0;                                // 2^40
        for (int j = tid; j < TP_BINS; j += FILT_NT) { hist_m[j] = 0; hist_n[j] = 0; }
        if (tid == 0) cut = 0;
        __syncthreads();
        double part = 0.0;
        each_of_mine(row, V, [&](int, float x) {
            const float e = expf(x - mx);
            part += (double)e;
            const int bin = bin_coarse(mx, x);
            if (bin < TP_BINS - 1) {
                atomicAdd(&hist_m[bin], (unsigned long long)((double)e * FIX));
                atomicAdd(&hist_n[bin], 1);
            }
        });
        const double total = block_sum1<double>(part, sh);
        // (block_sum1's barriers also order the atomics before the reads below)
        // a bin's fixed-point mass is below the true one by less than its count: the first bin
        // where the share may be reached, and the first where it is reached for certain
        const double goal = top_p * total * FIX;
        Bins b = {-1, -1, false, -1, -1, 0.f};
        int n_cand = 0;
        double have = 0.0, have_above = 0.0;           // fixed-point mass up to here / above the candidates
        for (int j = 0; j < TP_BINS - 1; ++j) {
            if (b.lo0 < 0 && have + (double)hist_m[j] + (double)V >= goal * (1.0 - 1e-9)) { b.lo0 = j; have_above = have; }
            have += (double)hist_m[j];
            if (b.lo0 >= 0) n_cand += hist_n[j];
            if (have >= goal * (1.0 + 1e-9)) { b.hi0 = j; break; }
        }
        __syncthreads();
        if (b.hi0 >= 0 && n_cand > TP_LIST) {
            b.s1 = (float)(TP_BINS - 1) / (float)(b.hi0 - b.lo0 + 1);
            for (int j = tid; j < TP_BINS; j += FILT_NT) { hist_m[j] = 0; hist_n[j] = 0; }
            __syncthreads();
            each_of_mine(row, V, [&](int, float x) {
                const int c = bin_coarse(mx, x);
                if (c >= b.lo0 && c <= b.hi0) {
                    const int f = bin_fine(mx, x, b.lo0, b.s1);
                    atomicAdd(&hist_m[f], (unsigned long long)((double)expf(x - mx) * FIX));
                    atomicAdd(&hist_n[f], 1);
                }
            });
            __syncthreads();
            have = have_above;
            n_cand = 0;
            for (int j = 0; j < TP_BINS - 1; ++j) {
                if (b.lo1 < 0 && have + (double)hist_m[j] + (double)V >= goal * (1.0 - 1e-9)) b.lo1 = j;
                have += (double)hist_m[j];
                if (b.lo1 >= 0) n_cand += hist_n[j];
                if (have >= goal * (1.0 + 1e-9)) { b.hi1 = j; break; }
            }
            b.fine = b.hi1 >= 0;
            if (!b.fine) n_cand = TP_LIST + 1;         // (cannot happen: the run held the boundary) -> the search below
            __syncthreads();
        }
        if (b.hi0 >= 0 && n_cand > 0 && n_cand <= TP_LIST) {
            int n_pad = 64;
            while (n_pad < n_cand) n_pad <<= 1;
            for (int j = tid; j < n_pad; j += FILT_NT) list[j] = 0;       // below every element
            __syncthreads();
            double sure = 0.0;                                            // mass of what lies above the candidates
            each_of_mine(row, V, [&](int i, float x) {
                const int c = bin_class(b, mx, x);
                if (c == 0) sure += (double)expf(x - mx);
                else if (c == 1) list[atomicAdd(&cut, 1)] = composite(x, i);
            });
            sure = block_sum1<double>(sure, sh);
            sort_falling(list, n_pad);
            // the shortest prefix whose share reaches p: every thread sums a run of the sorted
            // list, the runs' sums are added up in order, and the thread in whose run the share
            // is reached names the place
            const int per = n_pad / FILT_NT > 0 ? n_pad / FILT_NT : 1;
            const int b0 = tid * per;
            double mine = 0.0;
            for (int j = b0; j < b0 + per && j < n_cand; ++j) mine += (double)expf(key_float((uint32_t)(list[j] >> 32)) - mx);
            double* runs = sh;                        // FILT_NT doubles do not fit sh: in rounds of 256
            __shared__ double carry;
            __shared__ int place;
            if (tid == 0) { carry = sure; place = n_cand - 1; }
            __syncthreads();
            for (int round = 0; round < FILT_NT / 256; ++round) {
                const bool in = (tid >> 8) == round;
                if (in) runs[tid & 255] = mine;
                __syncthreads();
                if (in) {
                    double cum = carry;
                    for (int k = 0; k < (tid & 255); ++k) cum += runs[k];
                    for (int j = b0; j < b0 + per && j < n_cand; ++j) {
                        cum += (double)expf(key_float((uint32_t)(list[j] >> 32)) - mx);
                        if (cum / total >= top_p) { atomicMin(&place, j); break; }
                    }
                }
                __syncthreads();
                if (tid == 0) { double c = carry; for (int k = 0; k < 256; ++k) c += runs[k]; carry = c; }
                __syncthreads();
            }
            bound = list[place];
        } else {
            __syncthreads();
            double above;
            const uint32_t tau = select_key<true>(row, V, mx, total, top_p, above, sh, buckets);
            // of the elements equal to the boundary value the first `keep` in index order stay
            int n_eq = 0;
            each_of_mine(row, V, [&](int, float x) { n_eq += float_key(x) == tau; });
            n_eq = block_sum1<int>(n_eq, (int*)sh);
            const double e_tau = (double)expf(key_float(tau) - mx);
            int keep = n_eq;
            if (e_tau > 0.0 && n_eq > 1) {
                keep = 1;
                while (keep < n_eq && (above + keep * e_tau) / total < top_p) ++keep;
            }
            if (tid == 0) cut = V;
            __syncthreads();
            if (keep < n_eq) {
                // the index of the keep-th element equal to the boundary: a count in index order
                int* cnt = (int*)sh;                       // per wave
                int before = 0;
                for (int base = 0; base < V && before < keep; base += FILT_NT) {
                    const int i = base + tid;
                    const bool eq = i < V && float_key(row[i]) == tau;
                    const unsigned long long m = __ballot(eq);
                    const int lane = tid & 63, w = tid >> 6;
                    if (lane == 0) cnt[w] = __popcll(m);
                    __syncthreads();
                    int mine = before;
                    for (int k = 0; k < w; ++k) mine += cnt[k];
                    int all = before;
                    for (int k = 0; k < FILT_NT / 64; ++k) all += cnt[k];
                    mine += __popcll(m & ((1ull << lane) - 1));
                    if (eq && mine + 1 == keep) cut = i;
                    before = all;
                    __syncthreads();
                }
            }
            bound = ((unsigned long long)tau << 32) | (0xffffffffu - (uint32_t)cut);
        }
        each_of_mine(row, V, [&](int i, float x) { if (composite(x, i) < bound) row[i] = -INFINITY; });
    }
}

// `work` [n_rows, ld] fp32 is changed in place; `params` as described above; `pen_ids` are the
// distinct ids to penalise, row r's at pen_offsets[r] .. pen_offsets[r+1], each inside [0, V).
extern "C" int spite_filter_rows(float* work, int ld, int n_rows, int V, const double* params, const int* pen_ids,
                                 const int* pen_offsets, hipStream_t st) {
    SP_REQUIRE(n_rows >= 0 && V > 0 && ld >= V, "filter: bad sizes rows=%d V=%d ld=%d", n_rows, V, ld);
    SP_REQUIRE(params && pen_offsets, "filter: parameters missing");
    if (n_rows == 0) return 0;
    const size_t lds = (size_t)16 * FILT_NT * sizeof(double);
    static bool allowed = false;          // more LDS than the default limit
    if (!allowed) {
        hipError_t e = hipFuncSetAttribute((const void*)filter_rows_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        SP_REQUIRE(e == hipSuccess, "filter: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
        allowed = true;
    }
    filter_rows_kernel<<<n_rows, FILT_NT, lds, st>>>(work, ld, V, n_rows, params, pen_ids, pen_offsets);
    SP_LAUNCH_CHECK("filter_rows");
    return 0;
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
    const size_t lds = (size_t)((V + SAMP_SPAN - 1) / SAMP_SPAN) * sizeof(float);
    SP_REQUIRE(lds <= 40 * 1024, "sample: a vocabulary of %d is beyond this kernel (at most %d)", V, 10 * 1024 * SAMP_SPAN);
    sample_rows_kernel<<<n_rows, SAMP_NT, lds, st>>>(logits, ld, V, temperature, uniform, out);
    SP_LAUNCH_CHECK("sample_rows");
    return 0;
}
