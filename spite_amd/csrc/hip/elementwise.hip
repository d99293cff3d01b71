// Row-wise kernels of the step: embedding gather, residual add + RMSNorm, rotation /
// qk-norm / temperature + cache write, top-1 router and the expert plan.
// One workgroup per row (or per token and head); all reductions in fp32 in an order that
// depends on the row's width only, never on what else is in the batch.
#include "common.h"

static thread_local char g_err[512];
int sp_fail(const char* fmt, ...) {
    va_list ap; va_start(ap, fmt); vsnprintf(g_err, sizeof g_err, fmt, ap); va_end(ap);
    return -1;
}
extern "C" const char* spite_hip_last_error() { return g_err; }
extern "C" int spite_hip_abi_version() { return 1; }

int sp_cu_count() {
    static int count[64];                       // per device; 0 = not asked yet
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int c = __atomic_load_n(&count[dev], __ATOMIC_RELAXED);
    if (c <= 0) {
        if (hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || c <= 0) c = 256;
        __atomic_store_n(&count[dev], c, __ATOMIC_RELAXED);
    }
    return c;
}
extern "C" int spite_cu_count() { return sp_cu_count(); }

// ------------------------------------------------------------------ embedding
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                             float* __restrict__ h, int d, int vocab) {
    const int t = blockIdx.x;
    const int id = ids[t];
    const bool ok = id >= 0 && id < vocab;
    const T* row = table + (size_t)(ok ? id : 0) * d;
    for (int c = threadIdx.x; c < d; c += blockDim.x)
        h[(size_t)t * d + c] = ok ? to_f32<T>(row[c]) : 0.f;
}

extern "C" int spite_embed(const int* ids, const void* table, int dtype, float* h, int T, int d,
                           int vocab, hipStream_t st) {
    SP_REQUIRE(T >= 0 && d > 0 && vocab > 0, "embed: bad sizes T=%d d=%d vocab=%d", T, d, vocab);
    if (T == 0) return 0;
    if (dtype == SP_F32) embed_kernel<float><<<T, 256, 0, st>>>(ids, (const float*)table, h, d, vocab);
    else if (dtype == SP_BF16) embed_kernel<bf16><<<T, 256, 0, st>>>(ids, (const bf16*)table, h, d, vocab);
    else return sp_fail("embed: unknown dtype %d", dtype);
    SP_LAUNCH_CHECK("embed");
    return 0;
}

// ------------------------------------------------------------------ a wave's fp32 dot product
// sum_c w[c] * xs[c] over a row xs in LDS, by one wave: lane l takes the 16-byte groups l, l+64,
// ... and the lanes' sums meet in a butterfly.  Every kernel that forms router logits calls
// this, so a logit has the same bits wherever it is computed; its order of summation depends
// on the width alone.
__device__ __forceinline__ float wave_dot_row(const float* __restrict__ w, const float* xs, int d, bool vec, int lane) {
    float acc = 0.f;
    if (vec) {
        const int nv = d >> 2;
#pragma unroll 10
        for (int c = lane; c < nv; c += 64) {          // independent 16-byte loads, ten in flight
            const f32x4 ww = ((const f32x4*)w)[c];
            const f32x4 xx = ((const f32x4*)xs)[c];
            acc += ww[0] * xx[0] + ww[1] * xx[1] + ww[2] * xx[2] + ww[3] * xx[3];
        }
    } else {
        for (int c = lane; c < d; c += 64) acc += w[c] * xs[c];
    }
    return wave_sum(acc);
}

// ------------------------------------------------------------------ residual add + RMSNorm
// v = h[r] + d1[r] + d2[r]; (h[r] = v); out[i] = v * 1/sqrt(mean(v^2)+eps) * w, r = rows ? rows[i] : i.
// One workgroup of NT threads per row; a thread keeps its elements (groups of four, strided
// by NT) in registers between the sum and the scaling, so the row is read once.  The sum's
// order depends on the width alone.
// With `proj` ([P, d] fp32) the normed fp32 row also goes to LDS and the waves form its P
// products proj . y into proj_out[i][0..P): the router's logits, without the row going to
// memory in 32-bit and back.
#define NORM_NT 512
#define NORM_MAX_V 8     // widths up to 4*NT*MAX_V = 16384 stay in registers
template <typename TO, bool VEC>
__global__ __launch_bounds__(NORM_NT)
void add_rmsnorm_kernel(float* __restrict__ h, const float* __restrict__ d1,
                        const float* __restrict__ d2, const float* __restrict__ w,
                        TO* __restrict__ out, float* __restrict__ out32,
                        const int* __restrict__ rows, int d, float eps, int write_h,
                        const float* __restrict__ proj, float* __restrict__ proj_out, int P) {
    __shared__ float red[NORM_NT / 64];
    extern __shared__ __attribute__((aligned(16))) float ys[];            // [d] if proj
    const int i = blockIdx.x;
    const size_t r = rows ? (size_t)rows[i] : (size_t)i;
    float* hr = h + r * d;
    const float* a = d1 ? d1 + r * d : nullptr;
    const float* b = d2 ? d2 + r * d : nullptr;
    float ss = 0.f;
    if (VEC) {
        // d is a multiple of 4 and at most 4*NT*MAX_V
        f32x4 v[NORM_MAX_V];
        const int nv = d >> 2;
#pragma unroll
        for (int u = 0; u < NORM_MAX_V; ++u) {
            const int c = threadIdx.x + u * NORM_NT;
            if (c < nv) {
                f32x4 x = ((const f32x4*)hr)[c];
                if (a) x += ((const f32x4*)a)[c];
                if (b) x += ((const f32x4*)b)[c];
                if (write_h) ((f32x4*)hr)[c] = x;
                v[u] = x;
                ss += x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3];
            }
        }
        const float ms = block_sum<NORM_NT>(ss, red) / (float)d;
        const float scale = 1.0f / sqrtf(ms + eps);
#pragma unroll
        for (int u = 0; u < NORM_MAX_V; ++u) {
            const int c = threadIdx.x + u * NORM_NT;
            if (c < nv) {
                const f32x4 ww = ((const f32x4*)w)[c];
                f32x4 y;
#pragma unroll
                for (int e = 0; e < 4; ++e) y[e] = v[u][e] * scale * ww[e];
                if (out32) ((f32x4*)(out32 + (size_t)i * d))[c] = y;
                if (proj) ((f32x4*)ys)[c] = y;
                if (out) {
                    if constexpr (sizeof(TO) == 2) {             // four bf16 in one 8-byte store (d % 4 == 0 here)
                        bf16x4 o4;
#pragma unroll
                        for (int e = 0; e < 4; ++e) o4[e] = (bf16)y[e];
                        *(bf16x4*)((bf16*)out + (size_t)i * d + 4 * c) = o4;
                    } else {
                        ((f32x4*)((float*)out + (size_t)i * d))[c] = y;
                    }
                }
            }
        }
    } else {
        for (int c = threadIdx.x; c < d; c += NORM_NT) {
            float x = hr[c];
            if (a) x += a[c];
            if (b) x += b[c];
            if (write_h) hr[c] = x;
            ss += x * x;
        }
        const float ms = block_sum<NORM_NT>(ss, red) / (float)d;
        const float scale = 1.0f / sqrtf(ms + eps);
        for (int c = threadIdx.x; c < d; c += NORM_NT) {
            float x = hr[c];
            if (!write_h) { if (a) x += a[c]; if (b) x += b[c]; }
            const float y = x * scale * w[c];
            if (out) out[(size_t)i * d + c] = from_f32<TO>(y);
            if (out32) out32[(size_t)i * d + c] = y;
            if (proj) ys[c] = y;
        }
    }
    if (proj) {
        __syncthreads();
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const bool pvec = (d & 3) == 0 && (((uintptr_t)proj) & 15) == 0;
        for (int p = wave; p < P; p += NORM_NT / 64) {
            const float v = wave_dot_row(proj + (size_t)p * d, ys, d, pvec, lane);
            if (lane == 0) proj_out[(size_t)i * P + p] = v;
        }
    }
}

extern "C" int spite_add_rmsnorm(float* h, const float* d1, const float* d2, const float* w, void* out,
                                 int out_dtype, float* out32, const int* rows, int n_rows, int d,
                                 float eps, int write_h, const float* proj, float* proj_out, int P,
                                 hipStream_t st) {
    SP_REQUIRE(n_rows >= 0 && d > 0 && eps > 0.f, "add_rmsnorm: bad sizes rows=%d d=%d eps=%g", n_rows, d, eps);
    SP_REQUIRE(!proj || (proj_out && P > 0), "add_rmsnorm: a projection needs its output and size");
    const size_t sh = proj ? (size_t)d * sizeof(float) : 0;
    SP_REQUIRE(sh <= 48 * 1024, "add_rmsnorm: rows of %d do not fit the projection's LDS", d);
    if (n_rows == 0) return 0;
    auto al = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    const bool vec = d % 4 == 0 && d <= 4 * NORM_NT * NORM_MAX_V && al(h) && al(d1) && al(d2) && al(w) && al(out32) && al(out);
#define SP_NORM(TO) do { if (vec) add_rmsnorm_kernel<TO, true><<<n_rows, NORM_NT, sh, st>>>(h, d1, d2, w, (TO*)out, out32, rows, d, eps, write_h, proj, proj_out, P); \
        else add_rmsnorm_kernel<TO, false><<<n_rows, NORM_NT, sh, st>>>(h, d1, d2, w, (TO*)out, out32, rows, d, eps, write_h, proj, proj_out, P); } while (0)
    if (out_dtype == SP_F32) SP_NORM(float);
    else if (out_dtype == SP_BF16) SP_NORM(bf16);
    else return sp_fail("add_rmsnorm: unknown dtype %d", out_dtype);
#undef SP_NORM
    SP_LAUNCH_CHECK("add_rmsnorm");
    return 0;
}

// ------------------------------------------------------------------ rotation, qk-norm, temperature, cache write
// One wave per (token, head).  Heads [0,H) are queries, [H,H+G) keys, [H+G,H+2G) values of
// the fused projection row.  Queries and keys: rotate by pos*inv_freq (if use_rope), then
// the RMS norm over the head (if use_norm; weightless, or times w_q / w_k if given); queries alone
// are then multiplied by ln(floor((pos+1)/floor_scale)+1)*attn_scale+1 (if use_temp).  Keys and
// values go to the request's page: cache row = slot_map[t] = page*page_size + offset.  Key pages
// are laid out [page][kv head][offset][hd]; value pages transposed, [page][kv head][hd][offset],
// so that the attention kernels read eight consecutive keys of one value column in one load (the
// layout of an MFMA operand whose sum runs over keys).
// Options that other architectures' attention needs: `rot` < hd rotates the first `rot`
// elements of a head only (pairs (i, i + rot/2), or adjacent ones) and passes the rest through;
// `norm_first` norms (and weights) before the rotation instead of after it.
#define SP_MAX_PAIRS 4   // head sizes up to 512
// Four waves a workgroup; a wave takes `hpw` heads of one token in turn and computes the
// token's sines and cosines once for all of them.
template <typename T>
__global__ __launch_bounds__(256)
void rope_kvwrite_kernel(const T* __restrict__ qkv, T* __restrict__ q_out,
                         T* __restrict__ k_pages, T* __restrict__ v_pages,
                         const int* __restrict__ positions, const int* __restrict__ slot_map,
                         const float* __restrict__ inv_freq, int H, int G, int hd, int ps,
                         int use_rope, int adjacent, int use_norm, float norm_eps,
                         int use_temp, int floor_scale, float attn_scale, int n_heads, int hpw, int kv_tiled,
                         int rot, const float* __restrict__ w_q, const float* __restrict__ w_k, int norm_first) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int half = hd >> 1, rhalf = rot >> 1;
    const int row_w = (H + 2 * G) * hd;
    const int pos = positions[t];
    const int slot = slot_map ? slot_map[t] : -1;
    // pair i of a head: the rotating pairs first (i < rot/2), then the elements behind `rot` two by two
    auto first_of = [&](int i) { return adjacent ? 2 * i : (i < rhalf ? i : rot + (i - rhalf)); };
    auto second_of = [&](int i) { return adjacent ? 2 * i + 1 : (i < rhalf ? i + rhalf : rot + (i - rhalf) + (half - rhalf)); };
    float sn[SP_MAX_PAIRS], cs[SP_MAX_PAIRS];
#pragma unroll
    for (int u = 0; u < SP_MAX_PAIRS; ++u) {
        const int i = lane + u * 64;
        sn[u] = 0.f; cs[u] = 1.f;                    // pairs that do not rotate
        if (use_rope && i < rhalf) sincosf((float)pos * inv_freq[i], &sn[u], &cs[u]);
    }
    float temp = 1.f;
    if (use_temp) temp = logf((float)((pos + 1) / floor_scale) + 1.0f) * attn_scale + 1.0f;

    for (int it = 0; it < hpw; ++it) {
        const int hh = blockIdx.y * 4 * hpw + it * 4 + wave;
        if (hh >= n_heads) break;
        const T* src = qkv + (size_t)t * row_w + (size_t)hh * hd;
        const bool is_q = hh < H;
        const bool is_v = hh >= H + G;
        T* dst;
        int off = 0;
        const bool tiled_k = !is_q && kv_tiled;      // the key's elements go to their places in the operand tiles
        if (is_q) {
            dst = q_out + ((size_t)t * H + hh) * hd;
        } else {
            if (slot < 0) continue;
            const int g = is_v ? hh - H - G : hh - H;
            const size_t page = slot / ps;
            off = slot % ps;
            if (is_v) {
                T* slab = v_pages + (page * G + g) * hd * ps;
                for (int c = lane; c < hd; c += 64) slab[sp_v_index(c, off, hd, ps, kv_tiled)] = src[c];
                continue;
            }
            dst = k_pages + (page * G + g) * (size_t)ps * hd;
            if (!kv_tiled) dst += (size_t)off * hd;
        }
        const float* wn = is_q ? w_q : w_k;
        float x0[SP_MAX_PAIRS], x1[SP_MAX_PAIRS];
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < SP_MAX_PAIRS; ++u) {
            const int i = lane + u * 64;
            if (i < half) {
                float a = to_f32<T>(src[first_of(i)]), b = to_f32<T>(src[second_of(i)]);
                if (use_rope && !norm_first) {
                    const float ra = a * cs[u] - b * sn[u];
                    const float rb = a * sn[u] + b * cs[u];
                    a = ra; b = rb;
                }
                x0[u] = a; x1[u] = b;
                ss += a * a + b * b;
            }
        }
        float scale = 1.f;
        if (use_norm) {
            ss = wave_sum(ss);
            scale = 1.0f / sqrtf(ss / (float)hd + norm_eps);
        }
        const float last = is_q ? temp : 1.f;
#pragma unroll
        for (int u = 0; u < SP_MAX_PAIRS; ++u) {
            const int i = lane + u * 64;
            if (i < half) {
                const int i0 = first_of(i), i1 = second_of(i);
                float a = x0[u] * scale, b = x1[u] * scale;
                if (use_norm && wn) { a *= wn[i0]; b *= wn[i1]; }
                if (use_rope && norm_first) {
                    const float ra = a * cs[u] - b * sn[u];
                    const float rb = a * sn[u] + b * cs[u];
                    a = ra; b = rb;
                }
                if (!use_norm || wn || norm_first) { a *= last; b *= last; }
                else { a = x0[u] * (scale * last); b = x1[u] * (scale * last); }   // the plain case's one product
                dst[tiled_k ? sp_k_index(off, i0, hd, true) : (size_t)i0] = from_f32<T>(a);
                dst[tiled_k ? sp_k_index(off, i1, hd, true) : (size_t)i1] = from_f32<T>(b);
            }
        }
    }
}

// The same for bfloat16 rows whose head size gives every head a power-of-two group of lanes with
// four pairs each (hd = 32, 64, 128, 256, 512): a lane reads and writes eight bytes at a time
// instead of two, and a wave handles 64 / (hd/8) heads at once.  Every value is computed by the
// same operations in the same order as in the kernel above; only the sum of squares of the
// qk-norm meets in a different order.
__global__ __launch_bounds__(256)
void rope_kvwrite_vec_kernel(const bf16* __restrict__ qkv, bf16* __restrict__ q_out,
                             bf16* __restrict__ k_pages, bf16* __restrict__ v_pages,
                             const int* __restrict__ positions, const int* __restrict__ slot_map,
                             const float* __restrict__ inv_freq, int H, int G, int hd, int ps,
                             int use_rope, int adjacent, int use_norm, float norm_eps,
                             int use_temp, int floor_scale, float attn_scale, int n_heads, int hpw, int kv_tiled) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int half = hd >> 1;
    const int lph = half >> 2;                   // lanes a head: four pairs each
    const int sub = lane / lph, l = lane % lph;  // which head of the wave's group, which four pairs
    const int hpi = 64 / lph;                    // heads a wave takes at once
    const int row_w = (H + 2 * G) * hd;
    const int pos = positions[t];
    const int slot = slot_map ? slot_map[t] : -1;
    float sn[4], cs[4];
    if (use_rope) {
#pragma unroll
        for (int u = 0; u < 4; ++u) sincosf((float)pos * inv_freq[4 * l + u], &sn[u], &cs[u]);
    }
    float temp = 1.f;
    if (use_temp) temp = logf((float)((pos + 1) / floor_scale) + 1.0f) * attn_scale + 1.0f;

    for (int it = 0; it < hpw; ++it) {
        const int hh = (blockIdx.y * 4 * hpw + it * 4 + wave) * hpi + sub;
        const bool have = hh < n_heads;          // lanes past the last head idle, but join the shuffles
        const bf16* src = qkv + (size_t)t * row_w + (size_t)(have ? hh : 0) * hd;
        const bool is_q = hh < H;
        const bool is_v = hh >= H + G;
        const int g = is_v ? hh - H - G : hh - H;
        const size_t page = slot >= 0 ? slot / ps : 0;
        const int off = slot >= 0 ? slot % ps : 0;
        // the four pairs' elements: half-split (4l+u, half+4l+u) or adjacent (8l+2u, 8l+2u+1)
        bf16x4 lo4 = *(const bf16x4*)(src + (adjacent ? 8 * l : 4 * l));
        bf16x4 hi4 = *(const bf16x4*)(src + (adjacent ? 8 * l + 4 : half + 4 * l));
        if (have && is_v) {
            if (slot >= 0) {
                bf16* slab = v_pages + (page * G + g) * (size_t)hd * ps;
                const int c0 = adjacent ? 8 * l : 4 * l, c1 = adjacent ? 8 * l + 4 : half + 4 * l;
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    slab[sp_v_index(c0 + u, off, hd, ps, kv_tiled)] = lo4[u];
                    slab[sp_v_index(c1 + u, off, hd, ps, kv_tiled)] = hi4[u];
                }
            }
        }
        float x0[4], x1[4];
        float ss = 0.f;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            float a, b;
            if (adjacent) {              // pairs (8l+2u, 8l+2u+1): two from lo4, two from hi4
                a = (float)(u < 2 ? lo4[2 * u] : hi4[2 * u - 4]);
                b = (float)(u < 2 ? lo4[2 * u + 1] : hi4[2 * u - 3]);
            } else {
                a = (float)lo4[u]; b = (float)hi4[u];
            }
            if (use_rope) {
                const int su = adjacent ? u : u;
                // adjacent pairing: pair index 4l+u as well
                const float ra = a * cs[su] - b * sn[su];
                const float rb = a * sn[su] + b * cs[su];
                a = ra; b = rb;
            }
            x0[u] = a; x1[u] = b;
            ss += a * a + b * b;
        }
        float scale = 1.f;
        if (use_norm) {
            for (int o = 1; o < lph; o <<= 1) ss += __shfl_xor(ss, o, 64);
            scale = 1.0f / sqrtf(ss / (float)hd + norm_eps);
        }
        if (is_q) scale *= temp;
        if (!have || is_v || (!is_q && slot < 0)) continue;
        bf16x4 o_lo, o_hi;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const bf16 ya = (bf16)(x0[u] * scale), yb = (bf16)(x1[u] * scale);
            if (adjacent) {
                if (u < 2) { o_lo[2 * u] = ya; o_lo[2 * u + 1] = yb; } else { o_hi[2 * u - 4] = ya; o_hi[2 * u - 3] = yb; }
            } else {
                o_lo[u] = ya; o_hi[u] = yb;
            }
        }
        const int c0 = adjacent ? 8 * l : 4 * l, c1 = adjacent ? 8 * l + 4 : half + 4 * l;
        if (is_q) {
            bf16* dst = q_out + ((size_t)t * H + hh) * hd;
            *(bf16x4*)(dst + c0) = o_lo;
            *(bf16x4*)(dst + c1) = o_hi;
        } else {
            bf16* slab = k_pages + (page * G + g) * (size_t)ps * hd;
            // four elements in a row stay in a row in operand order too (they share a group of eight)
            *(bf16x4*)(slab + sp_k_index(off, c0, hd, kv_tiled)) = o_lo;
            *(bf16x4*)(slab + sp_k_index(off, c1, hd, kv_tiled)) = o_hi;
        }
    }
}

// `rotary_dim`: how many leading elements of a head rotate (0 or hd: all); `w_q`, `w_k`: weights of the
// qk-norm ([hd] fp32) or null for the weightless norm; `norm_first`: norm before the rotation.
extern "C" int spite_rope_kvwrite(const void* qkv, void* q_out, void* k_pages, void* v_pages, int dtype,
                                  const int* positions, const int* slot_map, const float* inv_freq,
                                  int T, int H, int G, int hd, int page_size, int use_rope, int adjacent,
                                  int use_norm, float norm_eps, int use_temp, int floor_scale,
                                  float attn_scale, int write_kv, int kv_tiled, int rotary_dim, const float* w_q,
                                  const float* w_k, int norm_first, hipStream_t st) {
    SP_REQUIRE(T >= 0 && H > 0 && G > 0 && hd > 0 && page_size > 0, "rope_kvwrite: bad sizes");
    SP_REQUIRE(hd % 2 == 0 && hd <= 128 * SP_MAX_PAIRS, "rope_kvwrite: head size %d must be even and <= %d",
               hd, 128 * SP_MAX_PAIRS);
    SP_REQUIRE(!use_temp || floor_scale > 0, "rope_kvwrite: floor_scale %d must be >= 1", floor_scale);
    SP_REQUIRE(!use_rope || inv_freq, "rope_kvwrite: rotation needs a frequency table");
    SP_REQUIRE(H + 2 * G <= 65535, "rope_kvwrite: too many heads");
    SP_REQUIRE(!write_kv || slot_map, "rope_kvwrite: writing the cache needs the rows' slots");
    SP_REQUIRE(!kv_tiled || (dtype == SP_BF16 && hd % 32 == 0 && page_size % 32 == 0),
               "rope_kvwrite: pages in operand order are bfloat16 with head size %d and page size %d multiples of 32", hd, page_size);
    const int rot = rotary_dim > 0 ? rotary_dim : hd;
    SP_REQUIRE(rot % 2 == 0 && rot <= hd, "rope_kvwrite: %d rotating elements of a head of %d", rot, hd);
    SP_REQUIRE((!w_q && !w_k) || use_norm, "rope_kvwrite: norm weights without a norm");
    if (T == 0) return 0;
    const int n_heads = write_kv ? H + 2 * G : H;
    const int hpw = T >= 256 ? 4 : 1;            // many tokens: fewer, longer workgroups
    const int lph = hd / 8;                      // lanes a head in the 8-byte kernel
    auto al8 = [](const void* p) { return ((uintptr_t)p & 7) == 0; };
    const bool plain = rot == hd && !w_q && !w_k && !norm_first;     // what the 8-byte kernel knows
    if (plain && dtype == SP_BF16 && hd % 8 == 0 && lph >= 1 && lph <= 64 && (lph & (lph - 1)) == 0 && al8(qkv) && al8(q_out)
        && al8(k_pages) && (page_size % 4 == 0 || !write_kv)) {
        const int hpi = 64 / lph;
        dim3 grid(T, (n_heads + 4 * hpw * hpi - 1) / (4 * hpw * hpi));
        rope_kvwrite_vec_kernel<<<grid, 256, 0, st>>>((const bf16*)qkv, (bf16*)q_out, (bf16*)k_pages, (bf16*)v_pages,
            positions, slot_map, inv_freq, H, G, hd, page_size, use_rope, adjacent, use_norm, norm_eps, use_temp,
            floor_scale, attn_scale, n_heads, hpw, kv_tiled);
        SP_LAUNCH_CHECK("rope_kvwrite");
        return 0;
    }
    dim3 grid(T, (n_heads + 4 * hpw - 1) / (4 * hpw));
    if (dtype == SP_F32)
        rope_kvwrite_kernel<float><<<grid, 256, 0, st>>>((const float*)qkv, (float*)q_out, (float*)k_pages,
            (float*)v_pages, positions, slot_map, inv_freq, H, G, hd, page_size, use_rope, adjacent, use_norm,
            norm_eps, use_temp, floor_scale, attn_scale, n_heads, hpw, kv_tiled, rot, w_q, w_k, norm_first);
    else if (dtype == SP_BF16)
        rope_kvwrite_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)qkv, (bf16*)q_out, (bf16*)k_pages,
            (bf16*)v_pages, positions, slot_map, inv_freq, H, G, hd, page_size, use_rope, adjacent, use_norm,
            norm_eps, use_temp, floor_scale, attn_scale, n_heads, hpw, kv_tiled, rot, w_q, w_k, norm_first);
    else return sp_fail("rope_kvwrite: unknown dtype %d", dtype);
    SP_LAUNCH_CHECK("rope_kvwrite");
    return 0;
}

// ------------------------------------------------------------------ top-1 sigmoid router
// logits = W_r . x in fp32, the largest logit wins and the lowest index wins a tie,
// weight = 1/(1+exp(-logit)).  A workgroup takes TB tokens: their rows sit in LDS, the waves
// take the experts in turn, and a wave reads an expert's row once for all TB tokens (with one
// token a workgroup the router's matrix would be fetched from L2 once per token, which is
// what a long prompt's time went into).  A lane's loads are independent 16-byte reads.  A
// logit's sum runs in an order that depends on the width alone, the same for every TB.
#define ROUTER_NT 1024
template <int TB>
__global__ __launch_bounds__(ROUTER_NT)
void router_top1_kernel(const float* __restrict__ x, const float* __restrict__ wr,
                        int* __restrict__ expert, float* __restrict__ weight,
                        float* __restrict__ logits_out, int T, int d, int E) {
    extern __shared__ float xs[];            // [TB][d] then [TB][E] logits
    float* lg = xs + (size_t)TB * d;
    const int t0 = blockIdx.x * TB;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int u = 0; u < TB; ++u) {
        const int t = t0 + u < T ? t0 + u : T - 1;          // rows past the end repeat the last one
        const float* xr = x + (size_t)t * d;
        for (int c = threadIdx.x; c < d; c += ROUTER_NT) xs[(size_t)u * d + c] = xr[c];
    }
    __syncthreads();
    const bool vec = (d & 3) == 0 && (((uintptr_t)wr) & 15) == 0;
    for (int e = wave; e < E; e += ROUTER_NT / 64) {
        const float* w = wr + (size_t)e * d;
        if (TB == 1) {
            const float v = wave_dot_row(w, xs, d, vec, lane);
            if (lane == 0) lg[e] = v;
            continue;
        }
        // TB rows against one read of the expert's row: the same terms in the same order as
        // wave_dot_row, row by row
        float acc[TB];
#pragma unroll
        for (int u = 0; u < TB; ++u) acc[u] = 0.f;
        if (vec) {
            const int nv = d >> 2;
#pragma unroll 10
            for (int c = lane; c < nv; c += 64) {
                const f32x4 ww = ((const f32x4*)w)[c];
#pragma unroll
                for (int u = 0; u < TB; ++u) {
                    const f32x4 xx = ((const f32x4*)(xs + (size_t)u * d))[c];
                    acc[u] += ww[0] * xx[0] + ww[1] * xx[1] + ww[2] * xx[2] + ww[3] * xx[3];
                }
            }
        } else {
            for (int c = lane; c < d; c += 64) {
                const float ww = w[c];
#pragma unroll
                for (int u = 0; u < TB; ++u) acc[u] += ww * xs[(size_t)u * d + c];
            }
        }
#pragma unroll
        for (int u = 0; u < TB; ++u) {
            const float v = wave_sum(acc[u]);
            if (lane == 0) lg[u * E + e] = v;
        }
    }
    __syncthreads();
    if (logits_out)
        for (int i = threadIdx.x; i < TB * E; i += ROUTER_NT)
            if (t0 + i / E < T) logits_out[(size_t)(t0 + i / E) * E + i % E] = lg[i];
    if (threadIdx.x < TB && t0 + threadIdx.x < T) {
        const float* l = lg + threadIdx.x * E;
        float best = l[0]; int best_e = 0;
        for (int e = 1; e < E; ++e) if (l[e] > best) { best = l[e]; best_e = e; }
        expert[t0 + threadIdx.x] = best_e;
        weight[t0 + threadIdx.x] = 1.0f / (1.0f + expf(-best));
    }
}

extern "C" int spite_router_top1(const float* x, const float* wr, int* expert, float* weight,
                                 float* logits_out, int T, int d, int E, hipStream_t st) {
    SP_REQUIRE(T >= 0 && d > 0 && E > 0, "router: bad sizes T=%d d=%d E=%d", T, d, E);
    const size_t sh1 = (size_t)(d + E) * sizeof(float);
    SP_REQUIRE(sh1 <= 48 * 1024, "router: width %d with %d experts does not fit the kernel's LDS", d, E);
    if (T == 0) return 0;
    if (T >= 256 && 4 * sh1 <= 150 * 1024) {           // many tokens: four a workgroup
        static bool allowed = false;
        if (!allowed) {
            hipError_t e = hipFuncSetAttribute((const void*)router_top1_kernel<4>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
            SP_REQUIRE(e == hipSuccess, "router: LDS refused: %s", hipGetErrorString(e));
            allowed = true;
        }
        router_top1_kernel<4><<<(T + 3) / 4, ROUTER_NT, 4 * sh1, st>>>(x, wr, expert, weight, logits_out, T, d, E);
    } else {
        router_top1_kernel<1><<<T, ROUTER_NT, sh1, st>>>(x, wr, expert, weight, logits_out, T, d, E);
    }
    SP_LAUNCH_CHECK("router_top1");
    return 0;
}

// ------------------------------------------------------------------ expert plan
// From expert[t], weight[t] build the row list that the grouped products walk:
//   slots [0,T): tokens in order of expert (stable), src[s] = token, scale[s] = its weight,
//                dst[s] = token;
//   slots [T,2T) (if shared): src = dst-T = token, scale 1, dst[s] = T + token  (the group E
//                that every token visits);
//   offsets[g] = first slot of group g, g in [0, E+1] (+1 with the shared group).
// With `logits` ([T, E] fp32) the kernels make the router's choice themselves and write it to
// expert[] and weight[]: the largest logit, the lowest index among equals, weight =
// 1/(1+exp(-logit)).
__device__ __forceinline__ int top1_of(const float* __restrict__ l, int E, float* best_out) {
    float best = -INFINITY; int best_e = 0;
    if ((E & 3) == 0 && (((uintptr_t)l) & 15) == 0) {           // four logits a load
        for (int e = 0; e < E; e += 4) {
            const f32x4 v = *(const f32x4*)(l + e);
#pragma unroll
            for (int i = 0; i < 4; ++i) if (v[i] > best || (e + i == 0)) { best = v[i]; best_e = e + i; }
        }
    } else {
        best = l[0];
        for (int e = 1; e < E; ++e) { const float v = l[e]; if (v > best) { best = v; best_e = e; } }
    }
    if (best_out) *best_out = best;
    return best_e;
}

// Each thread ranks one token by counting over all tokens in shared memory: no atomics, the
// order is the same on every run.
__global__ void moe_plan_kernel(int* __restrict__ expert, float* __restrict__ weight,
                                const float* __restrict__ logits,
                                int* __restrict__ src, float* __restrict__ scale, int* __restrict__ dst,
                                int* __restrict__ offsets, int T, int E, int shared) {
    extern __shared__ unsigned short e_of[];
    for (int i = threadIdx.x; i < T; i += blockDim.x)
        e_of[i] = (unsigned short)(logits ? top1_of(logits + (size_t)i * E, E, nullptr) : expert[i]);
    __syncthreads();
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t < T) {
        const int me = e_of[t];
        float wt;
        if (logits) {
            float best;
            top1_of(logits + (size_t)t * E, E, &best);
            wt = 1.0f / (1.0f + expf(-best));
            expert[t] = me; weight[t] = wt;
        } else {
            wt = weight[t];
        }
        int rank = 0;
        for (int j = 0; j < T; ++j) {
            const int ej = e_of[j];
            rank += (ej < me) || (ej == me && j < t);
        }
        src[rank] = t; scale[rank] = wt; dst[rank] = t;
        if (shared) { src[T + t] = t; scale[T + t] = 1.0f; dst[T + t] = T + t; }
    }
    if (blockIdx.x == 0) {
        for (int g = threadIdx.x; g <= E; g += blockDim.x) {
            int c = 0;
            for (int j = 0; j < T; ++j) c += e_of[j] < g;
            offsets[g] = c;
        }
        if (shared && threadIdx.x == 0) offsets[E + 1] = 2 * T;
    }
}

// The same plan for up to PLAN_MAX_E experts in time linear in T: a workgroup of 256 tokens
// counts, in LDS, the tokens of every expert in the whole step and among the tokens before its
// own; a token's slot is then its expert's first slot + the expert's tokens before the
// workgroup + those before it inside the workgroup.  Counts are integers, so the atomics
// leave the same list on every run.
#define PLAN_MAX_E 2048
__global__ __launch_bounds__(256)
void moe_plan_hist_kernel(int* __restrict__ expert, float* __restrict__ weight,
                          const float* __restrict__ logits,
                          int* __restrict__ src, float* __restrict__ scale, int* __restrict__ dst,
                          int* __restrict__ offsets, int T, int E, int shared) {
    extern __shared__ int sh[];              // total[E], before[E], first[E+1], mine[256]
    int* total = sh; int* before = sh + E; int* first = sh + 2 * E; int* mine = sh + 3 * E + 1;
    const int c0 = blockIdx.x * 256, t = c0 + threadIdx.x;
    for (int e = threadIdx.x; e < 2 * E; e += 256) sh[e] = 0;
    __syncthreads();
    for (int j = threadIdx.x; j < T; j += 256) {
        const int e = logits ? top1_of(logits + (size_t)j * E, E, nullptr) : expert[j];
        if ((unsigned)e >= (unsigned)E) continue;       // not a token of any group
        atomicAdd(&total[e], 1);
        if (j < c0) atomicAdd(&before[e], 1);
    }
    int me = -1;
    float wt = 0.f;
    if (t < T) {
        if (logits) {
            float best;
            me = top1_of(logits + (size_t)t * E, E, &best);
            wt = 1.0f / (1.0f + expf(-best));
            expert[t] = me; weight[t] = wt;
        } else {
            me = expert[t]; wt = weight[t];
        }
    }
    mine[threadIdx.x] = me;
    __syncthreads();
    for (int g = threadIdx.x; g <= E; g += 256) {
        int c = 0;
        for (int e = 0; e < g; ++e) c += total[e];
        first[g] = c;
    }
    __syncthreads();
    if (t < T && (unsigned)me < (unsigned)E) {
        int rank = first[me] + before[me];
        for (int j = 0; j < (int)threadIdx.x; ++j) rank += mine[j] == me;
        src[rank] = t; scale[rank] = wt; dst[rank] = t;
        if (shared) { src[T + t] = t; scale[T + t] = 1.0f; dst[T + t] = T + t; }
    }
    if (blockIdx.x == 0) {
        for (int g = threadIdx.x; g <= E; g += 256) offsets[g] = first[g];
        if (shared && threadIdx.x == 0) offsets[E + 1] = 2 * T;
    }
}

// `logits` null: expert[] and weight[] are inputs; else they are outputs.
extern "C" int spite_moe_plan(int* expert, float* weight, const float* logits, int* src, float* scale, int* dst,
                              int* offsets, int T, int E, int shared, hipStream_t st) {
    SP_REQUIRE(T >= 0 && E > 0 && E < 65535, "moe_plan: bad sizes T=%d E=%d", T, E);
    SP_REQUIRE(T <= 32768, "moe_plan: %d tokens in one step, at most 32768", T);
    const int grid = T > 0 ? (T + 255) / 256 : 1;
    if (T > 256 && E <= PLAN_MAX_E)
        moe_plan_hist_kernel<<<grid, 256, (size_t)(3 * E + 1 + 256) * sizeof(int), st>>>(
            expert, weight, logits, src, scale, dst, offsets, T, E, shared);
    else
        moe_plan_kernel<<<grid, 256, (size_t)(T > 0 ? T : 1) * sizeof(unsigned short), st>>>(
            expert, weight, logits, src, scale, dst, offsets, T, E, shared);
    SP_LAUNCH_CHECK("moe_plan");
    return 0;
}

// ------------------------------------------------------------------ small helpers
template <typename TI, typename TO>
__global__ void convert_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        out[i] = from_f32<TO>(to_f32<TI>(in[i]));
}
extern "C" int spite_convert(const void* in, int in_dtype, void* out, int out_dtype, size_t n, hipStream_t st) {
    if (n == 0) return 0;
    const int grid = (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
    if (in_dtype == SP_F32 && out_dtype == SP_BF16) convert_kernel<float, bf16><<<grid, 256, 0, st>>>((const float*)in, (bf16*)out, n);
    else if (in_dtype == SP_BF16 && out_dtype == SP_F32) convert_kernel<bf16, float><<<grid, 256, 0, st>>>((const bf16*)in, (float*)out, n);
    else if (in_dtype == SP_F32 && out_dtype == SP_F32) convert_kernel<float, float><<<grid, 256, 0, st>>>((const float*)in, (float*)out, n);
    else if (in_dtype == SP_BF16 && out_dtype == SP_BF16) convert_kernel<bf16, bf16><<<grid, 256, 0, st>>>((const bf16*)in, (bf16*)out, n);
    else return sp_fail("convert: unknown dtypes %d -> %d", in_dtype, out_dtype);
    SP_LAUNCH_CHECK("convert");
    return 0;
}

// h[i] += d[i] over rows of width `d_cols` (fp32): an increment of the residual stream that no
// norm's two addends have room for.  Row r of d is row r of h.
__global__ void add_into_kernel(float* __restrict__ h, const float* __restrict__ d, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        h[i] += d[i];
}
extern "C" int spite_add_into(float* h, const float* d, size_t n, hipStream_t st) {
    if (n == 0) return 0;
    const int grid = (int)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
    add_into_kernel<<<grid, 256, 0, st>>>(h, d, n);
    SP_LAUNCH_CHECK("add_into");
    return 0;
}

// ------------------------------------------------------------------ random weights
// out[i] = mean + std * z(seed, key, i), z standard normal: element i of a tensor depends on the
// seed, the tensor's key (a hash of its name) and i alone, not on the order in which tensors
// or elements are drawn.  A 64-bit mix of (seed, key, i / 2) gives two uniform numbers of 32 bits,
// and Box-Muller turns them into the normals of the elements i and i + 1.
//
// The same numbers can be drawn on the host, bit for bit: logarithm, sine and cosine are
// computed here from IEEE double additions, multiplications, divisions and one square root in
// a fixed order, never fused (a fused multiply-add rounds once where the host rounds twice),
// instead of the device library's routines, whose last bits differ from a host library's.
__device__ __forceinline__ unsigned long long mix64(unsigned long long x) {
    x ^= x >> 30; x *= 0xbf58476d1ce4e5b9ull;
    x ^= x >> 27; x *= 0x94d049bb133111ebull;
    return x ^ (x >> 31);
}
// ln(x) for x in (0, 1]: x = m * 2^e with m in [sqrt(1/2), sqrt(2)), ln(m) = 2 atanh(s) with
// s = (m-1)/(m+1), |s| < 0.172: the series up to s^23 is exact to double rounding.
__device__ __forceinline__ double exact_log(double x) {
#pragma clang fp contract(off)
    int e;
    double m = frexp(x, &e);
    if (m < 0.70710678118654752) { m = m * 2.0; e -= 1; }
    const double s = (m - 1.0) / (m + 1.0);
    const double s2 = s * s;
    double p = 1.0 / 23.0;
    p = p * s2 + 1.0 / 21.0;
    p = p * s2 + 1.0 / 19.0;
    p = p * s2 + 1.0 / 17.0;
    p = p * s2 + 1.0 / 15.0;
    p = p * s2 + 1.0 / 13.0;
    p = p * s2 + 1.0 / 11.0;
    p = p * s2 + 1.0 / 9.0;
    p = p * s2 + 1.0 / 7.0;
    p = p * s2 + 1.0 / 5.0;
    p = p * s2 + 1.0 / 3.0;
    p = p * s2 + 1.0;
    return (double)e * 0.6931471805599453 + 2.0 * (s * p);
}
// sine and cosine of the angle 2 pi k / 2^32: the quadrant from the two top bits, the angle inside
// it folded to [0, pi/4] (sin(pi/2 - t) = cos t), Taylor sums there up to t^17 and t^18.
__device__ __forceinline__ void exact_sincos_turns(unsigned k, double& sn, double& cs) {
#pragma clang fp contract(off)
    const unsigned quad = k >> 30, low = k & 0x3fffffffu;
    const bool fold = low > 0x20000000u;
    const unsigned a = fold ? 0x40000000u - low : low;
    const double t = (double)a * (1.5707963267948966 / 1073741824.0);
    const double t2 = t * t;
    double ps = 1.0 / 355687428096000.0;
    ps = ps * t2 - 1.0 / 1307674368000.0;
    ps = ps * t2 + 1.0 / 6227020800.0;
    ps = ps * t2 - 1.0 / 39916800.0;
    ps = ps * t2 + 1.0 / 362880.0;
    ps = ps * t2 - 1.0 / 5040.0;
    ps = ps * t2 + 1.0 / 120.0;
    ps = ps * t2 - 1.0 / 6.0;
    ps = ps * t2 + 1.0;
    double pc = -1.0 / 6402373705728000.0;
    pc = pc * t2 + 1.0 / 20922789888000.0;
    pc = pc * t2 - 1.0 / 87178291200.0;
    pc = pc * t2 + 1.0 / 479001600.0;
    pc = pc * t2 - 1.0 / 3628800.0;
    pc = pc * t2 + 1.0 / 40320.0;
    pc = pc * t2 - 1.0 / 720.0;
    pc = pc * t2 + 1.0 / 24.0;
    pc = pc * t2 - 1.0 / 2.0;
    pc = pc * t2 + 1.0;
    const double s0 = fold ? pc : t * ps, c0 = fold ? t * ps : pc;
    sn = quad == 0 ? s0 : quad == 1 ? c0 : quad == 2 ? -s0 : -c0;
    cs = quad == 0 ? c0 : quad == 1 ? -s0 : quad == 2 ? -c0 : s0;
}
template <typename T>
__global__ __launch_bounds__(256)
void randn_fill_kernel(T* __restrict__ out, size_t n, unsigned long long seed, unsigned long long key, float mean, float std) {
#pragma clang fp contract(off)
    const unsigned long long base = mix64(seed * 0x9e3779b97f4a7c15ull + key);
    const size_t pairs = (n + 1) / 2;
    for (size_t j = (size_t)blockIdx.x * blockDim.x + threadIdx.x; j < pairs; j += (size_t)gridDim.x * blockDim.x) {
        const unsigned long long h = mix64(base + j * 0xd1342543de82ef95ull);
        const double u1 = ((double)(unsigned)(h >> 32) + 1.0) * (1.0 / 4294967296.0);          // (0, 1]
        const double r = sqrt(-2.0 * exact_log(u1));
        double sn, cs;
        exact_sincos_turns((unsigned)h, sn, cs);
        const float z0 = (float)(r * cs), z1 = (float)(r * sn);
        out[2 * j] = from_f32<T>(std * z0 + mean);
        if (2 * j + 1 < n) out[2 * j + 1] = from_f32<T>(std * z1 + mean);
    }
}
extern "C" int spite_randn_fill(void* out, int dtype, size_t n, unsigned long long seed, unsigned long long key,
                                float mean, float std, hipStream_t st) {
    SP_REQUIRE(std >= 0.f, "randn_fill: a deviation of %g", std);
    if (n == 0) return 0;
    const size_t blocks = ((n + 1) / 2 + 255) / 256;
    const int grid = (int)(blocks < 16384 ? blocks : 16384);
    if (dtype == SP_BF16) randn_fill_kernel<bf16><<<grid, 256, 0, st>>>((bf16*)out, n, seed, key, mean, std);
    else if (dtype == SP_F32) randn_fill_kernel<float><<<grid, 256, 0, st>>>((float*)out, n, seed, key, mean, std);
    else return sp_fail("randn_fill: unknown dtype %d", dtype);
    SP_LAUNCH_CHECK("randn_fill");
    return 0;
}

// ------------------------------------------------------------------ what the memory gives
// Reads `n16` 16-byte words once, with non-temporal loads, a contiguous piece per workgroup
// (512 threads, four loads in flight each: the form that a sweep over threads, unrolling and
// workgroups found fastest), and leaves one float per wave in `out` so that the loads cannot be
// dropped: the measure of the read bandwidth that the weight-streaming kernels are held against.
__global__ __launch_bounds__(512)
void stream_read_kernel(const f32x4* __restrict__ p, size_t n16, size_t per_block, float* __restrict__ out) {
    const size_t b0 = (size_t)blockIdx.x * per_block;
    const size_t b1 = b0 + per_block < n16 ? b0 + per_block : n16;
    f32x4 acc[4] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
    size_t i = b0 + threadIdx.x;
    for (; i + 3 * 512 < b1; i += 4 * 512) {
#pragma unroll
        for (int u = 0; u < 4; ++u) acc[u] += __builtin_nontemporal_load(p + i + u * 512);
    }
    for (; i < b1; i += 512) acc[0] += __builtin_nontemporal_load(p + i);
    const f32x4 a = acc[0] + acc[1] + acc[2] + acc[3];
    const float v = wave_sum(a[0] + a[1] + a[2] + a[3]);
    if ((threadIdx.x & 63) == 0) out[blockIdx.x * 8 + (threadIdx.x >> 6)] = v;
}
extern "C" int spite_stream_read(const void* p, size_t nbytes, float* out, int n_blocks, hipStream_t st) {
    SP_REQUIRE(((uintptr_t)p & 15) == 0 && nbytes % 16 == 0, "stream_read: 16-byte words only");
    SP_REQUIRE(n_blocks > 0, "stream_read: no workgroups");
    const size_t n16 = nbytes / 16;
    if (n16 == 0) return 0;
    const size_t per = (n16 + n_blocks - 1) / n_blocks;
    stream_read_kernel<<<n_blocks, 512, 0, st>>>((const f32x4*)p, n16, per, out);
    SP_LAUNCH_CHECK("stream_read");
    return 0;
}

// ------------------------------------------------------------------ the matrix units alone, for measurement
// 32 independent MFMA 16x16x32 a step on operands that stay in registers: what the chip gives to the
// products when nothing else moves.  `gain` scales the operands' pseudo-random values; with 0 nothing
// toggles, and the rate shows how much of the time under real values is the chip's power limit.
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void mfma_loop_kernel(float* __restrict__ out, int steps, float gain) {
    const unsigned id = blockIdx.x * 512 + threadIdx.x;
    auto operand = [&](unsigned seed) {
        bf16x8 v;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            unsigned x = (id * 16 + seed) * 8 + e;
            x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
            v[e] = (bf16)(((int)(x & 0xffff) - 32768) / 32768.0f * gain);
        }
        return v;
    };
    bf16x8 a[4], b[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = operand(i);
#pragma unroll
    for (int i = 0; i < 8; ++i) b[i] = operand(4 + i);
    f32x4 acc[4][8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int t = 0; t < steps; ++t) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) s += acc[i][j][0] + acc[i][j][3];
    if (threadIdx.x == 0) out[blockIdx.x] = s;
}

// Runs `n_blocks` workgroups of eight waves, each wave `steps` times 32 MFMAs of 16,384 flops.
extern "C" int spite_mfma_loop(float* out, int n_blocks, int steps, float gain, hipStream_t st) {
    SP_REQUIRE(n_blocks > 0 && steps > 0 && out, "mfma_loop: %d workgroups, %d steps", n_blocks, steps);
    mfma_loop_kernel<<<n_blocks, 512, 0, st>>>(out, steps, gain);
    SP_LAUNCH_CHECK("mfma_loop");
    return 0;
}
