// Row-wise and element-wise kernels: embedding gather, (residual add +) RMSNorm,
// per-head QK-norm + rotary embedding + cache write, SwiGLU.
//
// Formulas follow the reference's kernels; the fusions are ours (the reference launches each
// op on its own and rounds to bf16 in between, src/qwen.cc:574-799):
//   embedding   src/kernels/embedding.cu:22-38
//   RMSNorm     src/kernels/rmsnorm.cu:56-97     y = x * rsqrt(mean(x^2) + eps) * w
//   residual    src/kernels/add.cu:11-14         a + b in fp32
//   QK-norm     src/qwen.cc:617-632              RMSNorm over head_dim, one [d] weight
//   rotary      src/kernels/rope.cu:28-60        pairs (i, i + d/2), angle = pos / theta^(2i/d)
//   cache write src/kernels/attention_paged.cu:26-44
//   SwiGLU      src/kernels/swiglu.cu:8,31-35    g / (1 + exp(-g)) * u
#include "common.h"

#include <cstdarg>
#include <cstdio>

namespace lc {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

// Asked once per process, of the device that is current then (the library serves one GPU).
int device_cus() {
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            return 256;     // no device to ask (a build check on a machine without one)
        }
        return n;
    }();
    return cus;
}

// ------------------------------------------------------------------------------- embedding
template <typename TW>
__global__ void embedding_kernel(const int* __restrict__ ids, const TW* __restrict__ table,
                                 float* __restrict__ out, int H, int V, float scale) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (id < 0 || id >= V) id = 0;  // the host has rejected such ids already
    const TW* row = table + (size_t)id * H;
    float* dst = out + (size_t)t * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = to_f32(row[i]) * scale;   // scale 1: exact
}

// ------------------------------------------------------------------------------- RMSNorm
// One workgroup per output row r.  src row = rows ? rows[r] : r.
//   v = h[src] (+ delta[src]);  if (write_h) h[src] = v;  out[r] = v * rsqrt(mean(v^2)+eps) * w
// With sumsq: out[r] = v * w and sumsq[r] = sum(v^2): the row's factor is left to the product
// that reads out (gemm_bf16.hip, scaled rows).
// With shares > 0, delta is not a tensor of T but float32 [shares][all rows of h][n]: the shares
// of a product that was cut along K (gemm_bf16.hip), added here in their order.
template <typename T>
__global__ void rmsnorm_kernel(float* __restrict__ h, const T* __restrict__ delta,
                               const int* __restrict__ rows, const float* __restrict__ w,
                               float eps, T* __restrict__ out, int n, int write_h,
                               float* __restrict__ sumsq, int shares, size_t share_stride) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    float* hr = h + (size_t)src * n;
    const T* dr = (delta && !shares) ? delta + (size_t)src * n : nullptr;
    const float* pr = shares ? reinterpret_cast<const float*>(delta) + (size_t)src * n : nullptr;
    auto branch = [&](int i) {
        if (dr) return to_f32(dr[i]);
        float t = 0.f;
        for (int s = 0; s < shares; ++s) t += pr[s * share_stride + i];
        return t;
    };
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = hr[i];
        if (dr || pr) {
            v += branch(i);
            if (write_h) hr[i] = v;
        }
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float inv = sumsq ? 1.f : rsqrtf(ss / (float)n + eps);
    if (sumsq && threadIdx.x == 0) sumsq[r] = ss;
    T* o = out + (size_t)r * n;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = hr[i];
        if ((dr || pr) && !write_h) v += branch(i);
        o[i] = from_f32<T>(v * inv * w[i]);
    }
}

// The same for rows of up to 8192 entries whose length is a multiple of 8: every thread keeps
// its entries in registers between the sum of squares and the scaling, and all of a thread's
// loads are issued before the first is used (the plain kernel above walks a row with one
// dependent load after the other).
template <typename T> struct Pack8;
template <> struct Pack8<float> {
    float4 a, b;
    __device__ __forceinline__ float get(int i) const { return i < 4 ? (&a.x)[i] : (&b.x)[i - 4]; }
    __device__ __forceinline__ void set(int i, float v) { if (i < 4) (&a.x)[i] = v; else (&b.x)[i - 4] = v; }
};
template <> struct Pack8<bf16> {
    typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
    bf16x8 v;
    __device__ __forceinline__ float get(int i) const { return static_cast<float>(v[i]); }
    __device__ __forceinline__ void set(int i, float f) { v[i] = static_cast<bf16>(f); }
};

constexpr int RN_THREADS = 256, RN_CHUNKS = 4;   // 256 threads x 4 chunks x 8 entries = 8192

// THREADS x CHUNKS x 8 entries at most.  Few rows (a decode step) leave most CUs without a
// workgroup, and the ones that have one are bound by what its waves keep in flight: 1024 threads
// with one chunk each then, 256 with four for many rows.
template <typename T, int THREADS, int CHUNKS>
__global__ __launch_bounds__(THREADS) void rmsnorm_vec_kernel(
    float* __restrict__ h, const T* __restrict__ delta, const int* __restrict__ rows,
    const float* __restrict__ w, float eps, T* __restrict__ out, int n, int write_h,
    float* __restrict__ sumsq, int shares, size_t share_stride) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    float* hr = h + (size_t)src * n;
    const T* dr = (delta && !shares) ? delta + (size_t)src * n : nullptr;
    const float* pr = shares ? reinterpret_cast<const float*>(delta) + (size_t)src * n : nullptr;
    const int chunks = n / 8;
    Pack8<float> hv[CHUNKS], wv[CHUNKS];
    Pack8<T> dv[CHUNKS];
    // everything the row needs is asked for at once, the weights too: one trip to memory
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int chunk = threadIdx.x + c * THREADS;
        if (chunk < chunks) {
            hv[c] = *reinterpret_cast<const Pack8<float>*>(hr + chunk * 8);
            if (dr) dv[c] = *reinterpret_cast<const Pack8<T>*>(dr + chunk * 8);
            wv[c] = *reinterpret_cast<const Pack8<float>*>(w + chunk * 8);
        }
    }
    if (pr) {   // the shares of the branch's product, in their order, then the stream
        // up to AT_ONCE shares are asked for together and added in their order once they are
        // back (a share past the last is the last one again, loaded and not added): a loop
        // that adds each share as it arrives makes one trip to memory per share
        constexpr int AT_ONCE = CHUNKS == 1 ? 8 : 4;
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int chunk = threadIdx.x + c * THREADS;
            if (chunk < chunks) {
                Pack8<float> sum = *reinterpret_cast<const Pack8<float>*>(pr + chunk * 8);
                for (int s0 = 1; s0 < shares; s0 += AT_ONCE) {
                    Pack8<float> part[AT_ONCE];
#pragma unroll
                    for (int a = 0; a < AT_ONCE; ++a)
                        part[a] = *reinterpret_cast<const Pack8<float>*>(
                            pr + (size_t)min(s0 + a, shares - 1) * share_stride + chunk * 8);
#pragma unroll
                    for (int a = 0; a < AT_ONCE; ++a) {
                        if (s0 + a < shares) {
#pragma unroll
                            for (int i = 0; i < 8; ++i) sum.set(i, sum.get(i) + part[a].get(i));
                        }
                    }
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) hv[c].set(i, hv[c].get(i) + sum.get(i));
            }
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int chunk = threadIdx.x + c * THREADS;
        if (chunk < chunks) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float v = hv[c].get(i);
                if (dr) v += dv[c].get(i);
                hv[c].set(i, v);
                ss += v * v;
            }
            if ((dr || pr) && write_h) *reinterpret_cast<Pack8<float>*>(hr + chunk * 8) = hv[c];
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = sumsq ? 1.f : rsqrtf(ss / (float)n + eps);
    if (sumsq && threadIdx.x == 0) sumsq[r] = ss;
    T* o = out + (size_t)r * n;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int chunk = threadIdx.x + c * THREADS;
        if (chunk < chunks) {
            Pack8<T> ov;
#pragma unroll
            for (int i = 0; i < 8; ++i) ov.set(i, hv[c].get(i) * inv * wv[c].get(i));
            *reinterpret_cast<Pack8<T>*>(o + chunk * 8) = ov;
        }
    }
}

// RMSNorm of rows held in the activation type (no residual stream involved).
template <typename T>
__global__ void rmsnorm_act_kernel(const T* __restrict__ x, const float* __restrict__ w,
                                   float eps, T* __restrict__ out, int n) {
    __shared__ float scratch[16];
    const T* xr = x + (size_t)blockIdx.x * n;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = to_f32(xr[i]);
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float inv = rsqrtf(ss / (float)n + eps);
    T* o = out + (size_t)blockIdx.x * n;
    for (int i = threadIdx.x; i < n; i += blockDim.x)
        o[i] = from_f32<T>(to_f32(xr[i]) * inv * w[i]);
}

// ------------------------------------------------------- QK-norm + rotary + cache write
// qkv: [T, nh + 2 nkv, d] (q heads, then k heads, then v heads).  One wave per (token, head).
//   q, k: optional RMSNorm over d, then rotation of the first `rot` dims with the angles of
//   the token's position (cos in table[pos][0:rot/2], sin in table[pos][rot/2:rot]).
//   q and k are written back in place; k and v also go to the cache page slot of the token.
// Cache layouts: keys [pages, nkv, page_size, d], values transposed [pages, nkv, d, page_size]
// (a value's positions lie next to each other, which is how the matrix cores want the P.V
// operand); slot = page * page_size + offset; slot < 0 skips.
template <typename T>
__global__ void qk_norm_rope_write_kernel(T* __restrict__ qkv, int T_tokens, int nh, int nkv, int d,
                                          const float* __restrict__ q_w,
                                          const float* __restrict__ k_w, float eps,
                                          const int* __restrict__ positions,
                                          const float* __restrict__ rope_table, int rot,
                                          T* __restrict__ k_cache, T* __restrict__ v_cache,
                                          const int* __restrict__ slots, int page_size, int first_head) {
    const int t = blockIdx.x;
    const int wave = threadIdx.x / kWave;
    const int lane = threadIdx.x & (kWave - 1);
    const int waves = blockDim.x / kWave;
    const int heads = nh + 2 * nkv;
    const int head = first_head + blockIdx.y * waves + wave;     // heads before first_head are left alone
    if (head >= heads) return;
    T* x = qkv + ((size_t)t * heads + head) * d;

    const bool is_q = head < nh;
    const bool is_k = !is_q && head < nh + nkv;
    const int kvh = is_q ? 0 : (is_k ? head - nh : head - nh - nkv);

    T* cache_row = nullptr;   // k: the slot's row of d entries;  v: the slot's column (stride page_size)
    if (!is_q && slots && k_cache) {
        const int slot = slots[t];
        if (slot >= 0) {
            const int page = slot / page_size, off = slot - page * page_size;
            if (is_k)
                cache_row = k_cache + (((size_t)page * nkv + kvh) * page_size + off) * d;
            else
                cache_row = v_cache + ((size_t)page * nkv + kvh) * d * page_size + off;
        }
    }

    if (!is_q && !is_k) {  // v: copy only, transposed into the page
        if (cache_row)
            for (int i = lane; i < d; i += kWave) cache_row[(size_t)i * page_size] = x[i];
        return;
    }

    const float* w = is_q ? q_w : k_w;
    float inv = 1.f;
    if (w) {
        float ss = 0.f;
        for (int i = lane; i < d; i += kWave) {
            float v = to_f32(x[i]);
            ss += v * v;
        }
        ss = wave_sum(ss);
        inv = rsqrtf(ss / (float)d + eps);
    }
    const int half = rot / 2;
    const float* cs = rope_table ? rope_table + (size_t)positions[t] * rot : nullptr;
    // rotated pairs
    for (int i = lane; i < half; i += kWave) {
        float a = to_f32(x[i]) * inv, b = to_f32(x[i + half]) * inv;
        if (w) { a *= w[i]; b *= w[i + half]; }
        float c = 1.f, s = 0.f;
        if (cs) { c = cs[i]; s = cs[half + i]; }
        const T ra = from_f32<T>(a * c - b * s);
        const T rb = from_f32<T>(a * s + b * c);
        x[i] = ra;
        x[i + half] = rb;
        if (cache_row) { cache_row[i] = ra; cache_row[i + half] = rb; }
    }
    // dims beyond the rotary part
    for (int i = rot + lane; i < d; i += kWave) {
        float a = to_f32(x[i]) * inv;
        if (w) a *= w[i];
        const T ra = from_f32<T>(a);
        x[i] = ra;
        if (cache_row) cache_row[i] = ra;
    }
}

// The same for bfloat16 heads of 128 entries that rotate whole or not at all: 16 lanes a head,
// 16-byte loads and stores, 16 heads a workgroup.
__global__ __launch_bounds__(256) void qk_norm_rope_write128_kernel(
    bf16* __restrict__ qkv, int T_tokens, int nh, int nkv, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps, const int* __restrict__ positions,
    const float* __restrict__ rope_table, bf16* __restrict__ k_cache, bf16* __restrict__ v_cache,
    const int* __restrict__ slots, int page_size, int first_head) {
    constexpr int d = 128;
    const int heads = nh + 2 * nkv, span = heads - first_head;   // heads before first_head are left alone
    const long long g = (long long)blockIdx.x * 16 + (threadIdx.x >> 4);
    if (g >= (long long)T_tokens * span) return;           // whole groups of 16 lanes leave together
    const int t = (int)(g / span), head = first_head + (int)(g - (long long)t * span), j = threadIdx.x & 15;
    bf16* x = qkv + ((size_t)t * heads + head) * d + 8 * j;
    const bool is_q = head < nh, is_k = !is_q && head < nh + nkv;
    const int kvh = is_q ? 0 : (is_k ? head - nh : head - nh - nkv);
    const int slot = (!is_q && slots && k_cache) ? slots[t] : -1;
    const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot - page * page_size : 0;
    const head_chunk raw = *reinterpret_cast<const head_chunk*>(x);
    if (!is_q && !is_k) {      // v: copied, transposed into the page
        if (slot >= 0) {
            bf16* col = v_cache + ((size_t)page * nkv + kvh) * d * page_size + off;
#pragma unroll
            for (int e = 0; e < 8; ++e) col[(size_t)(8 * j + e) * page_size] = raw[e];
        }
        return;
    }
    const float* cs = rope_table ? rope_table + (size_t)positions[t] * d : nullptr;
    const head_chunk done = head128_norm_rope(raw, j, is_q ? q_w : k_w, eps, cs);
    *reinterpret_cast<head_chunk*>(x) = done;
    if (is_k && slot >= 0)
        *reinterpret_cast<head_chunk*>(k_cache + (((size_t)page * nkv + kvh) * page_size + off) * d + 8 * j) = done;
}

// k and v alone (q is left to the attention kernels), bfloat16 heads of 128 as above: a
// workgroup takes 16 consecutive rows of the batch and one kv head, 16 lanes a row.  A value
// page holds its 16 positions side by side for every entry of the head, so a row's values go
// to 128 places 32 bytes apart.  When the workgroup's 16 rows fill one page in order (the rows
// of a prompt do, from a page's first position on), it turns the 16 x 128 values round in
// LDS and writes the page's 4 KB of this head in one piece; otherwise every row scatters its
// own.
__global__ __launch_bounds__(256) void kv_norm_rope_write128_kernel(
    bf16* __restrict__ qkv, int T_tokens, int nh, int nkv, const float* __restrict__ k_w, float eps,
    const int* __restrict__ positions, const float* __restrict__ rope_table,
    bf16* __restrict__ k_cache, bf16* __restrict__ v_cache, const int* __restrict__ slots,
    int page_size) {
    constexpr int d = 128, LD = d + 8;            // padded rows: the gather below spreads over the banks
    __shared__ __attribute__((aligned(16))) bf16 turned[16 * LD];
    __shared__ int whole;
    const int t0 = blockIdx.x * 16, kvh = blockIdx.y, g = threadIdx.x >> 4, j = threadIdx.x & 15;
    const int t = t0 + g, heads = nh + 2 * nkv;
    const bool live = t < T_tokens;                           // whole groups of 16 lanes
    const int slot = live ? slots[t] : -1, base = slots[t0];
    if (threadIdx.x == 0) whole = (page_size == 16 && base >= 0 && base % 16 == 0) ? 1 : 0;
    __syncthreads();
    if (j == 0 && slot != base + g) whole = 0;                // (everyone who writes, writes 0)
    __syncthreads();
    const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot - page * page_size : 0;
    head_chunk value;
    if (live) {
        bf16* x = qkv + ((size_t)t * heads + nh + kvh) * d + 8 * j;
        const float* cs = rope_table ? rope_table + (size_t)positions[t] * d : nullptr;
        const head_chunk key = head128_norm_rope(*reinterpret_cast<const head_chunk*>(x), j, k_w, eps, cs);
        *reinterpret_cast<head_chunk*>(x) = key;
        if (slot >= 0)
            *reinterpret_cast<head_chunk*>(k_cache + (((size_t)page * nkv + kvh) * page_size + off) * d + 8 * j) = key;
        value = *reinterpret_cast<const head_chunk*>(x + (size_t)nkv * d);
    }
    if (whole) {                                              // the same for the whole workgroup
        *reinterpret_cast<head_chunk*>(&turned[g * LD + 8 * j]) = value;
        __syncthreads();
        const int dim = threadIdx.x >> 1, half = threadIdx.x & 1;
        head_chunk column;
#pragma unroll
        for (int i = 0; i < 8; ++i) column[i] = turned[(8 * half + i) * LD + dim];
        const int first_page = base / 16;
        *reinterpret_cast<head_chunk*>(v_cache + (((size_t)first_page * nkv + kvh) * d + dim) * 16 + 8 * half) = column;
    } else if (live && slot >= 0) {
        bf16* col = v_cache + ((size_t)page * nkv + kvh) * d * page_size + off;
#pragma unroll
        for (int e = 0; e < 8; ++e) col[(size_t)(8 * j + e) * page_size] = value[e];
    }
}

// ------------------------------------------------------------------------------- SwiGLU
// gu: [T, 2 I] (gate columns, then up columns) -> out [T, I]
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total) {
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t t = idx / I;
        const int i = (int)(idx - t * I);
        const float g = to_f32(gu[t * 2 * I + i]);
        const float u = to_f32(gu[t * 2 * I + I + i]);
        out[idx] = from_f32<T>(g / (1.f + expf(-g)) * u);
    }
}

}  // namespace lc

using namespace lc;

LC_API const char* lc_last_error() { return g_error; }

LC_API int lc_embedding(const int* ids, const void* table, int table_dt, float* out, int T, int H,
                        int V, float scale, hipStream_t stream) {
    LC_CHECK(T >= 0 && H > 0 && V > 0, "embedding: bad sizes T=%d H=%d V=%d", T, H, V);
    if (T == 0) return 0;
    LC_CHECK(ids && table && out, "embedding: null pointer");
    const int threads = H >= 256 ? 256 : 64;
    if (table_dt == DT_F32)
        embedding_kernel<float><<<T, threads, 0, stream>>>(ids, (const float*)table, out, H, V, scale);
    else if (table_dt == DT_BF16)
        embedding_kernel<bf16><<<T, threads, 0, stream>>>(ids, (const bf16*)table, out, H, V, scale);
    else
        LC_CHECK(false, "embedding: unknown table dtype %d", table_dt);
    LC_LAUNCH_CHECK("embedding");
    return 0;
}

// sumsq (may be null): R floats; then out = (h + delta) * w without the rows' factors, and
// sumsq[r] = the row's sum of squares.
// shares > 0: delta is float32 [shares][h_rows][n], the shares of a product cut along K; what
// is added to h is their sum in the order of the shares.
LC_API int lc_rmsnorm(float* h, const void* delta, const int* rows, const float* w, float eps,
                      void* out, int dt, int R, int n, int write_h, float* sumsq, int shares,
                      int h_rows, hipStream_t stream) {
    LC_CHECK(shares >= 0 && (shares == 0 || (delta && h_rows > 0)), "rmsnorm: bad shares %d", shares);
    const size_t share_stride = (size_t)h_rows * n;
    LC_CHECK(R >= 0 && n > 0, "rmsnorm: bad sizes R=%d n=%d", R, n);
    if (R == 0) return 0;
    LC_CHECK(h && w && out, "rmsnorm: null pointer");
    LC_CHECK(!(rows && write_h), "rmsnorm: gathered rows cannot be written back");
    const int threads = n >= 1024 ? 256 : (n >= 256 ? 128 : 64);
    const bool vec = n % 8 == 0 && n >= 512 && n <= RN_THREADS * RN_CHUNKS * 8 &&
                     (uintptr_t)h % 16 == 0 && (uintptr_t)delta % 16 == 0 && (uintptr_t)out % 16 == 0 &&
                     (uintptr_t)w % 16 == 0;
    // float32 results must not depend on how many rows share a step: there the shape of the
    // kernel, and with it the grouping of a row's sum of squares, follows from n alone
    const bool few = dt == DT_BF16 && R <= 128 && n > 2048 && n <= 8192;
    if (dt == DT_F32) {
        if (vec)
            rmsnorm_vec_kernel<float, RN_THREADS, RN_CHUNKS><<<R, RN_THREADS, 0, stream>>>(h, (const float*)delta, rows, w, eps,
                                                                    (float*)out, n, write_h, sumsq, shares, share_stride);
        else
            rmsnorm_kernel<float><<<R, threads, 0, stream>>>(h, (const float*)delta, rows, w, eps,
                                                             (float*)out, n, write_h, sumsq, shares, share_stride);
    } else if (dt == DT_BF16) {
        if (vec && few)
            rmsnorm_vec_kernel<bf16, 1024, 1><<<R, 1024, 0, stream>>>(h, (const bf16*)delta, rows, w, eps,
                                                                      (bf16*)out, n, write_h, sumsq, shares, share_stride);
        else if (vec)
            rmsnorm_vec_kernel<bf16, RN_THREADS, RN_CHUNKS><<<R, RN_THREADS, 0, stream>>>(h, (const bf16*)delta, rows, w, eps,
                                                                   (bf16*)out, n, write_h, sumsq, shares, share_stride);
        else
            rmsnorm_kernel<bf16><<<R, threads, 0, stream>>>(h, (const bf16*)delta, rows, w, eps,
                                                            (bf16*)out, n, write_h, sumsq, shares, share_stride);
    } else {
        LC_CHECK(false, "rmsnorm: unknown dtype %d", dt);
    }
    LC_LAUNCH_CHECK("rmsnorm");
    return 0;
}

LC_API int lc_rmsnorm_act(const void* x, const float* w, float eps, void* out, int dt, int R,
                          int n, hipStream_t stream) {
    LC_CHECK(R >= 0 && n > 0, "rmsnorm_act: bad sizes R=%d n=%d", R, n);
    if (R == 0) return 0;
    LC_CHECK(x && w && out, "rmsnorm_act: null pointer");
    const int threads = n >= 1024 ? 256 : (n >= 256 ? 128 : 64);
    if (dt == DT_F32)
        rmsnorm_act_kernel<float><<<R, threads, 0, stream>>>((const float*)x, w, eps, (float*)out, n);
    else if (dt == DT_BF16)
        rmsnorm_act_kernel<bf16><<<R, threads, 0, stream>>>((const bf16*)x, w, eps, (bf16*)out, n);
    else
        LC_CHECK(false, "rmsnorm_act: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("rmsnorm_act");
    return 0;
}

LC_API int lc_qk_norm_rope_write(void* qkv, int dt, int T, int nh, int nkv, int d,
                                 const float* q_w, const float* k_w, float eps,
                                 const int* positions, const float* rope_table, int rot,
                                 void* k_cache, void* v_cache, const int* slots, int page_size,
                                 int first_head, hipStream_t stream) {
    LC_CHECK(T >= 0 && nh > 0 && nkv > 0 && d > 0, "qk_norm_rope_write: bad sizes T=%d nh=%d nkv=%d d=%d",
             T, nh, nkv, d);
    LC_CHECK(first_head == 0 || first_head == nh, "qk_norm_rope_write: first head %d (0: all heads, %d: k and v only)",
             first_head, nh);
    if (T == 0) return 0;
    LC_CHECK(qkv, "qk_norm_rope_write: null qkv");
    LC_CHECK(rot >= 0 && rot <= d && rot % 2 == 0,
             "qk_norm_rope_write: rotary dims %d must be even and at most head_dim %d", rot, d);
    LC_CHECK(!rope_table || positions, "qk_norm_rope_write: rotary table without positions");
    LC_CHECK(!(k_cache && slots) || (v_cache && page_size > 0),
             "qk_norm_rope_write: cache write needs v_cache and a page size");
    if (!rope_table) rot = 0;
    if (dt == DT_BF16 && d == 128 && (rot == 0 || rot == 128) && (q_w == nullptr) == (k_w == nullptr) &&
        (uintptr_t)qkv % 16 == 0 && (uintptr_t)k_cache % 16 == 0 && (uintptr_t)q_w % 16 == 0 &&
        (uintptr_t)k_w % 16 == 0 && (uintptr_t)rope_table % 16 == 0) {
        if (first_head == nh && k_cache && slots) {
            kv_norm_rope_write128_kernel<<<dim3((T + 15) / 16, nkv), 256, 0, stream>>>(
                (bf16*)qkv, T, nh, nkv, k_w, eps, positions, rope_table, (bf16*)k_cache, (bf16*)v_cache,
                slots, page_size);
            LC_LAUNCH_CHECK("kv_norm_rope_write128");
            return 0;
        }
        const long long groups = (long long)T * (nh + 2 * nkv - first_head);
        qk_norm_rope_write128_kernel<<<(unsigned)((groups + 15) / 16), 256, 0, stream>>>(
            (bf16*)qkv, T, nh, nkv, q_w, k_w, eps, positions, rope_table, (bf16*)k_cache, (bf16*)v_cache,
            slots, page_size, first_head);
        LC_LAUNCH_CHECK("qk_norm_rope_write128");
        return 0;
    }
    const int waves = 4;
    dim3 grid(T, (nh + 2 * nkv - first_head + waves - 1) / waves);
    if (dt == DT_F32)
        qk_norm_rope_write_kernel<float><<<grid, waves * kWave, 0, stream>>>(
            (float*)qkv, T, nh, nkv, d, q_w, k_w, eps, positions, rope_table, rot,
            (float*)k_cache, (float*)v_cache, slots, page_size, first_head);
    else if (dt == DT_BF16)
        qk_norm_rope_write_kernel<bf16><<<grid, waves * kWave, 0, stream>>>(
            (bf16*)qkv, T, nh, nkv, d, q_w, k_w, eps, positions, rope_table, rot,
            (bf16*)k_cache, (bf16*)v_cache, slots, page_size, first_head);
    else
        LC_CHECK(false, "qk_norm_rope_write: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("qk_norm_rope_write");
    return 0;
}

LC_API int lc_swiglu(const void* gu, void* out, int dt, int T, int I, hipStream_t stream) {
    LC_CHECK(T >= 0 && I > 0, "swiglu: bad sizes T=%d I=%d", T, I);
    if (T == 0) return 0;
    LC_CHECK(gu && out, "swiglu: null pointer");
    const size_t total = (size_t)T * I;
    const int threads = 256;
    size_t blocks = (total + threads - 1) / threads;
    if (blocks > 65536) blocks = 65536;
    if (dt == DT_F32)
        swiglu_kernel<float><<<(int)blocks, threads, 0, stream>>>((const float*)gu, (float*)out, I, total);
    else if (dt == DT_BF16)
        swiglu_kernel<bf16><<<(int)blocks, threads, 0, stream>>>((const bf16*)gu, (bf16*)out, I, total);
    else
        LC_CHECK(false, "swiglu: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("swiglu");
    return 0;
}
