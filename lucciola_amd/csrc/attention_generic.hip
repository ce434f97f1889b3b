// Attention over the paged cache for any batch, head size and page size, computed with
// float32 arithmetic throughout (scores, max, exp, sum, P.V).  One workgroup per (token, head).
//
// Formulas (reference: plain form src/kernels/attention.cu:51-67,84-107,129-144; paged decode
// src/kernels/attention_paged.cu:68-140):
//   kv head = h / (nh / nkv);   s_j = (q . k_j) / sqrt(d) for keys j <= p (the query's
//   absolute position), and, with a window w > 0, j > p - w;   P = softmax(s);  o = sum P_j v_j.
// Unlike the reference's decode kernel (which stops at 1024 keys,
// src/kernels/attention_paged.cu:80-81) the key loop streams chunks of 256 keys with a running
// maximum and sum, so any context length works.
//
// Cache layouts: keys [pages, nkv, page_size, d], values [pages, nkv, d, page_size].  The key
// and value at position j of request r live in page block_table[r][j / page_size], slot
// j % page_size.
#include "common.h"

namespace lc {

constexpr int AG_THREADS = 256;

template <typename T>
__global__ __launch_bounds__(AG_THREADS) void attention_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, T* __restrict__ out, const int* __restrict__ tok_req,
    const int* __restrict__ positions, const int* __restrict__ block_table, int max_blocks,
    int nh, int nkv, int d, int d_pow2, int page_size, float scale, int window) {
    __shared__ float qs[256];
    __shared__ float ps[AG_THREADS];
    __shared__ long long voff[AG_THREADS];
    __shared__ float scratch[16];

    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int r = tok_req[t];
    const int p = positions[t];
    const int kvh = h / (nh / nkv);
    const int* table = block_table + (size_t)r * max_blocks;
    const T* qrow = q + (size_t)t * q_stride + (size_t)h * d;
    for (int i = tid; i < d; i += AG_THREADS) qs[i] = to_f32(qrow[i]) * scale;
    __syncthreads();

    const int j_lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int groups = AG_THREADS / d_pow2;     // key groups that share the P.V work
    const int g = tid / d_pow2, di = tid % d_pow2;
    const bool pv_active = di < d;

    // Whole 16-byte (8-byte) pieces where the sizes allow it: four lanes share a key's row for
    // the scores (a wave then reads 16 rows as one contiguous stretch), and a lane takes four
    // neighbouring keys of its dim at a time for the values (they lie side by side in a page).
    const bool vec = (d & 15) == 0 && (page_size & 3) == 0;
    float m = -INFINITY, l = 0.f, acc = 0.f;
    for (int c0 = j_lo; c0 <= p; c0 += AG_THREADS) {
        const int j = c0 + tid;
        const bool valid = j <= p;
        float s = -INFINITY;
        long long off = 0;
        if (vec) {
            const int part = tid & 3, quarter = d >> 2;
#pragma unroll 1
            for (int pass = 0; pass < 4; ++pass) {
                const int kc = pass * (AG_THREADS / 4) + (tid >> 2), jk = c0 + kc;
                float dot = 0.f;
                if (jk <= p) {
                    const long long head = (long long)table[jk / page_size] * nkv + kvh;
                    const T* krow = k_cache + (head * page_size + (jk % page_size)) * d + part * quarter;
                    const float* qp = qs + part * quarter;
                    for (int i = 0; i < quarter; i += 4) {
                        float k4[4];
                        load4(k4, krow + i);
#pragma unroll
                        for (int e = 0; e < 4; ++e) dot = fmaf(qp[i + e], k4[e], dot);
                    }
                }
                dot += __shfl_xor(dot, 1, kWave);      // the row's four quarters, in a fixed order
                dot += __shfl_xor(dot, 2, kWave);
                if (part == 0) ps[kc] = dot;
            }
            __syncthreads();
            if (valid) s = ps[tid];
            __syncthreads();                            // ps is written again below
        } else if (valid) {
            const int page = table[j / page_size];
            const long long head = (long long)page * nkv + kvh;
            off = head * d * page_size + (j % page_size);          // of the value column
            const T* krow = k_cache + (head * page_size + (j % page_size)) * d;
            float dot = 0.f;
            for (int i = 0; i < d; ++i) dot = fmaf(qs[i], to_f32(krow[i]), dot);
            s = dot;
        }
        const float cmax = block_max(s, scratch);
        const float m_new = fmaxf(m, cmax);
        const float pj = valid ? expf(s - m_new) : 0.f;
        const float alpha = expf(m - m_new);  // 0 on the first chunk (m = -inf)
        ps[tid] = pj;
        voff[tid] = off;
        const float psum = block_sum(pj, scratch);  // has the barriers that publish ps/voff
        l = l * alpha + psum;
        m = m_new;
        acc *= alpha;
        if (pv_active) {
            const int count = min(AG_THREADS, p - c0 + 1);
            if (vec) {
                // runs of four keys that start at a multiple of four lie in one page; a run may
                // reach over the chunk's ends, where the keys count nothing
                const int first_run = c0 >> 2, last_run = (c0 + count - 1) >> 2;
                for (int run = first_run + g; run <= last_run; run += groups) {
                    const int j4 = run * 4;
                    const long long head = (long long)table[j4 / page_size] * nkv + kvh;
                    float v4[4];
                    load4(v4, v_cache + head * d * page_size + (long long)di * page_size + (j4 % page_size));
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int jj = j4 + e - c0;
                        if (jj >= 0 && jj < count) acc = fmaf(ps[jj], v4[e], acc);
                    }
                }
            } else {
                for (int jj = g; jj < count; jj += groups)
                    acc = fmaf(ps[jj], to_f32(v_cache[voff[jj] + (long long)di * page_size]), acc);
            }
        }
        __syncthreads();  // ps/voff are rewritten by the next chunk
    }
    // add the key groups' partial sums
    ps[tid] = pv_active ? acc : 0.f;
    __syncthreads();
    if (g == 0 && pv_active) {
        float total = 0.f;
        for (int gg = 0; gg < groups; ++gg) total += ps[gg * d_pow2 + di];
        out[((size_t)t * nh + h) * d + di] = from_f32<T>(total / l);
    }
}

}  // namespace lc

using namespace lc;

LC_API int lc_attention_generic(const void* q, int q_stride, const void* k_cache,
                                const void* v_cache, void* out, int dt, const int* tok_req,
                                const int* positions, const int* block_table, int max_blocks,
                                int T, int nh, int nkv, int d, int page_size, float scale,
                                int window, hipStream_t stream) {
    LC_CHECK(T >= 0 && nh > 0 && nkv > 0 && d > 0 && page_size > 0,
             "attention: bad sizes T=%d nh=%d nkv=%d d=%d page=%d", T, nh, nkv, d, page_size);
    if (T == 0) return 0;
    LC_CHECK(nh % nkv == 0, "attention: %d query heads are not a multiple of %d kv heads", nh, nkv);
    LC_CHECK(d <= 256, "attention: head size %d is above the supported 256", d);
    LC_CHECK(nh <= 65535, "attention: too many heads (%d)", nh);
    LC_CHECK(q && k_cache && v_cache && out && tok_req && positions && block_table,
             "attention: null pointer");
    int d_pow2 = 1;
    while (d_pow2 < d) d_pow2 <<= 1;
    dim3 grid(T, nh);
    if (dt == DT_F32)
        attention_generic_kernel<float><<<grid, AG_THREADS, 0, stream>>>(
            (const float*)q, q_stride, (const float*)k_cache, (const float*)v_cache, (float*)out,
            tok_req, positions, block_table, max_blocks, nh, nkv, d, d_pow2, page_size, scale, window);
    else if (dt == DT_BF16)
        attention_generic_kernel<bf16><<<grid, AG_THREADS, 0, stream>>>(
            (const bf16*)q, q_stride, (const bf16*)k_cache, (const bf16*)v_cache, (bf16*)out,
            tok_req, positions, block_table, max_blocks, nh, nkv, d, d_pow2, page_size, scale, window);
    else
        LC_CHECK(false, "attention: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("attention_generic");
    return 0;
}
