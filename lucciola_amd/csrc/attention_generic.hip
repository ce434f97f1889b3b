// Attention over the paged cache for any batch, head size and page size, computed with
// float32 arithmetic throughout (scores, max, exp, sum, P.V).  One workgroup per token and up to
// four query heads of one kv head, which share every key and value they load.
//
// Formulas (reference: plain form src/kernels/attention.cu:51-67,84-107,129-144; paged decode
// src/kernels/attention_paged.cu:68-140):
//   kv head = h / (nh / nkv);   s_j = (q . k_j) / sqrt(d) for keys j <= p (the query's
//   absolute position), and, with a window w > 0, j > p - w;   P = softmax(s);  o = sum P_j v_j.
// Unlike the reference's decode kernel (which stops at 1024 keys,
// src/kernels/attention_paged.cu:80-81) the key loop streams chunks of 256 keys with a running
// maximum and sum, so any context length works.
//
// The order of the additions is a function of the query alone (its position and window): the
// keys are cut at multiples of 512 into spans; a span's maximum, sum and P.V are made on their
// own from its first key on, and the spans are taken into the total one after the other from
// the first.  With few tokens the spans are shared out over workgroups that leave their sums
// in a workspace, and a second kernel takes them in, in the same order and with the same
// operations: a query's result has the same bits whether it is computed alone or in a prompt.
//
// Cache layouts: keys [pages, nkv, page_size, d], values [pages, nkv, d, page_size].  The key
// and value at position j of request r live in page block_table[r][j / page_size], slot
// j % page_size.
#include "common.h"

namespace lc {

constexpr int AG_THREADS = 256;
constexpr int AG_WAVES = AG_THREADS / kWave;
constexpr int AG_SPAN = 512;              // keys whose sums are made on their own
constexpr int AG_HEADS = 4;               // query heads a workgroup serves together
constexpr int AG_PART = AG_THREADS + 2;   // floats a span leaves per head: every thread's sum, m, l

// The running (M, L, ACC) takes in a span's (m, l, acc).  Written with explicit operations so
// that both kernels that use it round alike.
__device__ __forceinline__ void take_in(float& M, float& L, float& ACC, float m, float l, float acc) {
    const float m_new = fmaxf(M, m);
    const float a = expf(M - m_new), b = expf(m - m_new);   // a = 0 for the first span (M = -inf)
    L = fmaf(L, a, __fmul_rn(l, b));
    ACC = fmaf(ACC, a, __fmul_rn(acc, b));
    M = m_new;
}

// out[di] = (the key groups' sums of dim di, added from group 0 on) / L
template <typename T>
__device__ __forceinline__ void finish(float ACC, float L, float* ps, T* out_row, int d, int d_pow2) {
    const int tid = threadIdx.x, g = tid / d_pow2, di = tid % d_pow2;
    __syncthreads();
    ps[tid] = di < d ? ACC : 0.f;
    __syncthreads();
    if (g == 0 && di < d) {
        float total = 0.f;
        for (int gg = 0; gg < AG_THREADS / d_pow2; ++gg) total = __fadd_rn(total, ps[gg * d_pow2 + di]);
        out_row[di] = from_f32<T>(total / L);
    }
}

template <int GH, bool MAX>
__device__ __forceinline__ void block_reduce(float (&v)[GH], float (*scratch)[AG_WAVES]) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
    for (int i = 0; i < GH; ++i) v[i] = MAX ? wave_max(v[i]) : wave_sum(v[i]);
    __syncthreads();  // scratch may still be read from an earlier call
    if (lane == 0)
#pragma unroll
        for (int i = 0; i < GH; ++i) scratch[i][wave] = v[i];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < GH; ++i) {
        float total = scratch[i][0];
        for (int w = 1; w < AG_WAVES; ++w)
            total = MAX ? fmaxf(total, scratch[i][w]) : __fadd_rn(total, scratch[i][w]);
        v[i] = total;
    }
}

// part == nullptr: a workgroup works through all spans of its token and writes the result.
// Else blockIdx.z is the span (counted from the query's first) and its sums go to
// part[token][head][span][AG_PART].
template <typename T, int GH>
__global__ __launch_bounds__(AG_THREADS) void attention_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, T* __restrict__ out, const int* __restrict__ tok_req,
    const int* __restrict__ positions, const int* __restrict__ block_table, int max_blocks,
    int nh, int nkv, int d, int d_pow2, int page_size, float scale, int window,
    float* __restrict__ part, int part_spans) {
    __shared__ __align__(16) float qs[GH][256];
    __shared__ __align__(16) float ps[GH][AG_THREADS];
    __shared__ float scratch[GH][AG_WAVES];
    __shared__ int pages[AG_THREADS + 1];      // the chunk's pages, looked up once a chunk

    const int t = blockIdx.x, tid = threadIdx.x;
    const int group = nh / nkv, batches = (group + GH - 1) / GH;
    const int kvh = blockIdx.y / batches;
    const int h0 = kvh * group + (blockIdx.y % batches) * GH;
    const int heads = min(GH, (kvh + 1) * group - h0);
    const int r = tok_req[t];
    const int p = positions[t];
    const int* table = block_table + (size_t)r * max_blocks;
    const int j_lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int s_first = j_lo / AG_SPAN, s_last = p / AG_SPAN;
    int s_begin = s_first, s_end = s_last;
    if (part) {
        s_begin = s_end = s_first + blockIdx.z;
        if (s_begin > s_last) return;
    }
    for (int i = tid; i < GH * 256; i += AG_THREADS) {
        const int hh = i >> 8, e = i & 255;
        qs[hh][e] = (hh < heads && e < d) ? to_f32(q[(size_t)t * q_stride + (size_t)(h0 + hh) * d + e]) * scale : 0.f;
    }
    __syncthreads();

    const int groups = AG_THREADS / d_pow2;     // key groups that share the P.V work
    const int g = tid / d_pow2, di = tid % d_pow2;
    const bool pv_active = di < d;
    // Whole 16-byte (8-byte) pieces where the sizes allow it: four lanes share a key's row for
    // the scores (a wave then reads 16 rows as one contiguous stretch), and a lane takes four
    // neighbouring keys of its dim at a time for the values (they lie side by side in a page).
    const bool vec = (d & 15) == 0 && (page_size & 3) == 0;

    float M[GH], L[GH], ACC[GH];
#pragma unroll
    for (int hh = 0; hh < GH; ++hh) { M[hh] = -INFINITY; L[hh] = 0.f; ACC[hh] = 0.f; }

    for (int s = s_begin; s <= s_end; ++s) {
        const int lo = max(s * AG_SPAN, j_lo), hi = min(s * AG_SPAN + AG_SPAN - 1, p);
        float m[GH], l[GH], acc[GH];
#pragma unroll
        for (int hh = 0; hh < GH; ++hh) { m[hh] = -INFINITY; l[hh] = 0.f; acc[hh] = 0.f; }
        for (int c0 = lo; c0 <= hi; c0 += AG_THREADS) {
            const int count = min(AG_THREADS, hi - c0 + 1);
            const bool valid = tid < count;
            float sc[GH];
            // the numbers of the chunk's pages go to LDS first: one trip to the block table a
            // chunk instead of one before every key's and value's own load
            const int page0 = c0 / page_size, page_n = (c0 + count - 1) / page_size - page0 + 1;
            for (int i = tid; i < page_n; i += AG_THREADS) pages[i] = table[page0 + i];
            __syncthreads();
            if (vec) {
                const int piece = tid & 3;
                for (int pass = 0; pass < 4; ++pass) {
                    const int kc = pass * (AG_THREADS / 4) + (tid >> 2);
                    float dot[GH];
#pragma unroll
                    for (int hh = 0; hh < GH; ++hh) dot[hh] = 0.f;
                    if (kc < count) {
                        const int jk = c0 + kc;
                        const long long head = (long long)pages[jk / page_size - page0] * nkv + kvh;
                        // the four lanes of a key take its pieces of four entries in turn (lane
                        // `piece` the pieces piece, piece + 4, ...): one load instruction then reads
                        // 64 bytes in a row of each of a wave's 16 keys; four loads are asked for
                        // before the first is used
                        const T* krow = k_cache + (head * page_size + (jk % page_size)) * d + piece * 4;
                        for (int i0 = 0; i0 < d; i0 += 64) {
                            float k4[4][4];
#pragma unroll
                            for (int u = 0; u < 4; ++u)
                                if (i0 + 16 * u < d) load4(k4[u], krow + i0 + 16 * u);
#pragma unroll
                            for (int u = 0; u < 4; ++u)
                                if (i0 + 16 * u < d)
#pragma unroll
                                    for (int hh = 0; hh < GH; ++hh)
#pragma unroll
                                        for (int e = 0; e < 4; ++e)
                                            dot[hh] = fmaf(qs[hh][piece * 4 + i0 + 16 * u + e], k4[u][e], dot[hh]);
                        }
                    }
#pragma unroll
                    for (int hh = 0; hh < GH; ++hh) {   // the row's four quarters, in a fixed order
                        dot[hh] = __fadd_rn(dot[hh], __shfl_xor(dot[hh], 1, kWave));
                        dot[hh] = __fadd_rn(dot[hh], __shfl_xor(dot[hh], 2, kWave));
                        if (piece == 0) ps[hh][kc] = dot[hh];
                    }
                }
                __syncthreads();
#pragma unroll
                for (int hh = 0; hh < GH; ++hh) sc[hh] = valid ? ps[hh][tid] : -INFINITY;
                __syncthreads();                            // ps is written again below
            } else {
#pragma unroll
                for (int hh = 0; hh < GH; ++hh) sc[hh] = 0.f;
                if (valid) {
                    const int j = c0 + tid;
                    const long long head = (long long)pages[j / page_size - page0] * nkv + kvh;
                    const T* krow = k_cache + (head * page_size + (j % page_size)) * d;
                    for (int i = 0; i < d; ++i) {
                        const float kv = to_f32(krow[i]);
#pragma unroll
                        for (int hh = 0; hh < GH; ++hh) sc[hh] = fmaf(qs[hh][i], kv, sc[hh]);
                    }
                } else {
#pragma unroll
                    for (int hh = 0; hh < GH; ++hh) sc[hh] = -INFINITY;
                }
            }
            float red[GH], alpha[GH];
#pragma unroll
            for (int hh = 0; hh < GH; ++hh) red[hh] = sc[hh];
            block_reduce<GH, true>(red, scratch);
#pragma unroll
            for (int hh = 0; hh < GH; ++hh) {
                const float m_new = fmaxf(m[hh], red[hh]);
                const float pj = valid ? expf(sc[hh] - m_new) : 0.f;
                alpha[hh] = expf(m[hh] - m_new);  // 0 on a span's first chunk (m = -inf)
                m[hh] = m_new;
                ps[hh][tid] = pj;
                red[hh] = pj;
            }
            block_reduce<GH, false>(red, scratch);  // has the barriers that publish ps
#pragma unroll
            for (int hh = 0; hh < GH; ++hh) {
                l[hh] = fmaf(l[hh], alpha[hh], red[hh]);
                acc[hh] = __fmul_rn(acc[hh], alpha[hh]);
            }
            if (pv_active) {
                if (vec) {
                    // runs of four keys that start at a multiple of four lie in one page; a run
                    // may reach over the chunk's ends, where the keys count nothing
                    // (four runs are asked for before the first is used; they are taken in in
                    // their order)
                    const int last_run = (c0 + count - 1) >> 2;
                    for (int run0 = (c0 >> 2) + g; run0 <= last_run; run0 += 4 * groups) {
                        float v4[4][4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int j4 = (run0 + u * groups) * 4;
                            if (run0 + u * groups <= last_run) {
                                // a run may begin before the chunk's first key, in the page before its first
                                const int pg = j4 >= c0 ? pages[j4 / page_size - page0] : table[j4 / page_size];
                                const long long head = (long long)pg * nkv + kvh;
                                load4(v4[u], v_cache + head * d * page_size + (long long)di * page_size + (j4 % page_size));
                            }
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int j4 = (run0 + u * groups) * 4;
                            if (run0 + u * groups <= last_run) {
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    const int jj = j4 + e - c0;
                                    if (jj >= 0 && jj < count)
#pragma unroll
                                        for (int hh = 0; hh < GH; ++hh) acc[hh] = fmaf(ps[hh][jj], v4[u][e], acc[hh]);
                                }
                            }
                        }
                    }
                } else {
                    for (int jj = g; jj < count; jj += groups) {
                        const int j = c0 + jj;
                        const long long head = (long long)pages[j / page_size - page0] * nkv + kvh;
                        const float v = to_f32(v_cache[head * d * page_size + (long long)di * page_size + (j % page_size)]);
#pragma unroll
                        for (int hh = 0; hh < GH; ++hh) acc[hh] = fmaf(ps[hh][jj], v, acc[hh]);
                    }
                }
            }
            __syncthreads();  // ps is rewritten by the next chunk
        }
        if (part) {
            for (int hh = 0; hh < heads; ++hh) {
                float* mine = part + (((size_t)t * nh + h0 + hh) * part_spans + blockIdx.z) * AG_PART;
                mine[tid] = pv_active ? acc[hh] : 0.f;
                if (tid == 0) { mine[AG_THREADS] = m[hh]; mine[AG_THREADS + 1] = l[hh]; }
            }
            return;
        }
#pragma unroll
        for (int hh = 0; hh < GH; ++hh) take_in(M[hh], L[hh], ACC[hh], m[hh], l[hh], acc[hh]);
    }
#pragma unroll
    for (int hh = 0; hh < GH; ++hh)
        if (hh < heads) finish<T>(ACC[hh], L[hh], ps[0], out + ((size_t)t * nh + h0 + hh) * d, d, d_pow2);
}

// One workgroup per (token, head): the spans' sums from the workspace, taken in from the first.
template <typename T>
__global__ __launch_bounds__(AG_THREADS) void attention_generic_join_kernel(
    const float* __restrict__ part, int part_spans, T* __restrict__ out,
    const int* __restrict__ positions, int nh, int d, int d_pow2, int window) {
    __shared__ float ps[AG_THREADS];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int p = positions[t];
    const int j_lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int spans = p / AG_SPAN - j_lo / AG_SPAN + 1;
    float M = -INFINITY, L = 0.f, ACC = 0.f;
    for (int z = 0; z < spans; ++z) {
        const float* its = part + (((size_t)t * nh + h) * part_spans + z) * AG_PART;
        take_in(M, L, ACC, its[AG_THREADS], its[AG_THREADS + 1], its[tid]);
    }
    finish<T>(ACC, L, ps, out + ((size_t)t * nh + h) * d, d, d_pow2);
}

// Spans a launch is cut into (0: it is not): when the workgroups would not fill the card and
// the block table is wide enough for more than one span.
static int shared_spans(int T, int nh, int nkv, int max_blocks, int page_size) {
    const int group = nh / nkv;
    const long long workgroups = (long long)T * nkv * ((group + AG_HEADS - 1) / AG_HEADS);
    const long long keys = (long long)max_blocks * page_size;
    if (workgroups >= 1024 || keys <= AG_SPAN) return 0;
    const long long spans = (keys + AG_SPAN - 1) / AG_SPAN;
    if ((long long)T * nh * spans * AG_PART > (64ll << 20)) return 0;   // 256 MiB of float32
    return (int)spans;
}

template <typename T>
static void launch_attention_generic(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                     void* out, const int* tok_req, const int* positions,
                                     const int* block_table, int max_blocks, int T_, int nh, int nkv, int d,
                                     int page_size, float scale, int window, float* workspace, int spans,
                                     hipStream_t stream) {
    int d_pow2 = 1;
    while (d_pow2 < d) d_pow2 <<= 1;
    const int group = nh / nkv;
    dim3 grid(T_, nkv * ((group + AG_HEADS - 1) / AG_HEADS), spans > 0 ? spans : 1);
    attention_generic_kernel<T, AG_HEADS><<<grid, AG_THREADS, 0, stream>>>(
        (const T*)q, q_stride, (const T*)k_cache, (const T*)v_cache, (T*)out, tok_req, positions,
        block_table, max_blocks, nh, nkv, d, d_pow2, page_size, scale, window,
        spans > 0 ? workspace : nullptr, spans);
    if (spans > 0)
        attention_generic_join_kernel<T><<<dim3(T_, nh), AG_THREADS, 0, stream>>>(
            workspace, spans, (T*)out, positions, nh, d, d_pow2, window);
}

}  // namespace lc

using namespace lc;

// float32 words of workspace that lc_attention_generic needs for these sizes (0: none)
LC_API long long lc_attention_generic_workspace(int T, int nh, int nkv, int max_blocks, int page_size) {
    if (T <= 0 || nh <= 0 || nkv <= 0 || nh % nkv || max_blocks <= 0 || page_size <= 0) return 0;
    return (long long)T * nh * shared_spans(T, nh, nkv, max_blocks, page_size) * AG_PART;
}

LC_API int lc_attention_generic(const void* q, int q_stride, const void* k_cache,
                                const void* v_cache, void* out, int dt, const int* tok_req,
                                const int* positions, const int* block_table, int max_blocks,
                                int T, int nh, int nkv, int d, int page_size, float scale,
                                int window, float* workspace, hipStream_t stream) {
    LC_CHECK(T >= 0 && nh > 0 && nkv > 0 && d > 0 && page_size > 0 && max_blocks > 0,
             "attention: bad sizes T=%d nh=%d nkv=%d d=%d page=%d blocks=%d", T, nh, nkv, d, page_size,
             max_blocks);
    if (T == 0) return 0;
    LC_CHECK(nh % nkv == 0, "attention: %d query heads are not a multiple of %d kv heads", nh, nkv);
    LC_CHECK(d <= 256, "attention: head size %d is above the supported 256", d);
    LC_CHECK(nh <= 65535, "attention: too many heads (%d)", nh);
    LC_CHECK(q && k_cache && v_cache && out && tok_req && positions && block_table,
             "attention: null pointer");
    const int spans = shared_spans(T, nh, nkv, max_blocks, page_size);
    LC_CHECK(spans == 0 || workspace, "attention: T=%d with %d blocks needs a workspace", T, max_blocks);
    LC_CHECK(spans <= 65535, "attention: too many spans (%d)", spans);
    if (dt == DT_F32)
        launch_attention_generic<float>(q, q_stride, k_cache, v_cache, out, tok_req, positions, block_table,
                                        max_blocks, T, nh, nkv, d, page_size, scale, window, workspace, spans,
                                        stream);
    else if (dt == DT_BF16)
        launch_attention_generic<bf16>(q, q_stride, k_cache, v_cache, out, tok_req, positions, block_table,
                                       max_blocks, T, nh, nkv, d, page_size, scale, window, workspace, spans,
                                       stream);
    else
        LC_CHECK(false, "attention: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("attention_generic");
    return 0;
}
