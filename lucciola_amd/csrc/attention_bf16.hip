// bfloat16 attention over the paged cache on the matrix cores, for pages of 16 tokens:
//   * decode: one query token per request; a workgroup owns (request, kv head, a share of the
//     pages), its 4 waves take pages in turn and meet in LDS; with several shares per request
//     the partial results (max, sum, unnormalised output) go to a workspace and a second
//     kernel joins them.  The query heads that share a kv head form the columns of one
//     matrix-core tile, so keys and values are read once per group.
//   * prefill: a workgroup owns 64 query rows of one request and one head; each wave 16 rows.
//
// Both run the same inner step on one page of 16 keys, written for the operand layouts of
// the matrix instructions:
//   S^T[key, q]  = K[key, :] . Q[q, :]       v_mfma_f32_16x16x32_bf16, A = K rows (as they lie
//                                            in the page), B = Q^T; the result leaves each
//                                            lane with 4 consecutive keys of one query column
//   P^T          = exp2(S^T * scale*log2(e) - max)   per query column, float32
//   O^T[dim, q] += V^T[dim, key] . P^T[key, q]       v_mfma_f32_16x16x16bf16_1k, A = V^T rows
//                                            (values are stored transposed inside a page,
//                                            [d][16]), B = P^T exactly as the lanes hold it.
// Scores, maxima, exponentials and sums are float32; P is rounded to bfloat16 for the second
// product.  Masking: a query at position p sees keys j <= p, and with a window w, j > p - w.
//
// Reference kernels: src/kernels/attention_paged.cu:47-141 (decode; stops at 1024 keys) and
// src/kernels/flash_attention.cu:36-349 (prefill; page 16 and head size <= 128 fixed at compile
// time).
#include "common.h"

namespace lc {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int PAGE = 16;

template <int D>
struct AttnState {
    float m, l;              // running maximum (log2 domain) and this lane's share of the sum
    floatx4 o[D / 16];       // O^T tiles: o[t][v] = O[dim = 16 t + 4 (lane/16) + v][q = lane%16]
};

template <int D>
struct PageRegs {
    bf16x8 k[D / 32];
    short4v v[D / 16];
};

template <int D>
__device__ __forceinline__ void load_page(PageRegs<D>& r, const bf16* __restrict__ k_cache,
                                          const bf16* __restrict__ v_cache, int page, int nkv,
                                          int kvh, int lane) {
    const size_t head = (size_t)page * nkv + kvh;
    const bf16* kb = k_cache + (head * PAGE + (lane & 15)) * D + (lane >> 4) * 8;
    const bf16* vb = v_cache + (head * D + (lane & 15)) * PAGE + (lane >> 4) * 4;
#pragma unroll
    for (int i = 0; i < D / 32; ++i) r.k[i] = *reinterpret_cast<const bf16x8*>(kb + i * 32);
#pragma unroll
    for (int i = 0; i < D / 16; ++i) r.v[i] = *reinterpret_cast<const short4v*>(vb + i * 16 * PAGE);
}

__device__ __forceinline__ short bf16_bits(float f) {
    const bf16 b = static_cast<bf16>(f);
    return *reinterpret_cast<const short*>(&b);
}

// One page of 16 keys starting at position `key0`.  lo/hi: the lowest and highest position
// this lane's query column may see.
template <int D>
__device__ __forceinline__ void attend_page(AttnState<D>& st, const PageRegs<D>& r,
                                            const bf16x8 (&bq)[D / 32], int key0, int lo, int hi,
                                            float scale_log2, int lane) {
    floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < D / 32; ++i)
        s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(r.k[i], bq[i], s, 0, 0, 0);
    const int j0 = key0 + (lane >> 4) * 4;
    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int j = j0 + v;
        s[v] = (j >= lo && j <= hi) ? s[v] * scale_log2 : -INFINITY;
        mx = fmaxf(mx, s[v]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(st.m, mx);
    const float alpha = (st.m == -INFINITY) ? 0.f : exp2f(st.m - m_new);
    float p[4], psum = 0.f;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        p[v] = (s[v] == -INFINITY) ? 0.f : exp2f(s[v] - m_new);
        psum += p[v];
    }
    st.l = st.l * alpha + psum;
    st.m = m_new;
    short4v pb;
#pragma unroll
    for (int v = 0; v < 4; ++v) pb[v] = bf16_bits(p[v]);
#pragma unroll
    for (int t = 0; t < D / 16; ++t) {
        st.o[t] *= alpha;
        st.o[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(r.v[t], pb, st.o[t], 0, 0, 0);
    }
}

template <int D>
__device__ __forceinline__ void init_state(AttnState<D>& st) {
    st.m = -INFINITY;
    st.l = 0.f;
#pragma unroll
    for (int t = 0; t < D / 16; ++t) st.o[t] = floatx4{0.f, 0.f, 0.f, 0.f};
}

// Walk pages [begin, end) with stride `step`, the next page's loads in flight while the
// current one is multiplied.
template <int D>
__device__ __forceinline__ void attend_range(AttnState<D>& st, const bf16x8 (&bq)[D / 32],
                                             const bf16* __restrict__ k_cache,
                                             const bf16* __restrict__ v_cache,
                                             const int* __restrict__ table, int begin, int end,
                                             int step, int nkv, int kvh, int lo, int hi,
                                             float scale_log2, int lane) {
    if (begin >= end) return;
    PageRegs<D> cur, nxt;
    load_page<D>(cur, k_cache, v_cache, table[begin], nkv, kvh, lane);
    int next_page = (begin + step < end) ? table[begin + step] : 0;
    for (int pg = begin; pg < end; pg += step) {
        const bool more = pg + step < end;
        if (more) {
            load_page<D>(nxt, k_cache, v_cache, next_page, nkv, kvh, lane);
            if (pg + 2 * step < end) next_page = table[pg + 2 * step];
        }
        attend_page<D>(st, cur, bq, pg * PAGE, lo, hi, scale_log2, lane);
        if (more) cur = nxt;
    }
}

// ------------------------------------------------------------------------------- decode
template <int D>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    const bf16* __restrict__ qkv, int q_stride, const bf16* __restrict__ k_cache,
    const bf16* __restrict__ v_cache, bf16* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, const int* __restrict__ decode_tokens,
    const int* __restrict__ tok_req, const int* __restrict__ positions,
    const int* __restrict__ block_table, int max_blocks, int nh, int nkv, float scale_log2,
    int window, int splits) {
    __shared__ float sm_o[4][D * 16];
    __shared__ float sm_m[4][16], sm_l[4][16];

    const int split = blockIdx.x, kvh = blockIdx.y, di = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int q = lane & 15, kg = lane >> 4;
    const int t = decode_tokens[di];
    const int req = tok_req[t], p = positions[t];
    const int G = nh / nkv;
    const int j_lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int first_page = j_lo / PAGE, last_page = p / PAGE;
    const int per = (last_page - first_page + splits) / splits;   // ceil(pages / splits)
    const int begin = first_page + split * per;
    const int end = min(begin + per, last_page + 1);
    const int* table = block_table + (size_t)req * max_blocks;

    bf16x8 bq[D / 32];
    {
        const bf16* qrow = qkv + (size_t)t * q_stride + (size_t)(kvh * G + min(q, G - 1)) * D + kg * 8;
#pragma unroll
        for (int i = 0; i < D / 32; ++i) bq[i] = *reinterpret_cast<const bf16x8*>(qrow + i * 32);
    }
    AttnState<D> st;
    init_state<D>(st);
    attend_range<D>(st, bq, k_cache, v_cache, table, begin + wave, end, 4, nkv, kvh, j_lo, p,
                    scale_log2, lane);

    // the waves' results meet in LDS
    float l = st.l;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (kg == 0) { sm_m[wave][q] = st.m; sm_l[wave][q] = l; }
#pragma unroll
    for (int tt = 0; tt < D / 16; ++tt)
#pragma unroll
        for (int v = 0; v < 4; ++v) sm_o[wave][(tt * 16 + kg * 4 + v) * 16 + q] = st.o[tt][v];
    __syncthreads();
    for (int idx = threadIdx.x; idx < D * 16; idx += 256) {
        const int dim = idx >> 4, qq = idx & 15;
        if (qq >= G) continue;
        float m_all = fmaxf(fmaxf(sm_m[0][qq], sm_m[1][qq]), fmaxf(sm_m[2][qq], sm_m[3][qq]));
        float o = 0.f, lsum = 0.f;
        if (m_all != -INFINITY) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float f = (sm_m[w][qq] == -INFINITY) ? 0.f : exp2f(sm_m[w][qq] - m_all);
                o += f * sm_o[w][idx];
                lsum += f * sm_l[w][qq];
            }
        }
        const int h = kvh * G + qq;
        if (splits == 1) {
            out[((size_t)t * nh + h) * D + dim] = static_cast<bf16>(o / lsum);
        } else {
            const size_t slot = ((size_t)di * nh + h) * splits + split;
            part_o[slot * D + dim] = o;
            if (dim == 0) { part_ml[slot * 2] = m_all; part_ml[slot * 2 + 1] = lsum; }
        }
    }
}

// Joins the shares of a request's pages: out = sum_s o_s 2^(m_s - m) / sum_s l_s 2^(m_s - m).
// The factors are worked out once (one thread per share) and left in LDS, so that the sum over
// the shares is a run of independent loads.
template <int D>
__global__ __launch_bounds__(128) void attn_decode_join_kernel(const float* __restrict__ part_o,
                                                               const float* __restrict__ part_ml,
                                                               const int* __restrict__ decode_tokens,
                                                               bf16* __restrict__ out, int nh,
                                                               int splits) {
    __shared__ float f[64];
    __shared__ float inv_l;
    const int di = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int t = decode_tokens[di];
    const size_t base = ((size_t)di * nh + h) * splits;
    if (tid < 64) {
        const float ms = tid < splits ? part_ml[(base + tid) * 2] : -INFINITY;
        const float ls = tid < splits ? part_ml[(base + tid) * 2 + 1] : 0.f;
        const float m = wave_max(ms);
        const float fs = (ms == -INFINITY) ? 0.f : exp2f(ms - m);
        f[tid] = fs;
        const float l = wave_sum(fs * ls);
        if (tid == 0) inv_l = 1.f / l;
    }
    __syncthreads();
    for (int dim = tid; dim < D; dim += 128) {
        float o = 0.f;
#pragma unroll 8
        for (int s = 0; s < splits; ++s) o += f[s] * part_o[(base + s) * D + dim];
        out[((size_t)t * nh + h) * D + dim] = static_cast<bf16>(o * inv_l);
    }
}

// ------------------------------------------------------------------------------- prefill
// tiles: [NT, 4] = (request, first token row, rows (<= 64), position of the first row)
template <int D>
__global__ __launch_bounds__(256) void attn_prefill_kernel(
    const bf16* __restrict__ qkv, int q_stride, const bf16* __restrict__ k_cache,
    const bf16* __restrict__ v_cache, bf16* __restrict__ out, const int* __restrict__ tiles,
    const int* __restrict__ block_table, int max_blocks, int nh, int nkv, float scale_log2,
    int window) {
    const int* tile = tiles + (size_t)blockIdx.x * 4;
    const int req = tile[0], row0 = tile[1], rows = tile[2], pos0 = tile[3];
    const int h = blockIdx.y, kvh = h / (nh / nkv);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int q = lane & 15, kg = lane >> 4;
    const int wrow = wave * 16;
    if (wrow >= rows) return;
    const int my = wrow + q;                      // this lane's query row inside the tile
    const bool valid = my < rows;
    const int p = pos0 + min(my, rows - 1);
    const int hi = valid ? p : 0x7fffffff;        // idle columns see everything (never stored)
    const int lo = (valid && window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int p_min = pos0 + wrow, p_max = pos0 + min(wrow + 15, rows - 1);
    const int j_lo = (window > 0 && p_min - window + 1 > 0) ? p_min - window + 1 : 0;
    const int* table = block_table + (size_t)req * max_blocks;

    bf16x8 bq[D / 32];
    {
        const bf16* qrow = qkv + (size_t)(row0 + min(my, rows - 1)) * q_stride + (size_t)h * D + kg * 8;
#pragma unroll
        for (int i = 0; i < D / 32; ++i) bq[i] = *reinterpret_cast<const bf16x8*>(qrow + i * 32);
    }
    AttnState<D> st;
    init_state<D>(st);
    attend_range<D>(st, bq, k_cache, v_cache, table, j_lo / PAGE, p_max / PAGE + 1, 1, nkv, kvh, lo,
                    hi, scale_log2, lane);
    float l = st.l;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!valid) return;
    const float inv = 1.f / l;
    bf16* orow = out + ((size_t)(row0 + my) * nh + h) * D + kg * 4;
#pragma unroll
    for (int tt = 0; tt < D / 16; ++tt) {
        short4v packed;
#pragma unroll
        for (int v = 0; v < 4; ++v) packed[v] = bf16_bits(st.o[tt][v] * inv);
        *reinterpret_cast<short4v*>(orow + tt * 16) = packed;
    }
}

template <int D>
static int launch_decode(const bf16* qkv, int q_stride, const bf16* k, const bf16* v, bf16* out,
                         float* part_o, float* part_ml, const int* decode_tokens, const int* tok_req,
                         const int* positions, const int* table, int max_blocks, int ND, int nh,
                         int nkv, float scale_log2, int window, int splits, hipStream_t s) {
    dim3 grid(splits, nkv, ND);
    attn_decode_kernel<D><<<grid, 256, 0, s>>>(qkv, q_stride, k, v, out, part_o, part_ml,
                                               decode_tokens, tok_req, positions, table, max_blocks,
                                               nh, nkv, scale_log2, window, splits);
    LC_LAUNCH_CHECK("attn_decode");
    if (splits > 1) {
        attn_decode_join_kernel<D><<<dim3(ND, nh), 128, 0, s>>>(
            part_o, part_ml, decode_tokens, out, nh, splits);
        LC_LAUNCH_CHECK("attn_decode_join");
    }
    return 0;
}

template <int D>
static int launch_prefill(const bf16* qkv, int q_stride, const bf16* k, const bf16* v, bf16* out,
                          const int* tiles, const int* table, int max_blocks, int NT, int nh,
                          int nkv, float scale_log2, int window, hipStream_t s) {
    attn_prefill_kernel<D><<<dim3(NT, nh), 256, 0, s>>>(qkv, q_stride, k, v, out, tiles, table,
                                                        max_blocks, nh, nkv, scale_log2, window);
    LC_LAUNCH_CHECK("attn_prefill");
    return 0;
}

}  // namespace lc

using namespace lc;

// Head sizes and group sizes the matrix-core kernels take (pages must hold 16 tokens).
LC_API int lc_attn_bf16_supported(int nh, int nkv, int d, int page_size) {
    if (page_size != PAGE || nkv <= 0 || nh % nkv != 0) return 0;
    if (nh / nkv > 16 || nh > 65535 || nkv > 65535) return 0;
    return d == 32 || d == 64 || d == 96 || d == 128;
}

// Into how many shares the decode kernel cuts a request's pages.
LC_API int lc_attn_decode_splits(int num_decode, int nkv, int max_ctx) {
    if (num_decode <= 0) return 1;
    const int pages = (max_ctx + PAGE - 1) / PAGE;
    const long long base = (long long)num_decode * nkv;
    long long splits = (1024 + base - 1) / base;          // aim at ~4 workgroups per CU
    const int most = (pages + 7) / 8;                     // at least 8 pages per workgroup
    if (splits > most) splits = most;
    if (splits > 64) splits = 64;
    if (splits < 1) splits = 1;
    return (int)splits;
}

#define LC_DISPATCH_D(d, CALL)                   \
    switch (d) {                                 \
        case 32: return CALL(32);                \
        case 64: return CALL(64);                \
        case 96: return CALL(96);                \
        case 128: return CALL(128);              \
        default: LC_CHECK(false, "attention_bf16: head size %d has no matrix-core kernel", d); \
    }

LC_API int lc_attn_decode_bf16(const void* qkv, int q_stride, const void* k_cache, const void* v_cache,
                               void* out, float* part_o, float* part_ml, const int* decode_tokens,
                               const int* tok_req, const int* positions, const int* block_table,
                               int max_blocks, int num_decode, int nh, int nkv, int d, int page_size,
                               float scale, int window, int splits, hipStream_t stream) {
    if (num_decode == 0) return 0;
    LC_CHECK(lc_attn_bf16_supported(nh, nkv, d, page_size),
             "attn_decode_bf16: unsupported sizes nh=%d nkv=%d d=%d page=%d", nh, nkv, d, page_size);
    LC_CHECK(qkv && k_cache && v_cache && out && decode_tokens && tok_req && positions && block_table,
             "attn_decode_bf16: null pointer");
    LC_CHECK(splits >= 1 && splits <= 65535 && (splits == 1 || (part_o && part_ml)),
             "attn_decode_bf16: %d shares need a workspace", splits);
    LC_CHECK(q_stride % 8 == 0 && (uintptr_t)qkv % 16 == 0, "attn_decode_bf16: q must be 16-byte aligned");
    const float sl2 = scale * 1.4426950408889634f;
#define CALL(DD) launch_decode<DD>((const bf16*)qkv, q_stride, (const bf16*)k_cache, (const bf16*)v_cache, \
        (bf16*)out, part_o, part_ml, decode_tokens, tok_req, positions, block_table, max_blocks,           \
        num_decode, nh, nkv, sl2, window, splits, stream)
    LC_DISPATCH_D(d, CALL)
#undef CALL
    return 0;
}

LC_API int lc_attn_prefill_bf16(const void* qkv, int q_stride, const void* k_cache, const void* v_cache,
                                void* out, const int* tiles, const int* block_table, int max_blocks,
                                int num_tiles, int nh, int nkv, int d, int page_size, float scale,
                                int window, hipStream_t stream) {
    if (num_tiles == 0) return 0;
    LC_CHECK(lc_attn_bf16_supported(nh, nkv, d, page_size),
             "attn_prefill_bf16: unsupported sizes nh=%d nkv=%d d=%d page=%d", nh, nkv, d, page_size);
    LC_CHECK(qkv && k_cache && v_cache && out && tiles && block_table, "attn_prefill_bf16: null pointer");
    LC_CHECK(q_stride % 8 == 0 && (uintptr_t)qkv % 16 == 0, "attn_prefill_bf16: q must be 16-byte aligned");
    const float sl2 = scale * 1.4426950408889634f;
#define CALL(DD) launch_prefill<DD>((const bf16*)qkv, q_stride, (const bf16*)k_cache, (const bf16*)v_cache, \
        (bf16*)out, tiles, block_table, max_blocks, num_tiles, nh, nkv, sl2, window, stream)
    LC_DISPATCH_D(d, CALL)
#undef CALL
    return 0;
}
