// Attention over the paged cache for any batch, head size and page size, computed with
// float32 arithmetic throughout (scores, max, exp, sum, P.V).  One workgroup per token (per two
// tokens of one request where a batch is mostly rows of prompts) and up to four query heads of
// one kv head, which share every key and value they load.
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
constexpr int AG_DIMS = 4;                // dims of the output a thread sums where the sizes allow whole pieces
constexpr int AG_PART = AG_THREADS * AG_DIMS + 2;   // floats a span leaves per head: every thread's sums, m, l

// The running (M, L, ACC) takes in a span's (m, l, acc).  Written with explicit operations so
// that both kernels that use it round alike.
template <int DV>
__device__ __forceinline__ void take_in(float& M, float& L, float (&ACC)[DV], float m, float l,
                                        const float (&acc)[DV]) {
    const float m_new = fmaxf(M, m);
    const float a = expf(M - m_new), b = expf(m - m_new);   // a = 0 for the first span (M = -inf)
    L = fmaf(L, a, __fmul_rn(l, b));
#pragma unroll
    for (int x = 0; x < DV; ++x) ACC[x] = fmaf(ACC[x], a, __fmul_rn(acc[x], b));
    M = m_new;
}

// Thread t holds the sums of key group t / (d_pow2 / DV) for the dims DV (t % (d_pow2 / DV)) + x.
// out[di] = (the key groups' sums of dim di, added from group 0 on) / L; ps: AG_THREADS * DV floats
template <typename T, int DV>
__device__ __forceinline__ void finish(const float (&ACC)[DV], float L, float* ps, T* out_row, int d, int d_pow2) {
    const int tid = threadIdx.x;
    __syncthreads();
#pragma unroll
    for (int x = 0; x < DV; ++x) ps[tid * DV + x] = (tid * DV + x) % d_pow2 < d ? ACC[x] : 0.f;
    __syncthreads();
    if (tid < d) {
        float total = 0.f;
        for (int gg = 0; gg < AG_THREADS * DV / d_pow2; ++gg) total = __fadd_rn(total, ps[gg * d_pow2 + tid]);
        out_row[tid] = from_f32<T>(total / L);
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

// What a workgroup keeps in LDS for R query rows.
template <int GH, int R>
struct AttendShared {
    __align__(16) float qs[R][GH][256];
    __align__(16) float ps[R][GH][AG_THREADS];
    float scratch[R * GH][AG_WAVES];
    int pages[AG_THREADS + 1];      // the chunk's pages, looked up once a chunk
};

// The rows t0 .. t0 + live - 1 (live <= R) of one request, GH query heads of one kv head: every
// key and value that is loaded serves all of them.  Each row's own sums are made exactly as if
// it were alone (a row takes no part in a chunk or span that lies behind its position), so its
// result has the same bits for every R.  R > 1: no window and no sharing out of spans (a
// window makes the chunks begin at a key of the row's own).
// DV = AG_DIMS where the head size is a multiple of 16 and the page size of 4 (whole 16-byte
// pieces: four lanes share a key's row for the scores, so that a wave reads 16 rows as one
// contiguous stretch each, and for the values a lane takes four neighbouring keys, which lie
// side by side in a page, of each of its DV dims: a weight read from LDS then serves DV sums);
// DV = 1 for any sizes.
// part == nullptr: the workgroup works through all spans of its rows and writes the results.
// Else (R = 1) blockIdx.z is the span (counted from the query's first) and its sums go to
// part[token][head][span][AG_PART].
template <typename T, int GH, int R, int DV>
__device__ __forceinline__ void attend_rows(
    AttendShared<GH, R>& sh, int t0, int live, int kvh, int h0, int heads,
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, T* __restrict__ out, const int* __restrict__ tok_req,
    const int* __restrict__ positions, const int* __restrict__ block_table, int max_blocks,
    int nh, int nkv, int d, int d_pow2, int page_size, float scale, int window,
    float* __restrict__ part, int part_spans) {
    const int tid = threadIdx.x;
    const int r = tok_req[t0];
    const int* table = block_table + (size_t)r * max_blocks;
    int p[R], p_max = -1;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        p[i] = i < live ? positions[t0 + i] : -1;
        p_max = max(p_max, p[i]);
    }
    const int j_lo = (R == 1 && window > 0 && p[0] - window + 1 > 0) ? p[0] - window + 1 : 0;
    const int s_first = j_lo / AG_SPAN;
    int s_begin = s_first, s_end = p_max / AG_SPAN;
    if (R == 1 && part) {
        s_begin = s_end = s_first + blockIdx.z;
        if (s_begin > p_max / AG_SPAN) return;
    }
    __syncthreads();                 // a call before this one may still read what is written now
    for (int i = tid; i < R * GH * 256; i += AG_THREADS) {
        const int row = i / (GH * 256), hh = (i >> 8) % GH, e = i & 255;
        (&sh.qs[0][0][0])[i] = (row < live && hh < heads && e < d)
            ? to_f32(q[(size_t)(t0 + row) * q_stride + (size_t)(h0 + hh) * d + e]) * scale : 0.f;
    }
    __syncthreads();

    static_assert(DV == 1 || (DV == AG_DIMS && GH >= DV), "finish() borrows ps for AG_THREADS * DV floats");
    constexpr bool vec = DV > 1;
    const int tpg = d_pow2 / DV;                // threads of a key group
    const int groups = AG_THREADS / tpg;        // key groups that share the P.V work
    const int g = tid / tpg, di = (tid % tpg) * DV;
    const bool pv_active = di < d;

    float M[R][GH], L[R][GH], ACC[R][GH][DV];
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
        for (int hh = 0; hh < GH; ++hh) {
            M[i][hh] = -INFINITY; L[i][hh] = 0.f;
#pragma unroll
            for (int x = 0; x < DV; ++x) ACC[i][hh][x] = 0.f;
        }

    for (int s = s_begin; s <= s_end; ++s) {
        const int lo = max(s * AG_SPAN, j_lo), hi_max = min(s * AG_SPAN + AG_SPAN - 1, p_max);
        int hi[R];
#pragma unroll
        for (int i = 0; i < R; ++i) hi[i] = min(s * AG_SPAN + AG_SPAN - 1, p[i]);   // below lo: the row has no such span
        float m[R][GH], l[R][GH], acc[R][GH][DV];
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int hh = 0; hh < GH; ++hh) {
                m[i][hh] = -INFINITY; l[i][hh] = 0.f;
#pragma unroll
                for (int x = 0; x < DV; ++x) acc[i][hh][x] = 0.f;
            }
        for (int c0 = lo; c0 <= hi_max; c0 += AG_THREADS) {
            const int count_max = min(AG_THREADS, hi_max - c0 + 1);
            int count[R];                 // the row's keys in this chunk; none: the row sits the chunk out
#pragma unroll
            for (int i = 0; i < R; ++i) count[i] = min(AG_THREADS, hi[i] - c0 + 1);
            float sc[R][GH];
            // the numbers of the chunk's pages go to LDS first: one trip to the block table a
            // chunk instead of one before every key's and value's own load
            const int page0 = c0 / page_size, page_n = (c0 + count_max - 1) / page_size - page0 + 1;
            for (int i = tid; i < page_n; i += AG_THREADS) sh.pages[i] = table[page0 + i];
            __syncthreads();
            if constexpr (vec) {
                // The four lanes of a key take its pieces of four entries in turn (lane `piece`
                // the pieces piece, piece + 4, ...): one load instruction then reads 64 bytes in
                // a row of each of a wave's 16 keys.  A thread works on its four keys (64 apart)
                // at once: a piece of q that it reads from LDS then serves all four, and their
                // loads are in flight together.  Each key's sum still takes its entries in order.
                const int piece = tid & 3;
                constexpr int UB = R == 1 ? 4 : 2;     // pieces of a key asked for before the first is used
                float dot[4][R][GH];
                const T* krow[4];
#pragma unroll
                for (int pass = 0; pass < 4; ++pass) {
                    // behind the chunk's last key: that key once more, whose score nobody reads
                    const int jk = c0 + min(pass * (AG_THREADS / 4) + (tid >> 2), count_max - 1);
                    const long long head = (long long)sh.pages[jk / page_size - page0] * nkv + kvh;
                    krow[pass] = k_cache + (head * page_size + (jk % page_size)) * d + piece * 4;
#pragma unroll
                    for (int i = 0; i < R; ++i)
#pragma unroll
                        for (int hh = 0; hh < GH; ++hh) dot[pass][i][hh] = 0.f;
                }
                for (int i0 = 0; i0 < d; i0 += 16 * UB) {
                    float k4[4][UB][4];
#pragma unroll
                    for (int u = 0; u < UB; ++u)
                        if (i0 + 16 * u < d)
#pragma unroll
                            for (int pass = 0; pass < 4; ++pass)
                                load4(k4[pass][u], krow[pass] + i0 + 16 * u);
#pragma unroll
                    for (int u = 0; u < UB; ++u)
                        if (i0 + 16 * u < d)
#pragma unroll
                            for (int i = 0; i < R; ++i)
#pragma unroll
                                for (int hh = 0; hh < GH; ++hh) {
                                    const float4 q4 = *reinterpret_cast<const float4*>(&sh.qs[i][hh][piece * 4 + i0 + 16 * u]);
#pragma unroll
                                    for (int pass = 0; pass < 4; ++pass) {
                                        float t = dot[pass][i][hh];
                                        t = fmaf(q4.x, k4[pass][u][0], t);
                                        t = fmaf(q4.y, k4[pass][u][1], t);
                                        t = fmaf(q4.z, k4[pass][u][2], t);
                                        t = fmaf(q4.w, k4[pass][u][3], t);
                                        dot[pass][i][hh] = t;
                                    }
                                }
                }
#pragma unroll
                for (int pass = 0; pass < 4; ++pass) {
                    const int kc = pass * (AG_THREADS / 4) + (tid >> 2);
#pragma unroll
                    for (int i = 0; i < R; ++i)
#pragma unroll
                        for (int hh = 0; hh < GH; ++hh) {   // the row's four quarters, in a fixed order
                            float t = dot[pass][i][hh];
                            t = __fadd_rn(t, __shfl_xor(t, 1, kWave));
                            t = __fadd_rn(t, __shfl_xor(t, 2, kWave));
                            if (piece == 0) sh.ps[i][hh][kc] = t;
                        }
                }
                __syncthreads();
#pragma unroll
                for (int i = 0; i < R; ++i)
#pragma unroll
                    for (int hh = 0; hh < GH; ++hh) sc[i][hh] = tid < count[i] ? sh.ps[i][hh][tid] : -INFINITY;
                __syncthreads();                            // ps is written again below
            } else {
#pragma unroll
                for (int i = 0; i < R; ++i)
#pragma unroll
                    for (int hh = 0; hh < GH; ++hh) sc[i][hh] = 0.f;
                if (tid < count_max) {
                    const int j = c0 + tid;
                    const long long head = (long long)sh.pages[j / page_size - page0] * nkv + kvh;
                    const T* krow = k_cache + (head * page_size + (j % page_size)) * d;
                    for (int e = 0; e < d; ++e) {
                        const float kv = to_f32(krow[e]);
#pragma unroll
                        for (int i = 0; i < R; ++i)
#pragma unroll
                            for (int hh = 0; hh < GH; ++hh) sc[i][hh] = fmaf(sh.qs[i][hh][e], kv, sc[i][hh]);
                    }
                }
#pragma unroll
                for (int i = 0; i < R; ++i)
                    if (tid >= count[i])
#pragma unroll
                        for (int hh = 0; hh < GH; ++hh) sc[i][hh] = -INFINITY;
            }
            float red[R * GH], alpha[R][GH];
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int hh = 0; hh < GH; ++hh) red[i * GH + hh] = sc[i][hh];
            block_reduce<R * GH, true>(red, sh.scratch);
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int hh = 0; hh < GH; ++hh) {
                    float pj = 0.f;
                    alpha[i][hh] = 1.f;
                    if (count[i] > 0) {
                        const float m_new = fmaxf(m[i][hh], red[i * GH + hh]);
                        pj = tid < count[i] ? expf(sc[i][hh] - m_new) : 0.f;
                        alpha[i][hh] = expf(m[i][hh] - m_new);  // 0 on a span's first chunk (m = -inf)
                        m[i][hh] = m_new;
                    }
                    sh.ps[i][hh][tid] = pj;
                    red[i * GH + hh] = pj;
                }
            block_reduce<R * GH, false>(red, sh.scratch);  // has the barriers that publish ps
#pragma unroll
            for (int i = 0; i < R; ++i)
                if (count[i] > 0)
#pragma unroll
                    for (int hh = 0; hh < GH; ++hh) {
                        l[i][hh] = fmaf(l[i][hh], alpha[i][hh], red[i * GH + hh]);
#pragma unroll
                        for (int x = 0; x < DV; ++x) acc[i][hh][x] = __fmul_rn(acc[i][hh][x], alpha[i][hh]);
                    }
            if (pv_active) {
                if constexpr (vec) {
                    // runs of four keys that start at a multiple of four lie in one page; a run
                    // may reach over the chunk's ends, where the keys count nothing (two runs
                    // of each of the thread's dims are asked for before the first is used; they
                    // are taken in in their order).
                    // Nothing in the loop is left out by a branch: a run behind the chunk's last is
                    // the last run once more, and a key outside the chunk counts as a value of
                    // zero with the weight of a key inside it (p >= 0, so the sum is only ever
                    // given a +0; a row that the key lies behind has p = 0 for it).
                    constexpr int UV = 2;      // runs asked for before the first is used
                    const int last_run = (c0 + count_max - 1) >> 2;
                    for (int run0 = (c0 >> 2) + g; run0 <= last_run; run0 += UV * groups) {
                        float v4[UV][DV][4];
#pragma unroll
                        for (int u = 0; u < UV; ++u) {
                            const int j4 = min(run0 + u * groups, last_run) * 4;
                            // a run may begin before the chunk's first key, in the page before its first
                            const int pg = j4 >= c0 ? sh.pages[j4 / page_size - page0] : table[j4 / page_size];
                            const T* vrow = v_cache + (((long long)pg * nkv + kvh) * d + di) * page_size + (j4 % page_size);
#pragma unroll
                            for (int x = 0; x < DV; ++x) load4(v4[u][x], vrow + x * page_size);
                        }
#pragma unroll
                        for (int u = 0; u < UV; ++u) {
                            const bool run_on = run0 + u * groups <= last_run;
                            const int j4 = min(run0 + u * groups, last_run) * 4;
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const int jj = j4 + e - c0;
                                const bool key_on = run_on && jj >= 0 && jj < count_max;
                                const int at = min(max(jj, 0), AG_THREADS - 1);
                                float v[DV];
#pragma unroll
                                for (int x = 0; x < DV; ++x) v[x] = key_on ? v4[u][x][e] : 0.f;
#pragma unroll
                                for (int i = 0; i < R; ++i)
#pragma unroll
                                    for (int hh = 0; hh < GH; ++hh) {
                                        const float pw = sh.ps[i][hh][at];
#pragma unroll
                                        for (int x = 0; x < DV; ++x) acc[i][hh][x] = fmaf(pw, v[x], acc[i][hh][x]);
                                    }
                            }
                        }
                    }
                } else {
                    for (int jj = g; jj < count_max; jj += groups) {
                        const int j = c0 + jj;
                        const long long head = (long long)sh.pages[j / page_size - page0] * nkv + kvh;
                        const float v = to_f32(v_cache[head * d * page_size + (long long)di * page_size + (j % page_size)]);
#pragma unroll
                        for (int i = 0; i < R; ++i)
                            if (jj < count[i])
#pragma unroll
                                for (int hh = 0; hh < GH; ++hh) acc[i][hh][0] = fmaf(sh.ps[i][hh][jj], v, acc[i][hh][0]);
                    }
                }
            }
            __syncthreads();  // ps is rewritten by the next chunk
        }
        if (R == 1 && part) {
            for (int hh = 0; hh < heads; ++hh) {
                float* mine = part + (((size_t)t0 * nh + h0 + hh) * part_spans + blockIdx.z) * AG_PART;
#pragma unroll
                for (int x = 0; x < DV; ++x) mine[tid * DV + x] = pv_active ? acc[0][hh][x] : 0.f;
                if (tid == 0) { mine[AG_PART - 2] = m[0][hh]; mine[AG_PART - 1] = l[0][hh]; }
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < R; ++i)
            if (hi[i] >= lo)
#pragma unroll
                for (int hh = 0; hh < GH; ++hh) take_in(M[i][hh], L[i][hh], ACC[i][hh], m[i][hh], l[i][hh], acc[i][hh]);
    }
#pragma unroll
    for (int i = 0; i < R; ++i)
        if (i < live)
#pragma unroll
            for (int hh = 0; hh < GH; ++hh)
                if (hh < heads)
                    finish<T, DV>(ACC[i][hh], L[i][hh], &sh.ps[0][0][0], out + ((size_t)(t0 + i) * nh + h0 + hh) * d, d, d_pow2);
}

// One workgroup per RT tokens and up to GH query heads of one kv head.  RT > 1: the tokens
// RT blockIdx.x ... of the batch are worked together when they belong to one request (the rows
// of a prompt), one after the other when they do not.
template <typename T, int GH, int RT, int DV>
__global__ __launch_bounds__(AG_THREADS) void attention_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, T* __restrict__ out, const int* __restrict__ tok_req,
    const int* __restrict__ positions, const int* __restrict__ block_table, int max_blocks,
    int T_, int nh, int nkv, int d, int d_pow2, int page_size, float scale, int window,
    float* __restrict__ part, int part_spans) {
    __shared__ AttendShared<GH, RT> sh;
    const int group = nh / nkv, batches = (group + GH - 1) / GH;
    const int kvh = blockIdx.y / batches;
    const int h0 = kvh * group + (blockIdx.y % batches) * GH;
    const int heads = min(GH, (kvh + 1) * group - h0);
    const int t0 = blockIdx.x * RT, live = min(RT, T_ - t0);
    if constexpr (RT > 1) {
        bool together = window <= 0 && part == nullptr;
        for (int i = 1; i < live; ++i) together = together && tok_req[t0 + i] == tok_req[t0];
        if (together) {
            attend_rows<T, GH, RT, DV>(sh, t0, live, kvh, h0, heads, q, q_stride, k_cache, v_cache, out, tok_req,
                                       positions, block_table, max_blocks, nh, nkv, d, d_pow2, page_size, scale,
                                       window, part, part_spans);
            return;
        }
    }
    auto& one = *reinterpret_cast<AttendShared<GH, 1>*>(&sh);
    if constexpr (RT == 1) {
        attend_rows<T, GH, 1, DV>(one, t0, 1, kvh, h0, heads, q, q_stride, k_cache, v_cache, out, tok_req, positions,
                                  block_table, max_blocks, nh, nkv, d, d_pow2, page_size, scale, window, part,
                                  part_spans);
    } else {
        for (int i = 0; i < live; ++i)
            attend_rows<T, GH, 1, DV>(one, t0 + i, 1, kvh, h0, heads, q, q_stride, k_cache, v_cache, out, tok_req,
                                      positions, block_table, max_blocks, nh, nkv, d, d_pow2, page_size, scale,
                                      window, nullptr, 0);
    }
}

// One workgroup per (token, head): the spans' sums from the workspace, taken in from the first.
template <typename T, int DV>
__global__ __launch_bounds__(AG_THREADS) void attention_generic_join_kernel(
    const float* __restrict__ part, int part_spans, T* __restrict__ out,
    const int* __restrict__ positions, int nh, int d, int d_pow2, int window) {
    __shared__ float ps[AG_THREADS * DV];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int p = positions[t];
    const int j_lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int spans = p / AG_SPAN - j_lo / AG_SPAN + 1;
    float M = -INFINITY, L = 0.f, ACC[DV];
#pragma unroll
    for (int x = 0; x < DV; ++x) ACC[x] = 0.f;
    for (int z = 0; z < spans; ++z) {
        const float* its = part + (((size_t)t * nh + h) * part_spans + z) * AG_PART;
        float acc[DV];
#pragma unroll
        for (int x = 0; x < DV; ++x) acc[x] = its[tid * DV + x];
        take_in<DV>(M, L, ACC, its[AG_PART - 2], its[AG_PART - 1], acc);
    }
    finish<T, DV>(ACC, L, ps, out + ((size_t)t * nh + h) * d, d, d_pow2);
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

constexpr int AG_ROWS = 2;                // tokens of a prompt that a workgroup may serve together
static thread_local int g_rows = 0;       // 0: by size; 1 or AG_ROWS: forced (tests, tuning)

// Rows a workgroup takes together: AG_ROWS where the batch is large enough to be mostly rows of
// prompts and still fills the card, and nothing (a window, spans shared out) stands against it.
static int rows_together(int T, int nh, int nkv, int window, int spans) {
    if (window > 0 || spans > 0) return 1;
    if (g_rows > 0) return g_rows;
    const int group = nh / nkv;
    const long long workgroups = (long long)T * nkv * ((group + AG_HEADS - 1) / AG_HEADS);
    return workgroups >= AG_ROWS * 1024 ? AG_ROWS : 1;
}

template <typename T, int DV>
static void launch_attention_generic(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                     void* out, const int* tok_req, const int* positions,
                                     const int* block_table, int max_blocks, int T_, int nh, int nkv, int d,
                                     int page_size, float scale, int window, float* workspace, int spans,
                                     hipStream_t stream) {
    int d_pow2 = 1;
    while (d_pow2 < d) d_pow2 <<= 1;
    const int group = nh / nkv;
    const int rows = rows_together(T_, nh, nkv, window, spans);
    dim3 grid((T_ + rows - 1) / rows, nkv * ((group + AG_HEADS - 1) / AG_HEADS), spans > 0 ? spans : 1);
    if (rows == AG_ROWS)
        attention_generic_kernel<T, AG_HEADS, AG_ROWS, DV><<<grid, AG_THREADS, 0, stream>>>(
            (const T*)q, q_stride, (const T*)k_cache, (const T*)v_cache, (T*)out, tok_req, positions,
            block_table, max_blocks, T_, nh, nkv, d, d_pow2, page_size, scale, window, nullptr, 0);
    else
        attention_generic_kernel<T, AG_HEADS, 1, DV><<<grid, AG_THREADS, 0, stream>>>(
            (const T*)q, q_stride, (const T*)k_cache, (const T*)v_cache, (T*)out, tok_req, positions,
            block_table, max_blocks, T_, nh, nkv, d, d_pow2, page_size, scale, window,
            spans > 0 ? workspace : nullptr, spans);
    if (spans > 0)
        attention_generic_join_kernel<T, DV><<<dim3(T_, nh), AG_THREADS, 0, stream>>>(
            workspace, spans, (T*)out, positions, nh, d, d_pow2, window);
}

}  // namespace lc

using namespace lc;

// Tests and tuning: 0 lets the size decide how many rows of a prompt a workgroup serves together, 1
// forces one and any larger number the kernel's several (for the calling thread).  Returns the
// setting before.
LC_API int lc_attention_generic_rows(int rows) {
    const int before = g_rows;
    if (rows >= 0) g_rows = rows > 1 ? AG_ROWS : rows;
    return before;
}

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
    LC_CHECK(nkv * ((nh / nkv + AG_HEADS - 1) / AG_HEADS) <= 65535, "attention: too many heads (%d)", nh);
    LC_CHECK(q && k_cache && v_cache && out && tok_req && positions && block_table,
             "attention: null pointer");
    const int spans = shared_spans(T, nh, nkv, max_blocks, page_size);
    LC_CHECK(spans == 0 || workspace, "attention: T=%d with %d blocks needs a workspace", T, max_blocks);
    LC_CHECK(spans <= 65535, "attention: too many spans (%d)", spans);
    const bool pieces = (d & 15) == 0 && (page_size & 3) == 0;     // whole 16-byte pieces of keys and values
#define LC_AG_LAUNCH(T, DV)                                                                                       \
    launch_attention_generic<T, DV>(q, q_stride, k_cache, v_cache, out, tok_req, positions, block_table, max_blocks, \
                                    T_, nh, nkv, d, page_size, scale, window, workspace, spans, stream)
    const int T_ = T;
    if (dt == DT_F32) {
        if (pieces) LC_AG_LAUNCH(float, AG_DIMS); else LC_AG_LAUNCH(float, 1);
    } else if (dt == DT_BF16) {
        if (pieces) LC_AG_LAUNCH(bf16, AG_DIMS); else LC_AG_LAUNCH(bf16, 1);
    } else {
        LC_CHECK(false, "attention: unknown dtype %d", dt);
    }
#undef LC_AG_LAUNCH
    LC_LAUNCH_CHECK("attention_generic");
    return 0;
}
