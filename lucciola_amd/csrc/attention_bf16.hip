// bfloat16 attention over the paged cache on the matrix cores, for pages of 16 tokens:
//   * decode: one query token per request; a workgroup owns (request, kv head, a share of the
//     pages), its 4 waves take pages in turn and meet in LDS; with several shares per request
//     the partial results (max, sum, unnormalised output) go to a workspace and a second
//     kernel joins them.  The query heads that share a kv head form the columns of one
//     matrix-core tile, so keys and values are read once per group.
//   * prefill: a workgroup owns 64 query rows of one request and one or two heads of a kv
//     head; pages go through LDS once per workgroup.
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

// QT: query column tiles (of 16 columns) that one wave carries; they share every K/V load.
template <int D, int QT>
struct AttnState {
    float m[QT], l[QT];      // running maximum and this lane's share of the sum
    floatx4 o[QT][D / 16];   // O^T tiles: o[c][t][v] = O[dim = 16 t + 4 (lane/16) + v][q = 16 c + lane%16]
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

// Maximum and sum over the four lanes q, q + 16, q + 32, q + 48 that hold one column of a
// matrix-core tile: two lane swaps of gfx950 (v_permlane32_swap exchanges the upper half of one
// register with the lower half of another, v_permlane16_swap the odd rows of 16 lanes with the
// even ones), no trip through LDS.  Written in assembly because the compiler's builtin loses
// the second result when both operands hold the same value; the s_nops cover the hazards
// that the compiler would otherwise handle.
__device__ __forceinline__ void swap_halves(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_rows(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float column_max(float x) {
    float a = x, b = x;
    swap_halves(a, b);
    a = b = fmaxf(a, b);
    swap_rows(a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float column_sum(float x) {
    float a = x, b = x;
    swap_halves(a, b);
    a = b = a + b;
    swap_rows(a, b);
    return a + b;
}

__device__ __forceinline__ short bf16_bits(float f) {
    const bf16 b = static_cast<bf16>(f);
    return *reinterpret_cast<const short*>(&b);
}

// One page of 16 keys starting at position `key0`.  lo/hi: the lowest and highest position
// this lane's query column (of each column tile) may see.
template <int D, int QT>
__device__ __forceinline__ void attend_page(AttnState<D, QT>& st, const PageRegs<D>& r,
                                            const bf16x8 (&bq)[QT][D / 32], int key0,
                                            const int (&lo)[QT], const int (&hi)[QT],
                                            float scale_log2, int lane) {
    const int j0 = key0 + (lane >> 4) * 4;
#pragma unroll
    for (int c = 0; c < QT; ++c) {
        floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < D / 32; ++i)
            s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(r.k[i], bq[c][i], s, 0, 0, 0);
        float mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int j = j0 + v;
            s[v] = (j >= lo[c] && j <= hi[c]) ? s[v] * scale_log2 : -INFINITY;
            mx = fmaxf(mx, s[v]);
        }
        mx = column_max(mx);
        const float m_new = fmaxf(st.m[c], mx);
        const float alpha = (st.m[c] == -INFINITY) ? 0.f : exp2f(st.m[c] - m_new);
        float p[4], psum = 0.f;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            p[v] = (s[v] == -INFINITY) ? 0.f : exp2f(s[v] - m_new);
            psum += p[v];
        }
        st.l[c] = st.l[c] * alpha + psum;
        st.m[c] = m_new;
        short4v pb;
#pragma unroll
        for (int v = 0; v < 4; ++v) pb[v] = bf16_bits(p[v]);
#pragma unroll
        for (int t = 0; t < D / 16; ++t) {
            st.o[c][t] *= alpha;
            st.o[c][t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(r.v[t], pb, st.o[c][t], 0, 0, 0);
        }
    }
}

template <int D, int QT>
__device__ __forceinline__ void init_state(AttnState<D, QT>& st) {
#pragma unroll
    for (int c = 0; c < QT; ++c) {
        st.m[c] = -INFINITY;
        st.l[c] = 0.f;
#pragma unroll
        for (int t = 0; t < D / 16; ++t) st.o[c][t] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
}

// Walk pages [begin, end) with stride `step`, the next page's loads in flight while the
// current one is multiplied.
template <int D, int QT>
__device__ __forceinline__ void attend_range(AttnState<D, QT>& st, const bf16x8 (&bq)[QT][D / 32],
                                             const bf16* __restrict__ k_cache,
                                             const bf16* __restrict__ v_cache,
                                             const int* __restrict__ table, int begin, int end,
                                             int step, int nkv, int kvh, const int (&lo)[QT],
                                             const int (&hi)[QT], float scale_log2, int lane,
                                             const int (&first_pages)[2], PageRegs<D>& cur,
                                             bool loaded) {
    // first_pages: table[begin] and table[begin + step], where they exist; loaded: the caller
    // has asked for the first page's keys and values (into cur) already
    if (begin >= end) return;
    PageRegs<D> nxt;
    if (!loaded) load_page<D>(cur, k_cache, v_cache, first_pages[0], nkv, kvh, lane);
    int next_page = first_pages[1];
    for (int pg = begin; pg < end; pg += step) {
        const bool more = pg + step < end;
        if (more) {
            load_page<D>(nxt, k_cache, v_cache, next_page, nkv, kvh, lane);
            if (pg + 2 * step < end) next_page = table[pg + 2 * step];
        }
        attend_page<D, QT>(st, cur, bq, pg * PAGE, lo, hi, scale_log2, lane);
        if (more) cur = nxt;
    }
}

// The same walk with two pages in flight beside the one being multiplied, for the decode kernel's
// workgroups of four waves (what it gains, and where not, stands at the launch).  The compiler counts the loads it
// knows of and, across a loop's back edge, waits for all of them; so a page's loads are inline
// assembly that it does not count, the waits are counted here, and three sets of page registers
// take turns, unrolled, so that no set is ever copied.  A set is written by the hardware long
// after the statement that names it: nothing may touch it between its loads and the counted wait
// that is followed by page_landed (a spilled set would store what the registers held before;
// the library asks its compiled kernels for their scratch size and takes the walk above if there
// is any).  The page numbers come through scalar loads (their addresses are the same for the whole wave),
// which the counter of the vector loads does not see.
template <int D>
__device__ __forceinline__ void load_page_uncounted(PageRegs<D>& r, const bf16* k_cache, const bf16* v_cache,
                                                    int page, int nkv, int kvh, int lane) {
    const size_t head = (size_t)page * nkv + kvh;
    const bf16* kb = k_cache + (head * PAGE + (lane & 15)) * D + (lane >> 4) * 8;
    const bf16* vb = v_cache + (head * D + (lane & 15)) * PAGE + (lane >> 4) * 4;
#pragma unroll
    for (int i = 0; i < D / 32; ++i)
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r.k[i]) : "v"(kb + i * 32) : "memory");
#pragma unroll
    for (int i = 0; i < D / 16; ++i)
        asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(r.v[i]) : "v"(vb + i * 16 * PAGE) : "memory");
}
template <int D>
__device__ __forceinline__ void page_landed(PageRegs<D>& r) {
#pragma unroll
    for (int i = 0; i < D / 32; ++i) asm volatile("" : "+v"(r.k[i]));
#pragma unroll
    for (int i = 0; i < D / 16; ++i) asm volatile("" : "+v"(r.v[i]));
}

// p0: the first page's registers; if first_loaded, the caller has asked for the page already, with
// ordinary loads (they stay in flight across code of the caller's that the compiler is free to
// arrange).  They are waited for here before the first uncounted load is issued, so that from
// then on the compiler knows of no load in flight and adds no wait of its own to the loop.
template <int D, int QT>
__device__ __forceinline__ void attend_range_deep(AttnState<D, QT>& st, const bf16x8 (&bq)[QT][D / 32],
                                                  const bf16* k_cache, const bf16* v_cache,
                                                  const int* __restrict__ table, int begin, int end,
                                                  int step, int nkv, int kvh, const int (&lo)[QT],
                                                  const int (&hi)[QT], float scale_log2, int lane,
                                                  PageRegs<D>& p0, bool first_loaded) {
    if (begin >= end) return;
    constexpr int LOADS = D / 32 + D / 16;            // of one page
    static_assert(2 * LOADS <= 63, "the counter of loads in flight has six bits");
    const int count = (end - begin + step - 1) / step;
    PageRegs<D> p1, p2;
    const int second = count > 1 ? table[begin + step] : 0;
    int ahead = count > 2 ? table[begin + 2 * step] : 0;      // the page of the next loads
    if (!first_loaded) load_page<D>(p0, k_cache, v_cache, table[begin], nkv, kvh, lane);
    wait_vmcnt<0>();
    page_landed<D>(p0);
    if (count > 1) load_page_uncounted<D>(p1, k_cache, v_cache, second, nkv, kvh, lane);
    // page i, in `cur`; the loads of page i + 2 go into `third`, which page i - 1 has left
    auto turn = [&](PageRegs<D>& cur, PageRegs<D>& third, int i) {
        if (i + 2 < count) {
            load_page_uncounted<D>(third, k_cache, v_cache, ahead, nkv, kvh, lane);
            if (i + 3 < count) ahead = table[begin + (i + 3) * step];
            wait_vmcnt<2 * LOADS>();
        } else if (i + 1 < count) {
            wait_vmcnt<LOADS>();
        } else {
            wait_vmcnt<0>();
        }
        page_landed<D>(cur);
        attend_page<D, QT>(st, cur, bq, (begin + i * step) * PAGE, lo, hi, scale_log2, lane);
    };
    for (int i = 0; i < count; i += 3) {
        turn(p0, p2, i);
        if (i + 1 < count) turn(p1, p0, i + 1);
        if (i + 2 < count) turn(p2, p1, i + 2);
    }
}

// ------------------------------------------------------------------------------- decode
// What an attention kernel does to the raw q (the decode kernel also: k, v) of its tokens before
// it attends, when the step has no separate kernel for it: RMSNorm over the head (weights optional), rotary
// embedding of the first `rot` entries (table optional: row p holds rot/2 cosines, then rot/2
// sines), and, if write_kv, the token's k and v into their place in the cache.  The formulas
// and their order are those of the separate kernel (elementwise.hip, qk_norm_rope_write).
struct DecodePrologue {
    const float* q_w;
    const float* k_w;
    const float* rope;
    float eps;
    int rot;
    int write_kv;
    int enabled;
    // the raw q, k, v as the shares of a product cut along K (float32 [num_shares][rows][width],
    // summed in their order and rounded to bfloat16 as the kernel that sums them would), or null
    const float* shares;
    int num_shares;
    int width;
    long long share_stride;
};

// Every workgroup prepares the q heads of its group itself (into LDS); the one whose share of
// the pages holds the token's own position also prepares k and v and writes them to the
// cache before anyone in the workgroup reads that page.
// NW waves take the pages of the workgroup's share in turn, each with one page in flight beside
// the one it works on: a workgroup draws on memory at NW times a wave's pace.
// DEEP: the walk with two pages in flight (attend_range_deep).
template <int D, int NW, bool DEEP>
__global__ __launch_bounds__(64 * NW) void attn_decode_kernel(
    const bf16* __restrict__ qkv, int q_stride, bf16* k_cache, bf16* v_cache,
    bf16* __restrict__ out, float* __restrict__ part_o,
    float* __restrict__ part_ml, const int4* __restrict__ decode_rows, const int* __restrict__ items,
    const int* __restrict__ block_table, int max_blocks, int nh, int nkv, float scale_log2,
    int window, int splits, DecodePrologue pro) {
    constexpr int ROW = D + 4;       // a head's D sums lie together; the padding spreads the heads over the banks
    __shared__ __attribute__((aligned(16))) float sm_o[NW][16 * ROW];
    __shared__ float sm_m[NW][16], sm_l[NW][16];
    __shared__ __attribute__((aligned(16))) bf16 sm_q[16 * D];

    // Two ways to share the work out.  Without `items`, the grid is (shares, kv heads, rows) and every
    // row's pages are cut into `splits` equal shares.  With `items` (eight numbers each: token row,
    // request, position, row, first page, end page, the row's number of shares, 0), the grid is (items,
    // kv heads): a list made on the host from the requests' lengths, which gives a long request more
    // shares than a short one; an item of no shares is a spare that does nothing.
    const int kvh = blockIdx.y;
    int split = blockIdx.x, di = blockIdx.z, my_shares = splits, item_begin = 0, item_end = 0;
    int4 mine;
    if (items) {
        const int4* it = reinterpret_cast<const int4*>(items) + (size_t)blockIdx.x * 2;
        mine = it[0];
        const int4 range = it[1];
        di = mine.w;
        item_begin = range.x;
        item_end = range.y;
        my_shares = range.z;
        split = 0;
        if (my_shares == 0) return;
    } else {
        // the token's row in the batch, its request's row of the block table and its position come
        // in one load: every look-up that hangs on another is a trip to memory before the first key
        mine = decode_rows[di];
    }
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // the same for the whole wave: its page numbers are scalar loads
    const int q = lane & 15, kg = lane >> 4;
    const int t = mine.x, req = mine.y, p = mine.z;
    const int G = nh / nkv;
    const int j_lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int first_page = j_lo / PAGE, last_page = p / PAGE;
    const int per = (last_page - first_page + splits) / splits;   // ceil(pages / splits)
    const int begin = items ? max(first_page, item_begin) : first_page + split * per;
    const int end = items ? min(item_end, last_page + 1) : min(begin + per, last_page + 1);
    const int* table = block_table + (size_t)req * max_blocks;
    // the numbers of the wave's first two pages: asked for now, they are back before the q/k preparation below is done
    const int pg0 = begin + wave;
    const int first_pages[2] = {pg0 < end ? table[pg0] : 0, pg0 + NW < end ? table[pg0 + NW] : 0};
    // the page that takes the token's own k and v (asked for with the others, not when it is needed)
    const bool owner = pro.enabled && pro.write_kv && begin <= last_page && last_page < end;
    const int own_page = owner ? table[last_page] : 0;

    // the wave's first page is asked for before q is prepared, so that the two trips to memory
    // run side by side; not the page that this workgroup is about to write the token's own k and v into
    PageRegs<D> first;
    const bool early = pg0 < end && !(owner && pg0 == last_page);
    if (early) load_page<D>(first, k_cache, v_cache, first_pages[0], nkv, kvh, lane);

    bf16x8 bq[1][D / 32];
    if (pro.enabled) {
        const int ntask = G + (owner ? 2 : 0);            // the q heads, then k, then v
        const int half = pro.rot / 2;
        const float* cs = pro.rope ? pro.rope + (size_t)p * pro.rot : nullptr;
        const bf16* row = qkv + (size_t)t * q_stride;
        if (D == 128 && (pro.rot == 128 || pro.rot == 0)) {
            // 16 lanes a head, as the separate kernel does it (and to the same bits)
            const int j = threadIdx.x & 15;
            // eight entries of the token's row of q, k, v from column `col` on
            auto chunk_at = [&](size_t col) -> head_chunk {
                if (!pro.shares) return *reinterpret_cast<const head_chunk*>(row + col);
                const float* src = pro.shares + (size_t)t * pro.width + col;
                floatx4 lo4 = {0.f, 0.f, 0.f, 0.f}, hi4 = {0.f, 0.f, 0.f, 0.f};
                // the shares are asked for eight at a time and added in their order once all are
                // back: one trip to memory for up to eight shares instead of one trip each (a
                // share past the last is the last one again, loaded and not added)
                constexpr int AT_ONCE = 8;
                for (int s0 = 0; s0 < pro.num_shares; s0 += AT_ONCE) {
                    floatx4 got_lo[AT_ONCE], got_hi[AT_ONCE];
#pragma unroll
                    for (int i = 0; i < AT_ONCE; ++i) {
                        const float* at = src + (size_t)min(s0 + i, pro.num_shares - 1) * pro.share_stride;
                        got_lo[i] = *reinterpret_cast<const floatx4*>(at);
                        got_hi[i] = *reinterpret_cast<const floatx4*>(at + 4);
                    }
#pragma unroll
                    for (int i = 0; i < AT_ONCE; ++i) {
                        if (s0 + i < pro.num_shares) {
                            lo4 += got_lo[i];
                            hi4 += got_hi[i];
                        }
                    }
                }
                head_chunk out8;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    out8[e] = static_cast<bf16>(lo4[e]);
                    out8[4 + e] = static_cast<bf16>(hi4[e]);
                }
                return out8;
            };
            for (int task = threadIdx.x >> 4; task < ntask; task += 4 * NW) {
                if (task == G + 1) {                      // v: copied, transposed into the page
                    const head_chunk raw = chunk_at((size_t)(nh + nkv + kvh) * D + 8 * j);
                    bf16* col = v_cache + ((size_t)own_page * nkv + kvh) * D * PAGE + (p % PAGE);
#pragma unroll
                    for (int e = 0; e < 8; ++e) col[(size_t)(8 * j + e) * PAGE] = raw[e];
                    continue;
                }
                const bool is_k = task == G;
                const size_t col = (size_t)(is_k ? nh + kvh : kvh * G + task) * D + 8 * j;
                bf16* dst = is_k ? k_cache + (((size_t)own_page * nkv + kvh) * PAGE + (p % PAGE)) * D
                                 : sm_q + task * D;
                // the weights and the table's row are asked for before the raw entries are waited for
                const Head128Constants consts = head128_constants(j, is_k ? pro.k_w : pro.q_w, cs);
                const head_chunk done = head128_norm_rope(chunk_at(col), j, consts, pro.eps);
                *reinterpret_cast<head_chunk*>(dst + 8 * j) = done;
            }
        } else {
            for (int task = wave; task < ntask; task += NW) {
                if (task == G + 1) {                          // v: copied, transposed into the page
                    const bf16* x = row + (size_t)(nh + nkv + kvh) * D;
                    bf16* col = v_cache + ((size_t)own_page * nkv + kvh) * D * PAGE + (p % PAGE);
                    for (int i = lane; i < D; i += 64) col[(size_t)i * PAGE] = x[i];
                    continue;
                }
                const bool is_k = task == G;
                const bf16* x = row + (size_t)(is_k ? nh + kvh : kvh * G + task) * D;
                const float* w = is_k ? pro.k_w : pro.q_w;
                bf16* dst = is_k ? k_cache + (((size_t)own_page * nkv + kvh) * PAGE + (p % PAGE)) * D
                                 : sm_q + task * D;
                float inv = 1.f;
                if (w) {
                    float ss = 0.f;
                    for (int i = lane; i < D; i += 64) {
                        const float v = static_cast<float>(x[i]);
                        ss += v * v;
                    }
                    ss = wave_sum(ss);
                    inv = rsqrtf(ss / (float)D + pro.eps);
                }
                for (int i = lane; i < half; i += 64) {
                    float a = static_cast<float>(x[i]) * inv, b = static_cast<float>(x[i + half]) * inv;
                    if (w) { a *= w[i]; b *= w[i + half]; }
                    float c = 1.f, sn = 0.f;
                    if (cs) { c = cs[i]; sn = cs[half + i]; }
                    dst[i] = static_cast<bf16>(a * c - b * sn);
                    dst[i + half] = static_cast<bf16>(a * sn + b * c);
                }
                for (int i = pro.rot + lane; i < D; i += 64) {
                    float a = static_cast<float>(x[i]) * inv;
                    if (w) a *= w[i];
                    dst[i] = static_cast<bf16>(a);
                }
            }
        }
        __syncthreads();      // q is in LDS; the owner's k and v have reached memory
        const bf16* qrow = sm_q + min(q, G - 1) * D + kg * 8;
#pragma unroll
        for (int i = 0; i < D / 32; ++i) bq[0][i] = *reinterpret_cast<const bf16x8*>(qrow + i * 32);
    } else {
        const bf16* qrow = qkv + (size_t)t * q_stride + (size_t)(kvh * G + min(q, G - 1)) * D + kg * 8;
#pragma unroll
        for (int i = 0; i < D / 32; ++i) bq[0][i] = *reinterpret_cast<const bf16x8*>(qrow + i * 32);
    }
    AttnState<D, 1> st;
    init_state<D, 1>(st);
    const int lo[1] = {j_lo}, hi[1] = {p};
    if (DEEP)
        attend_range_deep<D, 1>(st, bq, k_cache, v_cache, table, begin + wave, end, NW, nkv, kvh, lo, hi,
                                scale_log2, lane, first, early);
    else
        attend_range<D, 1>(st, bq, k_cache, v_cache, table, begin + wave, end, NW, nkv, kvh, lo, hi,
                           scale_log2, lane, first_pages, first, early);

    // the waves' results meet in LDS
    float l = st.l[0];
    l = column_sum(l);
    if (kg == 0) { sm_m[wave][q] = st.m[0]; sm_l[wave][q] = l; }
    if (q < G) {
#pragma unroll
        for (int tt = 0; tt < D / 16; ++tt)
            *reinterpret_cast<floatx4*>(&sm_o[wave][q * ROW + tt * 16 + kg * 4]) = st.o[0][tt];
    }
    __syncthreads();
    // four sums of a head a thread
    for (int idx = threadIdx.x; idx < G * (D / 4); idx += 64 * NW) {
        const int qq = idx / (D / 4), dim = (idx % (D / 4)) * 4;
        float m_all = sm_m[0][qq];
#pragma unroll
        for (int w = 1; w < NW; ++w) m_all = fmaxf(m_all, sm_m[w][qq]);
        floatx4 o = {0.f, 0.f, 0.f, 0.f};
        float lsum = 0.f;
        if (m_all != -INFINITY) {
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const float f = (sm_m[w][qq] == -INFINITY) ? 0.f : exp2f(sm_m[w][qq] - m_all);
                o += f * *reinterpret_cast<const floatx4*>(&sm_o[w][qq * ROW + dim]);
                lsum += f * sm_l[w][qq];
            }
        }
        const int h = kvh * G + qq;
        if (my_shares == 1) {
            short4v packed;
#pragma unroll
            for (int v = 0; v < 4; ++v) packed[v] = bf16_bits(o[v] / lsum);
            *reinterpret_cast<short4v*>(out + ((size_t)t * nh + h) * D + dim) = packed;
        } else {
            const size_t slot = items ? (size_t)blockIdx.x * nh + h : ((size_t)di * nh + h) * splits + split;
            *reinterpret_cast<floatx4*>(part_o + slot * D + dim) = o;
            if (dim == 0) { part_ml[slot * 2] = m_all; part_ml[slot * 2 + 1] = lsum; }
        }
    }
}

template <int D, int MOST>
__device__ __forceinline__ void join_shares_of(const float* __restrict__ part_o,
                                               const float* __restrict__ part_ml, size_t base,
                                               size_t stride, int splits, bf16* __restrict__ out_row) {
    __shared__ float f[64];
    __shared__ float inv_l;
    const int tid = threadIdx.x;
    // the shares' sums are asked for before their factors are: one trip to memory instead of two
    float early[MOST];
    if (tid < D) {
#pragma unroll
        for (int s = 0; s < MOST; ++s) early[s] = s < splits ? part_o[(base + s * stride) * D + tid] : 0.f;
    }
    if (tid < 64) {
        const float ms = tid < splits ? part_ml[(base + tid * stride) * 2] : -INFINITY;
        const float ls = tid < splits ? part_ml[(base + tid * stride) * 2 + 1] : 0.f;
        const float m = wave_max(ms);
        const float fs = (ms == -INFINITY) ? 0.f : exp2f(ms - m);
        f[tid] = fs;
        const float l = wave_sum(fs * ls);
        if (tid == 0) inv_l = 1.f / l;
    }
    __syncthreads();
    if (tid < D) {
        float o = 0.f;
#pragma unroll
        for (int s = 0; s < MOST; ++s) o += f[s] * early[s];     // f is 0 beyond the shares
        out_row[tid] = static_cast<bf16>(o * inv_l);
    }
}

// Joins the shares of a row's keys: out = sum_s o_s 2^(m_s - m) / sum_s l_s 2^(m_s - m), the
// shares of (row, head) lying at part_o[base + s stride][D] and part_ml[base + s stride][2].  The factors are
// worked out once (one thread per share) and left in LDS.  128 threads (D <= 128); at most 64 shares.
template <int D>
__device__ __forceinline__ void join_shares(const float* __restrict__ part_o,
                                            const float* __restrict__ part_ml, size_t base,
                                            size_t stride, int splits, bf16* __restrict__ out_row) {
    if (splits <= 8) join_shares_of<D, 8>(part_o, part_ml, base, stride, splits, out_row);
    else if (splits <= 32) join_shares_of<D, 32>(part_o, part_ml, base, stride, splits, out_row);
    else join_shares_of<D, 64>(part_o, part_ml, base, stride, splits, out_row);
}

template <int D>
__global__ __launch_bounds__(128) void attn_decode_join_kernel(const float* __restrict__ part_o,
                                                               const float* __restrict__ part_ml,
                                                               const int4* __restrict__ decode_rows,
                                                               bf16* __restrict__ out, int nh,
                                                               int splits, int by_items) {
    const int di = blockIdx.x, h = blockIdx.y;
    const int4 row = decode_rows[di];
    bf16* out_row = out + ((size_t)row.x * nh + h) * D;
    if (by_items) {
        // the row's items are neighbours in the list: the first in the low 20 bits, their number above;
        // the only item of a row has written the row itself
        const int first = row.w & 0xFFFFF, count = row.w >> 20;
        if (count > 1) join_shares<D>(part_o, part_ml, (size_t)first * nh + h, nh, count, out_row);
    } else {
        join_shares<D>(part_o, part_ml, ((size_t)di * nh + h) * splits, 1, splits, out_row);
    }
}

// The same for the rows of prefill tiles, whose shares lie at the rows' places in the batch.
template <int D>
__global__ __launch_bounds__(128) void attn_prefill_join_kernel(const float* __restrict__ part_o,
                                                                const float* __restrict__ part_ml,
                                                                const int* __restrict__ tiles,
                                                                bf16* __restrict__ out, int nh,
                                                                int splits) {
    const int* tile = tiles + (size_t)(blockIdx.x >> 6) * 4;
    const int r = blockIdx.x & 63, h = blockIdx.y;
    if (r >= tile[2]) return;
    const int t = tile[1] + r;
    join_shares<D>(part_o, part_ml, ((size_t)t * nh + h) * splits, 1, splits, out + ((size_t)t * nh + h) * D);
}

// A lane's part of one raw q row of 128 entries, as the matrix-core operand holds it (entries
// 32 i + 8 kg + e, i < 4, so an entry and its partner 64 further on sit in the same lane):
// RMSNorm over the head and the rotary embedding at position p, on the operand registers.  The
// formulas and the order of their roundings are those of head128_norm_rope; only the sum of
// squares is added up in another order.
__device__ __forceinline__ void prepare_q128(bf16x8 (&bq)[4], const DecodePrologue& pro, int p, int kg) {
    if (!pro.enabled) return;
    float f[4][8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) f[i][e] = static_cast<float>(bq[i][e]);
    if (pro.q_w) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int e = 0; e < 8; ++e) ss = __fmaf_rn(f[i][e], f[i][e], ss);
        ss = column_sum(ss);
        const float inv = rsqrtf(ss / 128.f + pro.eps);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int e = 0; e < 8; ++e)
                f[i][e] = __fmul_rn(__fmul_rn(f[i][e], inv), pro.q_w[i * 32 + kg * 8 + e]);
    }
    if (pro.rope) {
        const float* cs = pro.rope + (size_t)p * 128;     // 64 cosines, then 64 sines
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float cosv = cs[i * 32 + kg * 8 + e], sinv = cs[64 + i * 32 + kg * 8 + e];
                const float a = f[i][e], b = f[i + 2][e];
                f[i][e] = __fsub_rn(__fmul_rn(a, cosv), __fmul_rn(b, sinv));
                f[i + 2][e] = __fadd_rn(__fmul_rn(a, sinv), __fmul_rn(b, cosv));
            }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) bq[i][e] = static_cast<bf16>(f[i][e]);
}

// ------------------------------------------------------------------------------- prefill
// tiles: [NT, 4] = (request, first token row, rows (<= 64), position of the first row), the
// tiles that see the most keys first.
// A workgroup takes one tile and HPW heads of one kv head and walks the pages the tile can
// see, PF_NP pages (64 keys) at a time.  Its 256 threads bring a group of pages into LDS
// together (the next group's loads are in flight in registers meanwhile), and every wave
// builds its matrix-core operands from LDS: keys and values cross the memory system once per
// workgroup.  One softmax update (maximum, rescale) serves the whole group of pages, and every
// key or value operand read from LDS serves all of the wave's column tiles.
// HPW = 2 (an even number of heads per kv head): wave w works on head w / 2 of the pair and on
// rows [32 (w % 2), +32) as two column tiles; HPW = 1: wave w works on rows [16 w, +16).
// Key rows are padded by 16 bytes in LDS, which spreads the 16 keys of an operand read over
// all banks; value pages are interleaved in pairs and rotated for the same reason.
constexpr int PF_NP = 4;   // even: value pages go to LDS in pairs


template <int D, int HPW>
__global__ __launch_bounds__(256, 2) void attn_prefill_kernel(
    const bf16* __restrict__ qkv, int q_stride, const bf16* __restrict__ k_cache,
    const bf16* __restrict__ v_cache, bf16* __restrict__ out, const int* __restrict__ tiles,
    const int* __restrict__ block_table, int max_blocks, int nh, int nkv, float scale_log2,
    int window, DecodePrologue pro, int splits, float* __restrict__ part_o,
    float* __restrict__ part_ml, int resident) {
    constexpr int QT = HPW, NP = PF_NP;
    constexpr int KLD = D + 8;
    constexpr int KPAGE = PAGE * KLD, VPAGE = D * PAGE;   // elements of a page in LDS
    constexpr int CHUNKS = 4 * D;                         // 8-byte chunks of a key (or value) page
    constexpr int CH = (CHUNKS + 255) / 256;
    __shared__ __attribute__((aligned(16))) bf16 ks[2][NP * KPAGE];
    __shared__ __attribute__((aligned(16))) bf16 vs[2][NP * VPAGE];

    // Which tile and which heads.  Workgroups start in the order of their number (x fastest)
    // and two fit on a CU; the tiles come longest first, and a tile's heads are neighbours, so
    // that the workgroups that read the same keys and values run at the same time.  With more
    // workgroups than fit at once, whoever is done takes the longest tile that is left.  When
    // all fit at once, nobody takes over from a CU that is done early, and the second workgroup
    // of a CU should be as short as its first is long: the second half of the numbers takes the
    // tasks from the shortest up.
    const int total = gridDim.x * gridDim.y, number = blockIdx.y * gridDim.x + blockIdx.x;
    const int half = (total + 1) / 2;
    const int task = (total <= resident && number >= half) ? total - 1 - (number - half) : number;
    // with few tiles and many keys, a tile's pages are cut into `splits` shares (x counts tile
    // and share), each a workgroup of its own whose sums a second kernel joins
    const int tile_share = task / gridDim.y, heads_index = task - tile_share * gridDim.y;
    const int tile_index = tile_share / splits, split = tile_share - tile_index * splits;
    const int* tile = tiles + (size_t)tile_index * 4;
    const int req = tile[0], row0 = tile[1], rows = tile[2], pos0 = tile[3];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q = lane & 15, kg = lane >> 4;
    const int G = nh / nkv;
    const int h = HPW == 2 ? heads_index * 2 + (wave >> 1) : heads_index;
    const int wrow = HPW == 2 ? (wave & 1) * 32 : wave * 16;
    const int kvh = (heads_index * HPW) / G;
    const bool active = h < nh && wrow < rows;
    const int* table = block_table + (size_t)req * max_blocks;

    bf16x8 bq[QT][D / 32];
    int lo[QT], hi[QT];
    bool valid[QT];
#pragma unroll
    for (int c = 0; c < QT; ++c) {
        const int my = wrow + c * 16 + q;                 // this lane's query row inside the tile
        valid[c] = active && my < rows;
        const int p = pos0 + min(my, rows - 1);
        hi[c] = valid[c] ? p : 0x7fffffff;                // idle columns see everything (never stored)
        lo[c] = (valid[c] && window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
        const bf16* qrow = qkv + (size_t)(row0 + min(my, rows - 1)) * q_stride +
                           (size_t)min(h, nh - 1) * D + kg * 8;
#pragma unroll
        for (int i = 0; i < D / 32; ++i) bq[c][i] = *reinterpret_cast<const bf16x8*>(qrow + i * 32);
        if constexpr (D == 128) prepare_q128(bq[c], pro, p, kg);
    }
    // pages the workgroup walks, and the part of them this wave needs
    const int t_lo = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
    int first = t_lo / PAGE, last = (pos0 + rows - 1) / PAGE;
    if (splits > 1) {       // this workgroup's share of them, in whole groups of pages
        const int per = ((last - first + splits) / splits + NP - 1) / NP * NP;
        first += split * per;
        last = min(last, first + per - 1);
    }
    const int w_min = pos0 + min(wrow, rows - 1), w_max = pos0 + min(wrow + 16 * QT - 1, rows - 1);
    const int w_lo = (window > 0 && w_min - window + 1 > 0) ? w_min - window + 1 : 0;
    const int w_first = w_lo / PAGE, w_last = w_max / PAGE;
    const int w_lo_max = (window > 0 && w_max - window + 1 > 0) ? w_max - window + 1 : 0;

    AttnState<D, QT> st;
    init_state<D, QT>(st);

    // a group's pages on their way from global memory to LDS: 32 bytes a thread and page
    short4v kreg[NP][CH], vreg[NP][CH];
    auto fetch = [&](int pg0) {
#pragma unroll
        for (int n = 0; n < NP; ++n) {
            const int pg = pg0 + n;
            const bool there = pg <= last;
            const size_t head = there ? (size_t)table[pg] * nkv + kvh : 0;
            const bf16* kp = k_cache + head * PAGE * D;
            const bf16* vp = v_cache + head * D * PAGE;
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                const int c = tid + i * 256;
                kreg[n][i] = short4v{0, 0, 0, 0};      // pages past the end read as zeros
                vreg[n][i] = short4v{0, 0, 0, 0};
                if (there && (CHUNKS % 256 == 0 || c < CHUNKS)) {
                    kreg[n][i] = *reinterpret_cast<const short4v*>(kp + c * 4);
                    vreg[n][i] = *reinterpret_cast<const short4v*>(vp + c * 4);
                }
            }
        }
    };
    fetch(first);

    for (int pg0 = first, it = 0; pg0 <= last; pg0 += NP, ++it) {
        const int stage = it & 1;
#pragma unroll
        for (int n = 0; n < NP; ++n)
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                const int c = tid + i * 256;
                if (CHUNKS % 256 == 0 || c < CHUNKS) {
                    const int key = c / (D / 4), col = (c % (D / 4)) * 4;
                    *reinterpret_cast<short4v*>(&ks[stage][n * KPAGE + key * KLD + col]) = kreg[n][i];
                    // values: the pages of a pair (n, n + 1) are interleaved, [dim][4 keys of n | the same
                    // 4 keys of n + 1] in 16-byte pieces, so that a product's operand is one 128-bit
                    // read; the pieces of a row rotate with the row, which spreads the 16 rows of
                    // a read (and the 16 pieces of a write) over all banks
                    if ((n & 1) == 0) {
                        const int dim = c >> 2, piece = (c & 3) ^ ((dim >> 2) & 3);
                        union { short4v h[2]; bf16x8 full; } both;
                        both.h[0] = vreg[n][i];
                        both.h[1] = vreg[n + 1][i];
                        *reinterpret_cast<bf16x8*>(&vs[stage][(n >> 1) * 2 * VPAGE + dim * 32 + piece * 8]) = both.full;
                    }
                }
            }
        if (pg0 + NP <= last) fetch(pg0 + NP);
        __syncthreads();    // also keeps a fast wave from overwriting the stage a slow one reads
        if (!active || pg0 > w_last || pg0 + NP - 1 < w_first) continue;

        // scores of the group: sc[c][n][v] = S[key 16 (pg0 + n) + 4 kg + v][column q of tile c]
        floatx4 sc[QT][NP];
#pragma unroll
        for (int n = 0; n < NP; ++n)
#pragma unroll
            for (int c = 0; c < QT; ++c) sc[c][n] = floatx4{0.f, 0.f, 0.f, 0.f};
        // i outermost: QT x NP independent accumulators lie between two products into the same one
#pragma unroll
        for (int i = 0; i < D / 32; ++i)
#pragma unroll
            for (int n = 0; n < NP; ++n) {
                const bf16x8 ka = *reinterpret_cast<const bf16x8*>(&ks[stage][n * KPAGE + q * KLD + i * 32 + kg * 8]);
#pragma unroll
                for (int c = 0; c < QT; ++c)
                    sc[c][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, bq[c][i], sc[c][n], 0, 0, 0);
            }
        // only groups that touch a row's own position (or the window's edge) need the mask
        const bool masked = (pg0 + NP) * PAGE - 1 > w_min || pg0 * PAGE < w_lo_max;
        bf16x8 pb[QT][NP / 2];
        bool rescale = false;
        float alpha[QT];
#pragma unroll
        for (int c = 0; c < QT; ++c) {
            float mx = -INFINITY;
            if (masked) {
#pragma unroll
                for (int n = 0; n < NP; ++n)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int j = (pg0 + n) * PAGE + kg * 4 + v;
                        if (j < lo[c] || j > hi[c]) sc[c][n][v] = -INFINITY;
                    }
            }
#pragma unroll
            for (int n = 0; n < NP; ++n)
#pragma unroll
                for (int v = 0; v < 4; ++v) mx = fmaxf(mx, sc[c][n][v]);
            mx = column_max(mx);
            // Maxima are kept as raw scores; p = 2^((s - m) scale_log2), one fma and one v_exp.
            // m is a reference point, not necessarily the maximum: it moves (and the sums are
            // rescaled) only when a score would exceed it by more than 2^8, which keeps every p
            // in range and makes rescaling rare.  The result sum p v / sum p is the same for
            // any reference; the choice is made per query row from that row's scores alone.
            const bool move = mx * scale_log2 > st.m[c] * scale_log2 + 8.f;   // true while m is -inf
            const float m_new = move ? mx : st.m[c];
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            alpha[c] = move ? __builtin_amdgcn_exp2f((st.m[c] - m_use) * scale_log2) : 1.f;   // 2^-inf = 0 at the start
            const float neg = -m_use * scale_log2;
            float psum = 0.f;
#pragma unroll
            for (int n = 0; n < NP; ++n)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(sc[c][n][v], scale_log2, neg));
                    psum += p;
                    pb[c][n / 2][(n & 1) * 4 + v] = static_cast<bf16>(p);
                }
            st.l[c] = st.l[c] * alpha[c] + psum;
            st.m[c] = m_new;
            rescale = rescale || move;
        }
        if (__any(rescale)) {
#pragma unroll
            for (int c = 0; c < QT; ++c)
#pragma unroll
                for (int t = 0; t < D / 16; ++t) st.o[c][t] *= alpha[c];
        }
        // two pages per product: lane group kg supplies keys 4 kg .. 4 kg + 3 of both pages
#pragma unroll
        for (int n = 0; n < NP; n += 2)
#pragma unroll
            for (int t = 0; t < D / 16; ++t) {
                const bf16x8 va = *reinterpret_cast<const bf16x8*>(
                    &vs[stage][(n >> 1) * 2 * VPAGE + (t * 16 + q) * 32 + ((kg ^ ((q >> 2) & 3)) * 8)]);
#pragma unroll
                for (int c = 0; c < QT; ++c)
                    st.o[c][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb[c][n / 2], st.o[c][t], 0, 0, 0);
            }
    }
    if (splits > 1) {       // sums as they are, with their reference point in the units of the exponent
#pragma unroll
        for (int c = 0; c < QT; ++c) {
            float l = st.l[c];
            l = column_sum(l);
            if (!valid[c]) continue;
            const size_t slot = ((size_t)(row0 + wrow + c * 16 + q) * nh + h) * splits + split;
            float* po = part_o + slot * D + kg * 4;
#pragma unroll
            for (int tt = 0; tt < D / 16; ++tt) *reinterpret_cast<floatx4*>(po + tt * 16) = st.o[c][tt];
            if (kg == 0) {
                part_ml[slot * 2] = st.m[c] == -INFINITY ? -INFINITY : st.m[c] * scale_log2;
                part_ml[slot * 2 + 1] = l;
            }
        }
        return;
    }
#pragma unroll
    for (int c = 0; c < QT; ++c) {
        float l = st.l[c];
        l = column_sum(l);
        if (!valid[c]) continue;
        const float inv = 1.f / l;
        bf16* orow = out + ((size_t)(row0 + wrow + c * 16 + q) * nh + h) * D + kg * 4;
#pragma unroll
        for (int tt = 0; tt < D / 16; ++tt) {
            short4v packed;
#pragma unroll
            for (int v = 0; v < 4; ++v) packed[v] = bf16_bits(st.o[c][tt][v] * inv);
            *reinterpret_cast<short4v*>(orow + tt * 16) = packed;
        }
    }
}

// ------------------------------------------------------------------------------- prefill, wide products
// For heads of 128 in pairs: the tiles and the LDS staging of attn_prefill_kernel<128, 2>, built
// from v_mfma_f32_32x32x16_bf16.  Two workgroups a CU; a wave does its group's scores, softmax
// and values one after the other, and the two waves of a SIMD fill each other's gaps.
// (Measured on this GPU: a product of 16x16x32 holds the vector unit for all of its 16 cycles,
// so products and softmax take turns even between two waves of a SIMD, 64 products and the
// softmax of their scores 1,495 ns for two waves; a product of 32x32x16 takes 32 cycles and
// lets the other wave's vector instructions through meanwhile, 1,065 ns for the same work.)
//
// A wave owns 32 query rows of one head.  Per group of 64 keys:
//   S^T[key, q]  = K[key, :] . Q[q, :]     16 products: A = 32 key rows x 16 dims from LDS,
//                                          B = Q^T from registers; a lane ends up with 16 keys
//                                          of one query column per 32-key tile
//   P^T          = exp2(S^T * scale*log2(e) - reference)       vector unit, float32
//   O^T[dim, q] += V^T[dim, key] . P^T[key, q]   16 products: A = 32 dims x 16 keys from LDS,
//                                          B = P^T as the lanes hold it
// Keys lie in LDS in rows padded by 16 bytes; values per page [dim][16 keys] with a row's four
// pieces of 4 keys in the order 0, 2, 1, 3, so that the 8 keys a lane supplies to a product (4
// and the 4 eight further on, as the scores left them in its registers) are one 16-byte read,
// and with the two halves of a row changing places in every other block of 8 rows, which
// spreads the 16 rows of a read over all banks (the counters show no bank conflict).  The
// page numbers come from the block table a group ahead, one page per lane in one vector load:
// a scalar load per page, each waited for before its page's loads could go out, took a third
// of the time of a group.
typedef float floatx16 __attribute__((ext_vector_type(16)));

// A lane's part of one raw q row of 128 entries in the layout of the 32x32x16 operand (entries
// 16 i + 8 half + e, i < 8, half = lane / 32: an entry and its partner 64 further on sit in the
// same lane, the row's other half in lane ^ 32): RMSNorm over the head and the rotary
// embedding at position p.  Formulas and roundings as in head128_norm_rope; the sum of
// squares is added up in another order.
__device__ __forceinline__ void prepare_q128_wide(bf16x8 (&bq)[8], const DecodePrologue& pro, int p, int half) {
    if (!pro.enabled) return;
    float f[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) f[i][e] = static_cast<float>(bq[i][e]);
    if (pro.q_w) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 8; ++e) ss = __fmaf_rn(f[i][e], f[i][e], ss);
        float a = ss, b = ss;
        swap_halves(a, b);
        ss = a + b;
        const float inv = rsqrtf(ss / 128.f + pro.eps);
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 8; ++e)
                f[i][e] = __fmul_rn(__fmul_rn(f[i][e], inv), pro.q_w[i * 16 + half * 8 + e]);
    }
    if (pro.rope) {
        const float* cs = pro.rope + (size_t)p * 128;     // 64 cosines, then 64 sines
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float cosv = cs[i * 16 + half * 8 + e], sinv = cs[64 + i * 16 + half * 8 + e];
                const float a = f[i][e], b = f[i + 4][e];
                f[i][e] = __fsub_rn(__fmul_rn(a, cosv), __fmul_rn(b, sinv));
                f[i + 4][e] = __fadd_rn(__fmul_rn(a, sinv), __fmul_rn(b, cosv));
            }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) bq[i][e] = static_cast<bf16>(f[i][e]);
}

template <int D>
__global__ __launch_bounds__(256, 2) void attn_prefill_wide_kernel(
    const bf16* __restrict__ qkv, int q_stride, const bf16* __restrict__ k_cache,
    const bf16* __restrict__ v_cache, bf16* __restrict__ out, const int* __restrict__ tiles,
    const int* __restrict__ block_table, int max_blocks, int nh, int nkv, float scale_log2,
    int window, DecodePrologue pro, int resident) {
    static_assert(D == 128, "heads of 128");
    constexpr int NP = PF_NP;
    constexpr int KLD = D + 8;
    constexpr int KPAGE = PAGE * KLD, VPAGE = D * PAGE;
    __shared__ __attribute__((aligned(16))) bf16 ks[2][NP * KPAGE];
    __shared__ __attribute__((aligned(16))) bf16 vs[2][NP * VPAGE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q = lane & 31, half = lane >> 5;
    const int G = nh / nkv;
    // Workgroups start in the order of their number (x, the head pair, fastest) and two fit on a
    // CU; the tiles come longest first.  With more workgroups than fit at once, whoever is done
    // takes the longest tile that is left.  When all fit at once, nobody takes over from a CU
    // that is done early, and the second workgroup of a CU should be as short as its first is
    // long: the second half of the numbers takes the tiles from the shortest up.
    const int total = gridDim.x * gridDim.y, number = blockIdx.y * gridDim.x + blockIdx.x;
    const int half_of = (total + 1) / 2;
    const int task = (total <= resident && number >= half_of) ? total - 1 - (number - half_of) : number;
    const int tile_index = task / gridDim.x, heads_index = task - tile_index * gridDim.x;
    // the pairs of heads of one kv head; with an odd number of heads a kv head, the last pair is
    // a single head, and the two waves of its other half only help to bring keys and values in
    const int pairs = (G + 1) / 2;
    const int kvh = heads_index / pairs, in_kv = (heads_index - kvh * pairs) * 2 + (wave >> 1);
    const int h = min(kvh * G + in_kv, nh - 1);
    const int wrow = (wave & 1) * 32;
    {
        const int* tile = tiles + (size_t)tile_index * 4;
        const int req = tile[0], row0 = tile[1], rows = tile[2], pos0 = tile[3];
        const bool active = wrow < rows && in_kv < G;
        const int* table = block_table + (size_t)req * max_blocks;

        const int my = wrow + q;
        const bool valid = active && my < rows;
        const int p = pos0 + min(my, rows - 1);
        const int hi = valid ? p : 0x7fffffff;
        const int lo = (valid && window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
        bf16x8 bq[D / 16];
        {
            const bf16* qrow = qkv + (size_t)(row0 + min(my, rows - 1)) * q_stride + (size_t)h * D + half * 8;
#pragma unroll
            for (int i = 0; i < D / 16; ++i) bq[i] = *reinterpret_cast<const bf16x8*>(qrow + i * 16);
            prepare_q128_wide(bq, pro, p, half);
        }
        const int t_lo = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
        const int first = t_lo / PAGE, last = (pos0 + rows - 1) / PAGE;
        const int groups = (last - first) / NP + 1;
        const int w_min = pos0 + min(wrow, rows - 1), w_max = pos0 + min(wrow + 31, rows - 1);
        const int w_lo_max = (window > 0 && w_max - window + 1 > 0) ? w_max - window + 1 : 0;

        float m_ref = -INFINITY, l_sum = 0.f;
        floatx16 o[D / 32];
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) o[t][v] = 0.f;

        bf16x8 kreg[NP], vreg[NP];
        int ids_ahead;                  // lane n % 4: page n of the group after the one on its way
        auto lookup = [&](int g) { ids_ahead = table[min(first + g * NP + (lane & 3), last)]; };
        auto fetch = [&](const int (&ids)[NP]) {
#pragma unroll
            for (int n = 0; n < NP; ++n) {
                const size_t head = (size_t)ids[n] * nkv + kvh;
                kreg[n] = *reinterpret_cast<const bf16x8*>(k_cache + head * PAGE * D + tid * 8);
                vreg[n] = *reinterpret_cast<const bf16x8*>(v_cache + head * D * PAGE + tid * 8);
            }
        };
        auto stage = [&](int g) {
            bf16* kd = ks[g & 1];
            bf16* vd = vs[g & 1];
            const int key = tid >> 4, col = (tid & 15) * 8;
            const int dim = tid >> 1, hsel = tid & 1, flip = (dim >> 3) & 1;
#pragma unroll
            for (int n = 0; n < NP; ++n) {
                *reinterpret_cast<bf16x8*>(&kd[n * KPAGE + key * KLD + col]) = kreg[n];
                union { bf16x8 full; short4v h[2]; } both;
                both.full = vreg[n];
                *reinterpret_cast<short4v*>(&vd[n * VPAGE + dim * 16 + flip * 8 + hsel * 4]) = both.h[0];
                *reinterpret_cast<short4v*>(&vd[n * VPAGE + dim * 16 + (flip ^ 1) * 8 + hsel * 4]) = both.h[1];
            }
        };
        {
            int ids[NP];
#pragma unroll
            for (int n = 0; n < NP; ++n) ids[n] = table[min(first + n, last)];
            fetch(ids);
            lookup(1);
        }
        for (int g = 0; g < groups; ++g) {
            stage(g);
            {
                int ids[NP];
#pragma unroll
                for (int n = 0; n < NP; ++n) ids[n] = __builtin_amdgcn_readlane(ids_ahead, n);
                lookup(g + 2);
                fetch(ids);             // group g + 1 (past the end: the last page again, unused)
            }
            __syncthreads();    // also keeps a fast wave from overwriting the stage a slow one reads
            const int pg0 = first + g * NP;
            if (!active) continue;
            const bf16* kd = ks[g & 1];
            const bf16* vd = vs[g & 1];
            floatx16 sc[2];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int v = 0; v < 16; ++v) sc[kt][v] = 0.f;
#pragma unroll
            for (int i = 0; i < D / 16; ++i)
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    const bf16x8 ka = *reinterpret_cast<const bf16x8*>(&kd[(kt * 32 + q) * KLD + i * 16 + half * 8]);
                    sc[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, bq[i], sc[kt], 0, 0, 0);
                }
            if ((pg0 + NP) * PAGE - 1 > w_min || pg0 * PAGE < w_lo_max) {     // the group touches a row's own position or the window's edge
                const int key0 = pg0 * PAGE + half * 4;
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int j = key0 + kt * 32 + (v >> 2) * 8 + (v & 3);
                        if (j < lo || j > hi) sc[kt][v] = -INFINITY;
                    }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sc[kt][v]);
            {
                float a = mx, b = mx;
                swap_halves(a, b);
                mx = fmaxf(a, b);
            }
            const bool move = mx * scale_log2 > m_ref * scale_log2 + 8.f;   // true while m_ref is -inf
            const float m_new = move ? mx : m_ref;
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = move ? __builtin_amdgcn_exp2f((m_ref - m_use) * scale_log2) : 1.f;
            const float neg = -m_use * scale_log2;
            float psum = 0.f;
            bf16x8 pb[2][2];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float pv = __builtin_amdgcn_exp2f(fmaf(sc[kt][v], scale_log2, neg));
                    psum += pv;
                    pb[kt][v >> 3][v & 7] = static_cast<bf16>(pv);
                }
            l_sum = l_sum * alpha + psum;
            m_ref = m_new;
            if (__any(move)) {
#pragma unroll
                for (int t = 0; t < D / 32; ++t)
#pragma unroll
                    for (int v = 0; v < 16; ++v) o[t][v] *= alpha;
            }
#pragma unroll
            for (int page = 0; page < NP; ++page)
#pragma unroll
                for (int t = 0; t < D / 32; ++t) {
                    const int dim = t * 32 + q;
                    const bf16x8 va = *reinterpret_cast<const bf16x8*>(
                        &vd[page * VPAGE + dim * 16 + ((half ^ ((dim >> 3) & 1)) * 8)]);
                    o[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb[page >> 1][page & 1], o[t], 0, 0, 0);
                }
        }
        {
            float a = l_sum, b = l_sum;
            swap_halves(a, b);
            const float l = a + b;
            if (valid) {
                const float inv = 1.f / l;
                bf16* orow = out + ((size_t)(row0 + my) * nh + h) * D + half * 4;
#pragma unroll
                for (int t = 0; t < D / 32; ++t)
#pragma unroll
                    for (int blk = 0; blk < 4; ++blk) {
                        short4v packed;
#pragma unroll
                        for (int v = 0; v < 4; ++v) packed[v] = bf16_bits(o[t][blk * 4 + v] * inv);
                        *reinterpret_cast<short4v*>(orow + t * 32 + blk * 8) = packed;
                    }
            }
        }
    }
}

static thread_local int g_decode_waves = 0;   // 0: by the launch's shape
static thread_local int g_decode_deep = 1;    // 0: never the walk with two pages in flight (tests, tuning)

// Whether the decode kernel that walks with two pages in flight keeps its page registers in
// registers: 1 yes, 0 it spills (its uncounted loads would not be safe), -1 could not ask.
template <int D>
static int decode_deep_state() {
    static const int state = [] {
        hipFuncAttributes attr;
        if (hipFuncGetAttributes(&attr, (const void*)attn_decode_kernel<D, 4, true>) != hipSuccess) {
            (void)hipGetLastError();
            return -1;
        }
        return attr.localSizeBytes != 0 ? 0 : 1;
    }();
    return state;
}

template <int D>
static int launch_decode(const bf16* qkv, int q_stride, bf16* k, bf16* v, bf16* out,
                         float* part_o, float* part_ml, const int4* decode_rows, const int* items,
                         int num_items, const int* table, int max_blocks, int ND, int nh,
                         int nkv, float scale_log2, int window, int splits, bool even_lengths,
                         DecodePrologue pro, hipStream_t s) {
    const dim3 grid = items ? dim3(num_items, nkv, 1) : dim3(splits, nkv, ND);
    // One workgroup per request and kv head (no shares): requests of unequal length leave the
    // long ones running alone at the end, each at the pace its waves draw on memory; eight
    // waves double that (64 requests of 16 to 2,176 tokens: 59 instead of 65 us; equal lengths
    // take the same time either way, short shares are slower with eight).  From four workgroups
    // a CU on, four waves: all of them are on the CUs at once instead of in two rounds (128
    // requests of 1,024 tokens: 116 instead of 125 us; 96 requests: 95 against 93).
    // One workgroup a CU or fewer: eight waves, which keep twice the loads in flight on the CU
    // (with cold caches, as in a step: 8 requests of 8,192 tokens in four shares each 55.8
    // instead of 57.4 us, 16 in two 104.7 instead of 107.4, one request with its join 16.1 instead
    // of 17.2, 8 of 1,024 tokens 15.7 instead of 16.8).  Two shares of more requests than CUs
    // likewise.
    const long long workgroups = items ? (long long)num_items * nkv : (long long)ND * nkv * splits;
    // Whole requests of about the same length, more of them than CUs: nobody is left running
    // alone, and four waves a workgroup are as good or better (with cold caches 48 requests of
    // 1,024 tokens 48.8 instead of 53.5 us, 64 requests 58.9 instead of 61.7, 32 of 8,192 192
    // instead of 194).
    const bool alone_at_the_end = !even_lengths || workgroups <= device_cus();
    // (a list of items is made for requests of unequal length: eight waves)
    const int waves = g_decode_waves ? g_decode_waves
                      : items ? 8
                      : (splits == 1 && max_blocks >= 32 && workgroups < 4ll * device_cus() && alone_at_the_end) ? 8
                      : (splits > 1 && workgroups <= device_cus()) ? 8
                      : (splits == 2 && workgroups > 2ll * device_cus()) ? 8 : 4;
    // Two pages in flight beside the one being multiplied where the workgroups have four waves (many
    // workgroups, or whole requests of even lengths): with cold caches 64 requests of 8,192 tokens
    // 375 -> 359 us (6.0 TB/s), of 1,024 tokens 55.1 -> 53.1, 256 of 1,024 210.8 -> 208.1.  Not with
    // eight waves: their launches are short shares or requests of unequal length, whose long ones run
    // on alone at the end at the pace at which a wave works through a page (about 1.5 us, two waves
    // a SIMD), not at what it has in flight (one request of 8,192 tokens among 63 of 512: 103.9 us
    // with one page ahead, 108.5 with two; 16 requests of 100 to 8,000: 58.3 and 60.3).
    const bool deep = waves == 4 && g_decode_deep && decode_deep_state<D>() == 1;
#define LC_DECODE(NW, DEEP)                                                                             \
    attn_decode_kernel<D, NW, DEEP><<<grid, 64 * NW, 0, s>>>(qkv, q_stride, k, v, out, part_o, part_ml, \
                                                             decode_rows, items, table, max_blocks, nh, \
                                                             nkv, scale_log2, window, splits, pro)
    if (waves == 8) LC_DECODE(8, false);
    else if (deep) LC_DECODE(4, true);
    else LC_DECODE(4, false);
#undef LC_DECODE
    LC_LAUNCH_CHECK("attn_decode");
    if (splits > 1 || items) {
        attn_decode_join_kernel<D><<<dim3(ND, nh), 128, 0, s>>>(
            part_o, part_ml, decode_rows, out, nh, splits, items ? 1 : 0);
        LC_LAUNCH_CHECK("attn_decode_join");
    }
    return 0;
}

// pairs of heads share the keys and values they read; with so few tiles that half of the CUs
// would get nothing to do, single heads and twice the workgroups are faster (measured)
// (where the keys are shared out, the shares fill the CUs, and pairs stay)
static bool prefill_head_pairs(int NT, int nh, int nkv, int splits) {
    return (nh / nkv) % 2 == 0 && ((long long)NT * (nh / 2) > device_cus() / 2 || splits > 1);
}

static thread_local int g_prefill_wide = 1;   // 0: never the kernel built from the wide products (tests, tuning)

template <int D>
static int launch_prefill(const bf16* qkv, int q_stride, const bf16* k, const bf16* v, bf16* out,
                          const int* tiles, const int* table, int max_blocks, int NT, int nh,
                          int nkv, float scale_log2, int window, DecodePrologue pro, int splits,
                          float* part_o, float* part_ml, hipStream_t s) {
    const int resident = 2 * device_cus();     // workgroups of these kernels that run at once: two a CU
    if constexpr (D == 128) {
        // heads of 128 in pairs, every tile's keys walked by one workgroup: the kernel built from
        // the wide products
        // (an odd number of heads a kv head from 3 on: the last pair is a single head, which leaves a CU's
        // matrix cores half idle for a sixth of the pairs of five heads, where one head a workgroup in the
        // kernel below takes 1.6 times as long for all of them)
        if (g_prefill_wide && ((nh / nkv) % 2 == 0 || nh / nkv >= 3) && splits == 1) {
            attn_prefill_wide_kernel<D><<<dim3(nkv * ((nh / nkv + 1) / 2), NT), 256, 0, s>>>(qkv, q_stride, k, v, out, tiles, table,
                                                                       max_blocks, nh, nkv, scale_log2, window, pro, resident);
            LC_LAUNCH_CHECK("attn_prefill_wide");
            return 0;
        }
    }
    if (prefill_head_pairs(NT, nh, nkv, splits))
        attn_prefill_kernel<D, 2><<<dim3(NT * splits, nh / 2), 256, 0, s>>>(qkv, q_stride, k, v, out, tiles, table,
                                                                            max_blocks, nh, nkv, scale_log2, window, pro,
                                                                            splits, part_o, part_ml, resident);
    else
        attn_prefill_kernel<D, 1><<<dim3(NT * splits, nh), 256, 0, s>>>(qkv, q_stride, k, v, out, tiles, table,
                                                                        max_blocks, nh, nkv, scale_log2, window, pro,
                                                                        splits, part_o, part_ml, resident);
    LC_LAUNCH_CHECK("attn_prefill");
    if (splits > 1) {
        attn_prefill_join_kernel<D><<<dim3(NT * 64, nh), 128, 0, s>>>(part_o, part_ml, tiles, out, nh, splits);
        LC_LAUNCH_CHECK("attn_prefill_join");
    }
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

// Tokens of a cache page as these kernels index it; a page of a multiple of it is served as so
// many pages of this size in a row.
LC_API int lc_attn_page_granule() { return PAGE; }

// Whether heads of 128 in pairs go to the prefill kernel built from the wide products (1, the
// default) or to the general one (0).  For tests and tuning.
LC_API int lc_attn_prefill_wide(int on) {
    g_prefill_wide = on ? 1 : 0;
    return 0;
}

// Waves of a decode workgroup (4 or 8; 0: chosen by the launch's shape).  For tests and tuning.
// 0: the decode kernel walks its pages with one page in flight beside the one it multiplies, 1
// (the default): with two where its workgroups have four waves and the kernel keeps its registers.
// Returns the setting before.
LC_API int lc_attn_decode_deep(int on) {
    const int before = g_decode_deep;
    g_decode_deep = on ? 1 : 0;
    return before;
}
// Whether the kernels of heads of d walk with two pages in flight when the switch is on (1), or
// cannot (0: a page register spills; -1: the runtime could not be asked; -2: no such head size).
LC_API int lc_attn_decode_deep_ok(int d) {
    switch (d) {
        case 32: return decode_deep_state<32>();
        case 64: return decode_deep_state<64>();
        case 96: return decode_deep_state<96>();
        case 128: return decode_deep_state<128>();
        default: return -2;
    }
}

LC_API int lc_attn_decode_waves(int waves) {
    LC_CHECK(waves == 0 || waves == 4 || waves == 8, "attn_decode: %d waves (0, 4 or 8)", waves);
    g_decode_waves = waves;
    return 0;
}

// Into how many shares the decode kernel cuts a request's pages.  Up to one workgroup of whole
// requests a CU: the number that costs least when the CUs take the workgroups in rounds, which is
// mostly what gives every CU one workgroup and no more (12 requests of 8,192 tokens are better
// off with five shares each, two rounds of 102 pages, than with two, one round of 256: 82.5
// against 97.1 us) (8 requests of 8,192
// tokens: 45.7 us in four shares each, 49.8 in eight, 50.3 in six; 4 requests 28.2 in eight,
// 30.7 in sixteen; 16 requests 102.8 in two, 106.6 in four; 24 requests 150.7 whole, 161.2 in
// two; a workgroup more than the CUs, and a second round has to wait for the first: 3 requests
// in 22 shares each took 31 us, in 21 26).  With more workgroups of whole requests than CUs:
// three shares each from 2,048 tokens on and while all of them fit on the CUs at once, four
// four-wave workgroups a CU (40 requests of 8,192 tokens: 249 instead of 271 us, of 1,024 tokens
// 47.3 against 44.7 whole; 44 requests of 4,096 in three shares each,
// 1,056 workgroups, 162, whole 152, in two shares of eight waves 146); beyond that, up to one
// and a half workgroups a CU and from 4,096 tokens on, two shares of eight waves (48 requests
// of 8,192 tokens: 289 us, 311 with four waves, 302 whole); else none (52 requests of 4,096
// tokens: 164 whole, 175 in two shares).  A share has 8 pages or more, and there are at most 32.
static thread_local int g_force_splits = 0;    // > 0: this many shares where the pages allow (tests, tuning)
LC_API int lc_attn_decode_force_splits(int splits) {
    g_force_splits = splits > 0 ? splits : 0;
    return 0;
}
LC_API int lc_attn_decode_splits(int num_decode, int nkv, int max_ctx) {
    if (num_decode <= 0) return 1;
    const int pages = (max_ctx + PAGE - 1) / PAGE;
    if (g_force_splits > 0) return g_force_splits < pages ? (g_force_splits > 32 ? 32 : g_force_splits) : (pages > 32 ? 32 : pages);
    const long long base = (long long)num_decode * nkv;
    const int cus = device_cus();       // the thresholds were measured with 256 of them
    int most = (pages + 7) / 8;
    if (most > 32) most = 32;
    if (most < 1) most = 1;
    long long splits = 1;
    if (base <= cus) {
        // the CUs work through the workgroups in rounds; a workgroup costs its pages and about as
        // much as 32 pages more to start, look up, prepare q and leave its sums
        long long best = -1;
        for (int s = 1; s <= most; ++s) {
            const long long rounds = (base * s + cus - 1) / cus;
            if (rounds > 2) break;      // more than two workgroups a CU were slower whenever measured
            // (two rounds, which are four-wave workgroups, count a tenth more than twice one round of
            // eight-wave workgroups: with cold caches 12 requests of 8,192 tokens take 81.5 us in
            // two shares each, 84.3 in five)
            const long long cost = (rounds == 1 ? 10 : 22) * ((pages + s - 1) / s + 32);
            if (best < 0 || cost < best) { best = cost; splits = s; }
        }
    } else {
        splits = (3 * base <= 4 * cus && pages >= 128) ? 3 : (2 * base <= 3 * cus && pages >= 256) ? 2 : 1;
        if (splits > most) splits = most;
    }
    return (int)splits;
}

// Whether a step's decode rows are better served through the planner's list of work items, which
// gives a long request more shares than a short one, than with the same number of shares for
// every request: longest and total are the requests' lengths in tokens.  With few requests (the
// workgroups of one share each fill half of the CUs at most) as soon as the lengths are uneven; with many
// only when a few requests hold most of the keys, because the list brings half as many workgroups
// more and always a join (with cold caches: one request of 8,192 tokens among 63 of 512 103 -> 45 us,
// 16 requests of 100 to 8,000 tokens 57.1 -> 52.8, 8 such 37.4 -> 33.6; but 64 of 16 to 2,200 tokens
// 57.1 -> 65.6, 128 such 107 -> 122, 64 of 1,024 53.3 -> 63.9, 8 of 1,024 14.6 -> 18.8).
LC_API int lc_attn_decode_by_items(int num_decode, int nkv, int longest, long long total) {
    if (num_decode < 2 || total <= 0) return 0;
    const long long spread = (long long)longest * num_decode;       // against the total: 1 for equal lengths
    if ((long long)num_decode * nkv * 2 <= device_cus()) return spread * 4 > total * 5;
    return spread >= total * 3;
}

#define LC_DISPATCH_D(d, CALL)                   \
    switch (d) {                                 \
        case 32: return CALL(32);                \
        case 64: return CALL(64);                \
        case 96: return CALL(96);                \
        case 128: return CALL(128);              \
        default: LC_CHECK(false, "attention_bf16: head size %d has no matrix-core kernel", d); \
    }

// Whether lc_attn_decode_bf16 takes the raw q, k, v as the float32 shares of a product cut along K
// (qkv_shares [num_shares][share_rows][q_stride], summed in their order and rounded to bfloat16 as
// the kernel that sums shares does): with its own preparation of whole heads of 128.
LC_API int lc_attn_decode_takes_shares(int d, int rot) { return d == 128 && (rot == 0 || rot == 128); }

// decode_rows: four numbers a row (token row, request, position, and with items: the row's first
// item in the low 20 bits, its number of items above).  items (or null): num_items work items of
// eight numbers (token row, request, position, row, first page, end page, the row's number of
// items, 0), a row's items neighbours in the list and their page ranges in ascending order, the
// last one reaching the row's last page; part_o and part_ml then hold num_items x nh entries.
// prologue != 0: qkv holds the raw projections; the kernel norms and rotates q and k itself
// (q_w, k_w, rope_table may be null; rot entries of a head rotate) and, if write_kv != 0, writes
// the tokens' k and v to the cache.  Otherwise qkv is ready and the cache holds the tokens.
LC_API int lc_attn_decode_bf16(const void* qkv, int q_stride, void* k_cache, void* v_cache,
                               void* out, float* part_o, float* part_ml, const int* decode_rows,
                               const int* items, int num_items, const int* block_table,
                               int max_blocks, int num_decode, int nh, int nkv, int d, int page_size,
                               float scale, int window, int splits, int even_lengths, int prologue, const float* q_w,
                               const float* k_w, float eps, const float* rope_table, int rot,
                               int write_kv, const float* qkv_shares, int num_shares, int share_rows,
                               hipStream_t stream) {
    if (num_decode == 0) return 0;
    LC_CHECK(!prologue || (rot >= 0 && rot <= d && rot % 2 == 0 && (q_w == nullptr) == (k_w == nullptr)),
             "attn_decode_bf16: bad prologue (rot=%d of %d)", rot, d);
    DecodePrologue pro = {q_w, k_w, rope_table, eps, rope_table ? rot : 0, write_kv, prologue,
                          qkv_shares, num_shares, q_stride, (long long)share_rows * q_stride};
    LC_CHECK(lc_attn_bf16_supported(nh, nkv, d, page_size),
             "attn_decode_bf16: unsupported sizes nh=%d nkv=%d d=%d page=%d", nh, nkv, d, page_size);
    LC_CHECK(!qkv_shares || lc_attn_decode_takes_shares(d, prologue ? pro.rot : -1),
             "attn_decode_bf16: q, k, v as shares of a product need the kernel's own preparation of heads of 128 "
             "(d=%d, %d rotary entries)", d, pro.rot);
    LC_CHECK(!qkv_shares || (num_shares >= 1 && share_rows >= 1 && q_stride % 4 == 0 && (uintptr_t)qkv_shares % 16 == 0),
             "attn_decode_bf16: bad shares (%d of %d rows)", num_shares, share_rows);
    if (qkv_shares && !qkv) qkv = qkv_shares;      // never read, but not null
    LC_CHECK(qkv && k_cache && v_cache && out && decode_rows && block_table,
             "attn_decode_bf16: null pointer");
    LC_CHECK((uintptr_t)decode_rows % 16 == 0, "attn_decode_bf16: the decode rows must be 16-byte aligned");
    LC_CHECK(splits >= 1 && splits <= 65535 && (splits == 1 || (part_o && part_ml)),
             "attn_decode_bf16: %d shares need a workspace", splits);
    LC_CHECK(!items || (num_items >= 1 && splits == 1 && part_o && part_ml && (uintptr_t)items % 16 == 0),
             "attn_decode_bf16: a list of items (%d) needs a workspace, 16-byte alignment and no equal shares beside it (%d)",
             num_items, splits);
    LC_CHECK(q_stride % 8 == 0 && (uintptr_t)qkv % 16 == 0, "attn_decode_bf16: q must be 16-byte aligned");
    LC_CHECK(!prologue || ((uintptr_t)q_w % 16 == 0 && (uintptr_t)k_w % 16 == 0 && (uintptr_t)rope_table % 16 == 0),
             "attn_decode_bf16: the norms' weights and the rotary table must be 16-byte aligned");
    const float sl2 = scale * 1.4426950408889634f;
#define CALL(DD) launch_decode<DD>((const bf16*)qkv, q_stride, (bf16*)k_cache, (bf16*)v_cache,             \
        (bf16*)out, part_o, part_ml, (const int4*)decode_rows, items, num_items, block_table, max_blocks,   \
        num_decode, nh, nkv, sl2, window, splits, even_lengths != 0, pro, stream)
    LC_DISPATCH_D(d, CALL)
#undef CALL
    return 0;
}

// Into how many shares the prefill kernel cuts the keys of every tile: more than one when the
// tiles are so few that CUs would stand idle while each workgroup walks a long history (a
// portion of a prompt that follows thousands of cached tokens); a share has at least 1,024 keys
// (measured: with fewer, writing and joining the shares costs more than the idle CUs).
LC_API int lc_attn_prefill_splits(int num_tiles, int nh, int nkv, int max_ctx) {
    if (num_tiles <= 0 || nkv <= 0) return 1;
    const long long groups = (long long)num_tiles * ((nh / nkv) % 2 == 0 ? nh / 2 : nh);
    if (groups >= device_cus()) return 1;
    long long splits = 2 * device_cus() / groups;         // no more workgroups than run at once
    const int most = (max_ctx + PAGE - 1) / PAGE / 64;
    if (splits > most) splits = most;
    if (splits > 16) splits = 16;
    return splits < 1 ? 1 : (int)splits;
}

// Whether the prefill kernel can norm and rotate q itself for this head size and rotary width
// (whole heads of 128 that rotate whole or not at all).
LC_API int lc_attn_prefill_prepares_q(int d, int rot) { return d == 128 && (rot == 0 || rot == 128); }

// prologue != 0 (lc_attn_prefill_prepares_q(d, rot) must hold): q in qkv is raw; the kernel norms
// (q_w may be null) and rotates it itself (rope_table may be null).  The step's keys and values
// are in the cache either way.  splits > 1 (at most 64): every tile's keys are cut into that
// many shares; part_o [T rows of the batch][nh][splits][d] and part_ml [T][nh][splits][2] float32.
LC_API int lc_attn_prefill_bf16(const void* qkv, int q_stride, const void* k_cache, const void* v_cache,
                                void* out, const int* tiles, const int* block_table, int max_blocks,
                                int num_tiles, int nh, int nkv, int d, int page_size, float scale,
                                int window, int prologue, const float* q_w, float eps,
                                const float* rope_table, int rot, int splits, float* part_o,
                                float* part_ml, hipStream_t stream) {
    if (num_tiles == 0) return 0;
    LC_CHECK(splits >= 1 && splits <= 64 && (splits == 1 || (part_o && part_ml)),
             "attn_prefill_bf16: %d shares (1 to 64; more than one need a workspace)", splits);
    LC_CHECK((long long)num_tiles * splits <= 0x7fffffff / 64, "attn_prefill_bf16: too many tiles (%d)", num_tiles);
    LC_CHECK(lc_attn_bf16_supported(nh, nkv, d, page_size),
             "attn_prefill_bf16: unsupported sizes nh=%d nkv=%d d=%d page=%d", nh, nkv, d, page_size);
    LC_CHECK(qkv && k_cache && v_cache && out && tiles && block_table, "attn_prefill_bf16: null pointer");
    LC_CHECK(q_stride % 8 == 0 && (uintptr_t)qkv % 16 == 0, "attn_prefill_bf16: q must be 16-byte aligned");
    if (!rope_table) rot = 0;
    LC_CHECK(!prologue || lc_attn_prefill_prepares_q(d, rot),
             "attn_prefill_bf16: the kernel cannot prepare q for head size %d with %d rotary entries", d, rot);
    const float sl2 = scale * 1.4426950408889634f;
    DecodePrologue pro = {q_w, nullptr, rope_table, eps, rot, 0, prologue};
#define CALL(DD) launch_prefill<DD>((const bf16*)qkv, q_stride, (const bf16*)k_cache, (const bf16*)v_cache, \
        (bf16*)out, tiles, block_table, max_blocks, num_tiles, nh, nkv, sl2, window, pro, splits,       \
        part_o, part_ml, stream)
    LC_DISPATCH_D(d, CALL)
#undef CALL
    return 0;
}
