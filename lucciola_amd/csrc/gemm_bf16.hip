// bfloat16 matrix products on the matrix cores: out[M, N] = x[M, K] . w[N, K]^T, float32
// accumulation, output bfloat16 or float32.  Two kernels:
//
//  * skinny (M <= 16, decode): bound by reading w once from HBM.  A workgroup owns 16 rows of
//    w; its waves split K in interleaved blocks of 128, each wave streaming its part of the
//    rows straight from global memory into v_mfma_f32_16x16x32_bf16 operands (w is the A
//    operand, x^T the B operand); the waves' partial sums meet in LDS.  No split-K workspace,
//    no atomics: the order of the sums is fixed.
//  * tiled (M > 16): 128x128x64 or 256x256x64 workgroup tiles (64x128x64 with K cut into shares
//    and a reduction kernel for 16 < M <= 64, where whole-K tiles would leave CUs idle) that go from global
//    memory straight into a ring of LDS stages, 4 waves built from v_mfma_f32_32x32x16_bf16 with
//    hand-pipelined operand reads.  Workgroups are renumbered so that each XCD's L2 sees
//    neighbouring tiles.
//
// The reference's linear kernel computes the same product with one thread per output element
// and no matrix instruction (src/kernels/linear.cu:7-56).
#include "common.h"

namespace lc {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

template <typename TO> __device__ __forceinline__ void store_out(TO* p, float v);
template <> __device__ __forceinline__ void store_out<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_out<bf16>(bf16* p, float v) { *p = static_cast<bf16>(v); }

// silu(g) * u with silu(g) = g / (1 + exp(-g))   (reference: src/kernels/swiglu.cu:8,31-35)
__device__ __forceinline__ float swiglu_f(float g, float u) { return g / (1.f + expf(-g)) * u; }

// ------------------------------------------------------------------------------- skinny
constexpr int SK_KBLOCK = 128; // k elements per wave iteration

// MT: tiles of 16 rows of x; NT: tiles of 16 rows of w per workgroup; the WAVES waves of a
// workgroup take the k blocks in turn.
template <int MT, int NT, int WAVES, int UNROLL, int EPI, typename TO>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16* __restrict__ x,
                                                                 const bf16* __restrict__ w,
                                                                 TO* __restrict__ out, int M, int N,
                                                                 int K) {
    __shared__ float red[WAVES * MT * NT * 256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * (16 * NT);
    const bf16* wp[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) wp[nt] = w + (size_t)min(n0 + nt * 16 + r, N - 1) * K + g * 8;
    const bf16* xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xp[mt] = x + (size_t)min(mt * 16 + r, M - 1) * K + g * 8;

    floatx4 acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int kblocks = K / SK_KBLOCK;
#pragma unroll UNROLL
    for (int kb = wave; kb < kblocks; kb += WAVES) {
        const int k0 = kb * SK_KBLOCK;
        bf16x8 a[NT][4];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int j = 0; j < 4; ++j) a[nt][j] = *reinterpret_cast<const bf16x8*>(wp[nt] + k0 + j * 32);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            bf16x8 b[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = *reinterpret_cast<const bf16x8*>(xp[mt] + k0 + j * 32);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt][j], b[j], acc[nt][mt], 0, 0, 0);
        }
    }
    // acc[nt][mt][v] = partial out[m = mt*16 + lane%16][n = n0 + nt*16 + (lane/16)*4 + v]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int v = 0; v < 4; ++v)
                red[((wave * NT + nt) * MT + mt) * 256 + v * 64 + lane] = acc[nt][mt][v];
    __syncthreads();
    if (EPI == 0) {
        for (int idx = threadIdx.x; idx < NT * MT * 256; idx += WAVES * 64) {
            float total = 0.f;
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) total += red[wv * NT * MT * 256 + idx];
            const int tile = idx >> 8, v = (idx >> 6) & 3, l = idx & 63;
            const int nt = tile / MT, mt = tile % MT;
            const int m = mt * 16 + (l & 15), n = n0 + nt * 16 + (l >> 4) * 4 + v;
            if (m < M && n < N) store_out<TO>(out + (size_t)m * N + n, total);
        }
    } else {
        // rows of w come in blocks of 16: 8 gate rows, then their 8 up rows; out has N / 2 columns
        for (int idx = threadIdx.x; idx < NT * MT * 128; idx += WAVES * 64) {
            const int tile = idx >> 7, v = (idx >> 5) & 3, l = idx & 31;   // l: lane of the gate half
            const int gi = tile * 256 + v * 64 + l, ui = gi + 32;
            float g = 0.f, u = 0.f;
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) {
                g += red[wv * NT * MT * 256 + gi];
                u += red[wv * NT * MT * 256 + ui];
            }
            const int nt = tile / MT, mt = tile % MT;
            const int m = mt * 16 + (l & 15), n = n0 + nt * 16 + (l >> 4) * 4 + v;   // gate row, n % 16 < 8
            const int col = (n >> 4) * 8 + (n & 7);
            if (m < M && n < N) store_out<TO>(out + (size_t)m * (N / 2) + col, swiglu_f(g, u));
        }
    }
}

// ------------------------------------------------------------------------------- tiled
// Workgroup tile BM x BN x 64, four waves in a 2 x 2 grid, each owning (BM/64) x (BN/64) tiles
// of 32 x 32.  128 x 128 (two workgroups to a CU) for most shapes, 256 x 256 where the grid
// still has two tiles per CU: it halves the bytes that cross the L2 per product.
//
// Operand tiles go from global memory straight into LDS (global_load_lds_dwordx4: lane l's 16
// bytes land at the instruction's LDS base + 16 l, no registers in between) into a ring of
// TL_STAGES stages; a stage is filled while the one before it is multiplied.  Inside a stage
// a row's eight 16-byte chunks are stored at column (chunk ^ (row & 7)), which spreads the 32
// rows of an operand read over all banks without padding.  The LDS reads are written by hand
// (ds_read_b128 + explicit waits), two k-steps deep, for two reasons: the products of one
// k-step then hide the reads of the next although a SIMD may hold a single wave, and the
// compiler, which cannot tell the stages apart, would otherwise make every load in flight
// land before any read.  Likewise the barrier is the bare instruction: each wave first waits
// for its own loads of the stage, the barrier then makes all waves' loads visible.
constexpr int TL_K = 64;
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) const void* glb_ptr_t;

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));   // other counters untouched
}
template <int N> __device__ __forceinline__ void wait_lgkmcnt() {
    __builtin_amdgcn_s_waitcnt(0xC07F | (N << 8));
}

// SPLIT: blockIdx.y owns a share of the k-blocks and writes its float32 partial sums to
// part[blockIdx.y][M][N]; splitk_reduce_kernel adds the shares in a fixed order.
template <int BM, int BN, int TL_STAGES, int EPI, bool SPLIT, typename TO>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const bf16* __restrict__ x,
                                                         const bf16* __restrict__ w,
                                                         TO* __restrict__ out, float* __restrict__ part,
                                                         int M, int N, int K, int tiles_m, int tiles_n) {
    constexpr int TM = BM / 64, TN = BN / 64;
    constexpr int LPA = BM * 8 / 256, LPB = BN * 8 / 256;   // load instructions per thread and stage
    __shared__ __attribute__((aligned(16))) bf16 As[TL_STAGES][BM * TL_K];
    __shared__ __attribute__((aligned(16))) bf16 Bs[TL_STAGES][BN * TL_K];

    // renumber: workgroups go round-robin over 8 XCDs; give each XCD a contiguous run of
    // tiles, m fastest, so that one XCD's L2 keeps the w tile that its workgroups share
    const int total = tiles_m * tiles_n;
    int id = blockIdx.x;
    {
        const int q = total >> 3, rem = total & 7;
        const int xcd = id & 7, local = id >> 3;
        id = xcd * q + min(xcd, rem) + local;   // a bijection of [0, total) for any total
    }
    const int tm = id % tiles_m, tn = id / tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * (BM / 2), wn = (wave & 1) * (BN / 2);
    const int lr = lane & 31, kg = lane >> 5;

    // chunk p = (i * 4 + wave) * 64 + lane of a stage holds row p / 8, global column (p % 8) ^ (row & 7)
    const bf16* xg[LPA];
    const bf16* wg[LPB];
#pragma unroll
    for (int i = 0; i < LPA; ++i) {
        const int p = (i * 4 + wave) * 64 + lane, row = p >> 3, kc = (p & 7) ^ (row & 7);
        xg[i] = x + (size_t)min(m0 + row, M - 1) * K + kc * 8;
    }
#pragma unroll
    for (int i = 0; i < LPB; ++i) {
        const int p = (i * 4 + wave) * 64 + lane, row = p >> 3, kc = (p & 7) ^ (row & 7);
        wg[i] = w + (size_t)min(n0 + row, N - 1) * K + kc * 8;
    }
    auto issue = [&](int kb, int stage) {
#pragma unroll
        for (int i = 0; i < LPA; ++i)
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(xg[i] + kb * TL_K),
                                             (lds_ptr_t)(&As[stage][(i * 4 + wave) * 512]), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < LPB; ++i)
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(wg[i] + kb * TL_K),
                                             (lds_ptr_t)(&Bs[stage][(i * 4 + wave) * 512]), 16, 0, 0);
    };
    const int nk_all = K / TL_K;
    const int kb0 = SPLIT ? (int)((long long)blockIdx.y * nk_all / gridDim.y) : 0;
    const int nk = (SPLIT ? (int)((long long)(blockIdx.y + 1) * nk_all / gridDim.y) : nk_all) - kb0;
#pragma unroll
    for (int s = 0; s < TL_STAGES - 1; ++s)
        if (s < nk) issue(kb0 + s, s);

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // byte offsets of this lane's operand rows inside a stage, and their swizzles
    unsigned arow[TM], brow[TN];
    int asw[TM], bsw[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) { const int row = wm + i * 32 + lr; arow[i] = row * 128; asw[i] = row & 7; }
#pragma unroll
    for (int j = 0; j < TN; ++j) { const int row = wn + j * 32 + lr; brow[j] = row * 128; bsw[j] = row & 7; }

    for (int it = 0; it < nk; ++it) {
        // block `it` has landed when at most the younger blocks' loads are still in flight
        if (it + TL_STAGES - 2 < nk) wait_vmcnt<(TL_STAGES - 2) * (LPA + LPB)>(); else wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        if (it + TL_STAGES - 1 < nk) issue(kb0 + it + TL_STAGES - 1, (it + TL_STAGES - 1) % TL_STAGES);
        const unsigned abase = (unsigned)(uintptr_t)(lds_ptr_t)As[it % TL_STAGES];
        const unsigned bbase = (unsigned)(uintptr_t)(lds_ptr_t)Bs[it % TL_STAGES];
        bf16x8 a[2][TM], b[2][TN];
        auto read = [&](int ks, int buf) {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const unsigned addr = abase + arow[i] + (((ks * 2 + kg) ^ asw[i]) * 16);
                asm volatile("ds_read_b128 %0, %1" : "=v"(a[buf][i]) : "v"(addr));
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const unsigned addr = bbase + brow[j] + (((ks * 2 + kg) ^ bsw[j]) * 16);
                asm volatile("ds_read_b128 %0, %1" : "=v"(b[buf][j]) : "v"(addr));
            }
        };
        read(0, 0);
#pragma unroll
        for (int ks = 0; ks < TL_K / 16; ++ks) {
            if (ks + 1 < TL_K / 16) {
                read(ks + 1, (ks + 1) & 1);
                wait_lgkmcnt<TM + TN>();       // this k-step's operands are in; the next one's may be out
            } else {
                wait_lgkmcnt<0>();
            }
            // the products below must not be moved above the wait: tie their operands to this point
#pragma unroll
            for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(a[ks & 1][i]));
#pragma unroll
            for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(b[ks & 1][j]));
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[ks & 1][i], b[ks & 1][j], acc[i][j], 0, 0, 0);
        }
    }
    // acc[i][j][v]: row m = (v/4)*8 + (lane/32)*4 + v%4, column n = lane%32 of the 32x32 tile
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn + j * 32 + lr;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + wm + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                if (SPLIT) {
                    if (m < M && n < N) part[((size_t)blockIdx.y * M + m) * N + n] = acc[i][j][v];
                } else if (EPI == 0) {
                    if (m < M && n < N) store_out<TO>(out + (size_t)m * N + n, acc[i][j][v]);
                } else {
                    // columns come in blocks of 16: 8 gate, then their 8 up (8 lanes further on)
                    const float other = __shfl_xor(acc[i][j][v], 8, 64);
                    if ((lr & 8) == 0 && m < M && n < N)
                        store_out<TO>(out + (size_t)m * (N / 2) + (n >> 4) * 8 + (n & 7),
                                      swiglu_f(acc[i][j][v], other));
                }
            }
        }
}

// out = sum over the shares of part[s][M][N], added in the order of s; EPI as in the products
template <int EPI, typename TO>
__global__ void splitk_reduce_kernel(const float* __restrict__ part, TO* __restrict__ out, int M, int N,
                                     int S) {
    const size_t MN = (size_t)M * N;
    if (EPI == 0) {
        for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < MN;
             idx += (size_t)gridDim.x * blockDim.x) {
            float t = 0.f;
            for (int s = 0; s < S; ++s) t += part[s * MN + idx];
            store_out<TO>(out + idx, t);
        }
    } else {
        const int half = N / 2;
        for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < (size_t)M * half;
             idx += (size_t)gridDim.x * blockDim.x) {
            const size_t m = idx / half;
            const int c = (int)(idx - m * half);
            const size_t gi = m * N + (size_t)(c >> 3) * 16 + (c & 7);
            float g = 0.f, u = 0.f;
            for (int s = 0; s < S; ++s) { g += part[s * MN + gi]; u += part[s * MN + gi + 8]; }
            store_out<TO>(out + idx, swiglu_f(g, u));
        }
    }
}

// How many shares of K the product of these sizes is cut into (1: no workspace needed): as
// many as it takes to give every CU a workgroup when whole-K tiles would be too few.
static int splitk_shares(int M, int N, int K) {
    if (M <= 16) return 1;
    const int tiles = M <= 64 ? (N + 127) / 128 : ((M + 127) / 128) * ((N + 127) / 128);
    if (tiles >= 200) return 1;
    const int nk = K / TL_K;
    int S = (320 + tiles / 2) / tiles;
    if (S > nk / 4) S = nk / 4;
    return S < 1 ? 1 : S;
}

template <int MT, int NT, int WAVES, int UNROLL, int EPI, typename TO>
static void launch_skinny(const bf16* x, const bf16* w, TO* out, int M, int N, int K, hipStream_t s) {
    const int rows = 16 * NT;
    gemm_skinny_kernel<MT, NT, WAVES, UNROLL, EPI, TO><<<(N + rows - 1) / rows, WAVES * 64, 0, s>>>(x, w, out, M, N, K);
}

template <int EPI, typename TO>
static int launch_bf16(const bf16* x, const bf16* w, TO* out, float* workspace, int M, int N, int K,
                       hipStream_t s) {
    if (M <= 16) {
        launch_skinny<1, 1, 16, 2, EPI, TO>(x, w, out, M, N, K, s);
        LC_LAUNCH_CHECK("gemm_skinny");
    } else if (M <= 64) {
        // 64 x 128 tiles, K cut into shares so that every CU has a workgroup
        const int S = splitk_shares(M, N, K), tiles_n = (N + 127) / 128;
        if (S == 1) {
            gemm_tiled_kernel<64, 128, 4, EPI, false, TO><<<tiles_n, 256, 0, s>>>(x, w, out, nullptr, M, N, K, 1, tiles_n);
            LC_LAUNCH_CHECK("gemm_tiled");
        } else {
            LC_CHECK(workspace, "gemm_bf16: M=%d N=%d K=%d needs a workspace", M, N, K);
            gemm_tiled_kernel<64, 128, 4, 0, true, TO><<<dim3(tiles_n, S), 256, 0, s>>>(x, w, out, workspace, M, N, K, 1, tiles_n);
            LC_LAUNCH_CHECK("gemm_tiled");
            const size_t work = EPI ? (size_t)M * N / 2 : (size_t)M * N;
            splitk_reduce_kernel<EPI, TO><<<(int)((work + 255) / 256), 256, 0, s>>>(workspace, out, M, N, S);
            LC_LAUNCH_CHECK("splitk_reduce");
        }
    } else {
        const int big_m = (M + 255) / 256, big_n = (N + 255) / 256;
        const int tiles_m = (M + 127) / 128, tiles_n = (N + 127) / 128;
        const int S = splitk_shares(M, N, K);
        if (S > 1) {
            LC_CHECK(workspace, "gemm_bf16: M=%d N=%d K=%d needs a workspace", M, N, K);
            gemm_tiled_kernel<128, 128, 2, 0, true, TO><<<dim3(tiles_m * tiles_n, S), 256, 0, s>>>(
                x, w, out, workspace, M, N, K, tiles_m, tiles_n);
            LC_LAUNCH_CHECK("gemm_tiled");
            const size_t work = EPI ? (size_t)M * N / 2 : (size_t)M * N;
            splitk_reduce_kernel<EPI, TO><<<(int)((work + 255) / 256), 256, 0, s>>>(workspace, out, M, N, S);
            LC_LAUNCH_CHECK("splitk_reduce");
            return 0;
        }
        if ((long long)big_m * big_n >= 512) {
            gemm_tiled_kernel<256, 256, 2, EPI, false, TO><<<big_m * big_n, 256, 0, s>>>(x, w, out, nullptr, M, N, K, big_m, big_n);
        } else {
            gemm_tiled_kernel<128, 128, 2, EPI, false, TO><<<tiles_m * tiles_n, 256, 0, s>>>(x, w, out, nullptr, M, N, K, tiles_m, tiles_n);
        }
        LC_LAUNCH_CHECK("gemm_tiled");
    }
    return 0;
}

}  // namespace lc

using namespace lc;

// Sizes the matrix-core kernels take; everything else goes to the generic kernel.
LC_API int lc_gemm_bf16_supported(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    if (K % SK_KBLOCK != 0) return 0;
    if ((size_t)((M + 127) / 128) * ((N + 127) / 128) > 0x7fffffffu) return 0;
    return 1;
}

// float32 words of workspace that lc_gemm_bf16 needs for these sizes (0: none).
LC_API long long lc_gemm_bf16_workspace(int M, int N, int K) {
    if (!lc_gemm_bf16_supported(M, N, K)) return 0;
    const int S = splitk_shares(M, N, K);
    return S > 1 ? (long long)S * M * N : 0;
}

// epilogue 0: out[M, N] = x . w^T.  epilogue 1 (SwiGLU): the rows of w come in blocks of 16,
// 8 gate rows followed by their 8 up rows; out[M, N / 2] = silu(gate) * up.
// workspace: lc_gemm_bf16_workspace(M, N, K) float32 words (may be null when that is 0).
LC_API int lc_gemm_bf16(const void* x, const void* w, void* out, int out_dt, int M, int N, int K,
                        int epilogue, float* workspace, hipStream_t stream) {
    LC_CHECK(lc_gemm_bf16_supported(M, N, K), "gemm_bf16: sizes M=%d N=%d K=%d are not supported "
             "(K must be a multiple of %d)", M, N, K, SK_KBLOCK);
    LC_CHECK(x && w && out, "gemm_bf16: null pointer");
    LC_CHECK(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_bf16: operands must be 16-byte aligned");
    LC_CHECK(epilogue == 0 || (epilogue == 1 && N % 16 == 0),
             "gemm_bf16: the SwiGLU epilogue needs N (%d) to be a multiple of 16", N);
    const bf16* xb = (const bf16*)x;
    const bf16* wb = (const bf16*)w;
    if (out_dt == DT_BF16)
        return epilogue ? launch_bf16<1, bf16>(xb, wb, (bf16*)out, workspace, M, N, K, stream)
                        : launch_bf16<0, bf16>(xb, wb, (bf16*)out, workspace, M, N, K, stream);
    if (out_dt == DT_F32)
        return epilogue ? launch_bf16<1, float>(xb, wb, (float*)out, workspace, M, N, K, stream)
                        : launch_bf16<0, float>(xb, wb, (float*)out, workspace, M, N, K, stream);
    LC_CHECK(false, "gemm_bf16: unknown output dtype %d", out_dt);
    return 0;
}
