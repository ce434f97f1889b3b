// out[M, N] = x[M, K] . w[N, K]^T for any sizes and any mix of float32 / bfloat16 operands, as a
// true 32-bit product: the operands are widened to float32 and multiplied on the matrix cores in
// float32 (v_mfma_f32_16x16x4_f32: float32 products, float32 sums, no reduced-precision mode).
// The weight layout is the checkpoint's: [out_features, in_features] row-major, applied as
// y = x . W^T without bias (reference: src/kernels/linear.cu:24-27, one thread per output
// element; here tiles of 128 x 128, 64 x 64 or, for up to 16 rows, 16 x 64, staged through LDS
// 16 k at a time, four waves with a grid of 16 x 16 products each).
//
// The order of the additions is a function of the output element alone: K is cut into chunks of
// 256; within a chunk the element's sum takes four k at a time, in order (one matrix
// instruction each, the same in every tile shape), and the chunks' sums are added one after the
// other from 0.  With few tiles (a decode step: up to 64 rows and a narrow N) the chunks are
// shared out over workgroups, which leave their sums in a workspace, and a second kernel adds
// them in the same order: a row's result has the same bits whether it is computed alone or
// among thousands.
#include "common.h"

namespace lc {

constexpr int GB_M = 64, GB_N = 64, GB_K = 16;
constexpr int GB_CHUNK = 256;   // k elements whose products are added up before they join the total
constexpr int GB_PAD = 16;      // a row of a stage is its tile's rows and 16 floats: the four k that a wave reads
                                // at once (16 lanes each) then lie in different banks
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Tile BM x BN, WM x WN waves, each with (BM / 16 / WM) x (BN / 16 / WN) products of 16 x 16.
// part == nullptr: out = x . w^T.  Else blockIdx.z owns the chunks [z * per, (z + 1) * per) and
// writes each chunk's sums to part[chunk][M][N].
template <typename TX, typename TW, typename TO, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(256, 2) void gemm_generic_kernel(const TX* __restrict__ x,
                                                           const TW* __restrict__ w,
                                                           TO* __restrict__ out, int M, int N,
                                                           int K, float* __restrict__ part, int per) {
    static_assert(WM * WN == 4, "four waves");
    constexpr int TM = BM / 16 / WM, TN = BN / 16 / WN;
    constexpr int XL = (BM * 4 + 255) / 256, WL = (BN * 4 + 255) / 256;   // 16-byte pieces a thread loads per stage
    __shared__ float xs[2][GB_K][BM + GB_PAD];     // two stages: one is filled while the other is multiplied
    __shared__ float ws[2][GB_K][BN + GB_PAD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int wm = (wave / WN) * (BM / WM), wn = (wave % WN) * (BN / WN);
    const int chunks = (K + GB_CHUNK - 1) / GB_CHUNK;
    const int c_begin = part ? blockIdx.z * per : 0;
    const int c_end = part ? min(c_begin + per, chunks) : chunks;
    floatx4 total[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) total[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    // loader mapping: rows x 16 k; a thread loads 4 consecutive k of a row (of up to XL rows of x
    // and WL of w, 64 apart), a step ahead of the products that use them (the loads of step
    // k0 + 16 are in flight while step k0 is multiplied)
    const int lrow = tid / 4, lk = (tid % 4) * 4;
    // whole 16-byte (8-byte) pieces where the row length allows it
    const bool vec = (K & 3) == 0 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0);
    float xr[XL][4], wr[WL][4];
    auto fetch_rows = [&](auto* rows_ptr, int first, int limit, int tile_rows, int count, float (*dst)[4], int k0) {
#pragma unroll
        for (int u = 0; u < count; ++u) {
            const int row = lrow + 64 * u;
            const bool live = row < tile_rows && first + row < limit;
            const auto* p = rows_ptr + (size_t)min(first + row, limit - 1) * K + lk;
            if (vec && k0 + lk + 3 < K) {
                load4(dst[u], p + k0);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) dst[u][j] = k0 + lk + j < K ? to_f32(p[k0 + j]) : 0.f;
            }
            if (!live) { dst[u][0] = dst[u][1] = dst[u][2] = dst[u][3] = 0.f; }
        }
    };
    auto fetch = [&](int k0) {
        fetch_rows(x, m0, M, BM, XL, xr, k0);
        fetch_rows(w, n0, N, BN, WL, wr, k0);
    };
    auto put = [&](int stage) {
#pragma unroll
        for (int u = 0; u < XL; ++u)
            if (lrow + 64 * u < BM)
#pragma unroll
                for (int j = 0; j < 4; ++j) xs[stage][lk + j][lrow + 64 * u] = xr[u][j];
#pragma unroll
        for (int u = 0; u < WL; ++u)
            if (lrow + 64 * u < BN)
#pragma unroll
                for (int j = 0; j < 4; ++j) ws[stage][lk + j][lrow + 64 * u] = wr[u][j];
    };
    // every step of 16 k, over all of this workgroup's chunks, is a stage: stage s is written to
    // LDS while stage s - 1 is multiplied, one barrier a stage
    int stage = 0;
    if (c_begin < c_end) {
        fetch(c_begin * GB_CHUNK);
        put(0);
    }
    for (int c = c_begin; c < c_end; ++c) {
        floatx4 acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
        const int k_end = min(K, (c + 1) * GB_CHUNK);
        for (int k0 = c * GB_CHUNK; k0 < k_end; k0 += GB_K) {
            __syncthreads();            // this stage is written; the other has been read by everybody
            const int next = k0 + GB_K;
            const bool more = next < k_end || c + 1 < c_end;
            if (more) fetch(next < k_end ? next : (c + 1) * GB_CHUNK);
            // lane l brings x[row l % 16][k l / 16] of each of its tiles, and w likewise; all of
            // the stage's operands are asked for before the first product
            float a[4][TM], b[4][TN];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int i = 0; i < TM; ++i) a[q][i] = xs[stage][4 * q + (lane >> 4)][wm + 16 * i + (lane & 15)];
#pragma unroll
                for (int j = 0; j < TN; ++j) b[q][j] = ws[stage][4 * q + (lane >> 4)][wn + 16 * j + (lane & 15)];
            }
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[q][i], b[q][j], acc[i][j], 0, 0, 0);
            stage ^= 1;
            if (more) put(stage);
        }
        // lane l holds the rows 4 (l / 16) + r and the column l % 16 of each of its tiles
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (part) {
                        const int m = m0 + wm + 16 * i + 4 * (lane >> 4) + r, n = n0 + wn + 16 * j + (lane & 15);
                        if (m < M && n < N) part[((size_t)c * M + m) * N + n] = acc[i][j][r];
                    } else {
                        total[i][j][r] = __fadd_rn(total[i][j][r], acc[i][j][r]);
                    }
                }
    }
    if (part) return;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + wm + 16 * i + 4 * (lane >> 4) + r, n = n0 + wn + 16 * j + (lane & 15);
                if (m < M && n < N) out[(size_t)m * N + n] = from_f32<TO>(total[i][j][r]);
            }
}

constexpr int GF_M = 16;        // rows of the tile for a decode step's few rows

// out = the chunks' sums part[c][M][N] added one after the other from 0, as the kernel above
// adds them when it keeps them to itself
template <typename TO>
__global__ void gemm_generic_sum_kernel(const float* __restrict__ part, TO* __restrict__ out, size_t MN,
                                        int chunks) {
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < MN;
         idx += (size_t)gridDim.x * blockDim.x) {
        float total = 0.f;
        for (int c = 0; c < chunks; ++c) total = __fadd_rn(total, part[(size_t)c * MN + idx]);
        out[idx] = from_f32<TO>(total);
    }
}

// Chunks a workgroup takes when they are shared out (0: they are not): with fewer than 1024
// tiles, as many workgroups as it takes to have about 2048, if the workspace stays modest.
static int chunks_per_workgroup(int M, int N, int K) {
    const long long tiles = (long long)((N + GB_N - 1) / GB_N) * ((M + GB_M - 1) / GB_M);
    const int chunks = (K + GB_CHUNK - 1) / GB_CHUNK;
    if (tiles >= 1024 || chunks < 2) return 0;
    // the workspace holds every chunk's sums for all of M x N: no more than 64 M floats (256 MiB),
    // beyond which the chunks stay with their tile (the same additions in the same order)
    if ((long long)chunks * M * N > (64ll << 20)) return 0;
    long long shares = (2048 + tiles - 1) / tiles;
    if (shares > chunks) shares = chunks;
    if (shares < 2) return 0;
    return (int)((chunks + shares - 1) / shares);
}

template <typename TX, typename TW, typename TO>
static int launch_generic(const void* x, const void* w, void* out, int M, int N, int K, float* workspace,
                          hipStream_t stream) {
    const int per = chunks_per_workgroup(M, N, K);
    const int chunks = (K + GB_CHUNK - 1) / GB_CHUNK;
    const bool few = M <= GF_M;
    // tiles of 128 x 128 where they fill the card (they bring half as many bytes into a CU per product)
    const bool large = per == 0 && M > GB_M && (long long)((N + 127) / 128) * ((M + 127) / 128) >= device_cus();
    float* part = nullptr;
    int shares = 1;
    if (per > 0) {
        LC_CHECK(workspace, "gemm: M=%d N=%d K=%d needs a workspace", M, N, K);
        part = workspace;
        shares = (chunks + per - 1) / per;
    }
    if (few) {
        dim3 grid((N + GB_N - 1) / GB_N, 1, shares);
        gemm_generic_kernel<TX, TW, TO, GF_M, GB_N, 1, 4><<<grid, 256, 0, stream>>>(
            (const TX*)x, (const TW*)w, (TO*)out, M, N, K, part, per);
    } else if (large) {
        dim3 grid((N + 127) / 128, (M + 127) / 128, 1);
        gemm_generic_kernel<TX, TW, TO, 128, 128, 2, 2><<<grid, 256, 0, stream>>>(
            (const TX*)x, (const TW*)w, (TO*)out, M, N, K, nullptr, 0);
    } else {
        dim3 grid((N + GB_N - 1) / GB_N, (M + GB_M - 1) / GB_M, shares);
        gemm_generic_kernel<TX, TW, TO, GB_M, GB_N, 2, 2><<<grid, 256, 0, stream>>>(
            (const TX*)x, (const TW*)w, (TO*)out, M, N, K, part, per);
    }
    LC_LAUNCH_CHECK("gemm_generic");
    if (per > 0) {
        const size_t MN = (size_t)M * N;
        gemm_generic_sum_kernel<TO><<<(int)((MN + 255) / 256 < 4096 ? (MN + 255) / 256 : 4096), 256, 0, stream>>>(
            workspace, (TO*)out, MN, chunks);
        LC_LAUNCH_CHECK("gemm_generic_sum");
    }
    return 0;
}

}  // namespace lc

using namespace lc;

// float32 words of workspace that lc_gemm_generic needs for these sizes (0: none)
LC_API long long lc_gemm_generic_workspace(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    return chunks_per_workgroup(M, N, K) > 0 ? (long long)((K + GB_CHUNK - 1) / GB_CHUNK) * M * N : 0;
}

LC_API int lc_gemm_generic(const void* x, int x_dt, const void* w, int w_dt, void* out, int out_dt,
                           int M, int N, int K, float* workspace, hipStream_t stream) {
    LC_CHECK(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    if (M == 0) return 0;
    LC_CHECK(x && w && out, "gemm: null pointer");
    LC_CHECK((size_t)((M + GB_M - 1) / GB_M) <= 65535, "gemm: M=%d is too large", M);
    const int key = x_dt * 4 + w_dt * 2 + out_dt;
    switch (key) {
        case 0: return launch_generic<float, float, float>(x, w, out, M, N, K, workspace, stream);
        case 2: return launch_generic<float, bf16, float>(x, w, out, M, N, K, workspace, stream);
        case 4: return launch_generic<bf16, float, float>(x, w, out, M, N, K, workspace, stream);
        case 5: return launch_generic<bf16, float, bf16>(x, w, out, M, N, K, workspace, stream);
        case 6: return launch_generic<bf16, bf16, float>(x, w, out, M, N, K, workspace, stream);
        case 7: return launch_generic<bf16, bf16, bf16>(x, w, out, M, N, K, workspace, stream);
        default:
            LC_CHECK(false, "gemm: unsupported dtypes x=%d w=%d out=%d", x_dt, w_dt, out_dt);
    }
    return 0;
}
