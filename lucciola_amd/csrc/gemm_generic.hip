// out[M, N] = x[M, K] . w[N, K]^T for any sizes and any mix of float32 / bfloat16 operands,
// accumulated with float32 FMAs (no matrix-core instruction, so that with float32 operands it
// is a true 32-bit product).  The weight layout is the checkpoint's: [out_features,
// in_features] row-major, applied as y = x . W^T without bias (reference:
// src/kernels/linear.cu:24-27, one thread per output element; here LDS-tiled 64x64x16 with a
// 4x4 register tile per thread; up to 16 rows: 16x64x16 with four rows of a column per thread).
//
// The order of the additions is a function of the output element alone: K is cut into chunks of
// 256; within a chunk the products are added one after the other from 0, and the chunks' sums
// are added one after the other from 0.  With few tiles (a decode step: up to 64 rows and a
// narrow N) the chunks are shared out over workgroups, which leave their sums in a workspace,
// and a second kernel adds them in the same order: a row's result has the same bits whether it
// is computed alone or among thousands.
#include "common.h"

namespace lc {

constexpr int GB_M = 64, GB_N = 64, GB_K = 16;
constexpr int GB_CHUNK = 256;   // k elements whose products are added up before they join the total

// part == nullptr: out = x . w^T.  Else blockIdx.z owns the chunks [z * per, (z + 1) * per) and
// writes each chunk's sums to part[chunk][M][N].
template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TX* __restrict__ x,
                                                           const TW* __restrict__ w,
                                                           TO* __restrict__ out, int M, int N,
                                                           int K, float* __restrict__ part, int per) {
    __shared__ float xs[GB_K][GB_M + 4];
    __shared__ float ws[GB_K][GB_N + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * GB_M, n0 = blockIdx.x * GB_N;
    const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
    const int chunks = (K + GB_CHUNK - 1) / GB_CHUNK;
    const int c_begin = part ? blockIdx.z * per : 0;
    const int c_end = part ? min(c_begin + per, chunks) : chunks;
    float total[4][4] = {};

    // loader mapping: 64 rows x 16 k; a thread loads 4 consecutive k of one row of x and of w,
    // a step ahead of the products that use them (the loads of step k0 + 16 are in flight while
    // step k0 is multiplied)
    const int lrow = tid / 4, lk = (tid % 4) * 4;
    const bool x_row = m0 + lrow < M, w_row = n0 + lrow < N;
    const TX* xp = x + (size_t)min(m0 + lrow, M - 1) * K + lk;
    const TW* wp = w + (size_t)min(n0 + lrow, N - 1) * K + lk;
    // whole 16-byte (8-byte) pieces where the row length allows it
    const bool vec = (K & 3) == 0 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0);
    float xr[4], wr[4];
    auto fetch = [&](int k0) {
        if (vec && k0 + lk + 3 < K) {
            load4(xr, xp + k0);
            load4(wr, wp + k0);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int k = k0 + lk + j;
                xr[j] = k < K ? to_f32(xp[k0 + j]) : 0.f;
                wr[j] = k < K ? to_f32(wp[k0 + j]) : 0.f;
            }
        }
        if (!x_row) { xr[0] = xr[1] = xr[2] = xr[3] = 0.f; }
        if (!w_row) { wr[0] = wr[1] = wr[2] = wr[3] = 0.f; }
    };
    if (c_begin < c_end) fetch(c_begin * GB_CHUNK);
    for (int c = c_begin; c < c_end; ++c) {
        float acc[4][4] = {};
        const int k_end = min(K, (c + 1) * GB_CHUNK);
        for (int k0 = c * GB_CHUNK; k0 < k_end; k0 += GB_K) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                xs[lk + j][lrow] = xr[j];
                ws[lk + j][lrow] = wr[j];
            }
            __syncthreads();
            {   // the step after this one, which may be the first of the next chunk
                const int next = k0 + GB_K;
                if (next < k_end || c + 1 < c_end) fetch(next < k_end ? next : (c + 1) * GB_CHUNK);
            }
#pragma unroll
            for (int kk = 0; kk < GB_K; ++kk) {
                float a[4], b[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) a[i] = xs[kk][tm + i];
#pragma unroll
                for (int j = 0; j < 4; ++j) b[j] = ws[kk][tn + j];
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
            }
            __syncthreads();
        }
        if (part) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = m0 + tm + i;
                if (m >= M) continue;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int n = n0 + tn + j;
                    if (n < N) part[((size_t)c * M + m) * N + n] = acc[i][j];
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) total[i][j] = __fadd_rn(total[i][j], acc[i][j]);
        }
    }
    if (part) return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + tm + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tn + j;
            if (n < N) out[(size_t)m * N + n] = from_f32<TO>(total[i][j]);
        }
    }
}

// The same product for up to 16 rows of x (a decode step): tiles of 16 x 64, a thread owns four
// rows of one column and reads four k of both operands at a time.  Every output element sees
// the same operations in the same order as in the kernel above.
constexpr int GF_M = 16;

template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void gemm_generic_few_kernel(const TX* __restrict__ x,
                                                               const TW* __restrict__ w,
                                                               TO* __restrict__ out, int M, int N,
                                                               int K, float* __restrict__ part, int per) {
    __shared__ __align__(16) float xs[GF_M][GB_K];
    __shared__ __align__(16) float ws[GB_N][GB_K + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * GF_M, n0 = blockIdx.x * GB_N;
    const int tn = tid % GB_N, tm = (tid / GB_N) * 4;
    const int chunks = (K + GB_CHUNK - 1) / GB_CHUNK;
    const int c_begin = part ? blockIdx.z * per : 0;
    const int c_end = part ? min(c_begin + per, chunks) : chunks;
    float total[4] = {};

    const int lrow = tid / 4, lk = (tid % 4) * 4;
    const bool x_loader = lrow < GF_M, x_row = x_loader && m0 + lrow < M, w_row = n0 + lrow < N;
    const TX* xp = x + (size_t)min(m0 + lrow, M - 1) * K + lk;
    const TW* wp = w + (size_t)min(n0 + lrow, N - 1) * K + lk;
    const bool vec = (K & 3) == 0 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0);
    float xr[4] = {}, wr[4];
    auto fetch = [&](int k0) {
        if (vec && k0 + lk + 3 < K) {
            if (x_row) load4(xr, xp + k0);
            load4(wr, wp + k0);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int k = k0 + lk + j;
                xr[j] = (x_row && k < K) ? to_f32(xp[k0 + j]) : 0.f;
                wr[j] = k < K ? to_f32(wp[k0 + j]) : 0.f;
            }
        }
        if (!x_row) { xr[0] = xr[1] = xr[2] = xr[3] = 0.f; }
        if (!w_row) { wr[0] = wr[1] = wr[2] = wr[3] = 0.f; }
    };
    if (c_begin < c_end) fetch(c_begin * GB_CHUNK);
    for (int c = c_begin; c < c_end; ++c) {
        float acc[4] = {};
        const int k_end = min(K, (c + 1) * GB_CHUNK);
        for (int k0 = c * GB_CHUNK; k0 < k_end; k0 += GB_K) {
            if (x_loader) *reinterpret_cast<float4*>(&xs[lrow][lk]) = make_float4(xr[0], xr[1], xr[2], xr[3]);
            *reinterpret_cast<float4*>(&ws[lrow][lk]) = make_float4(wr[0], wr[1], wr[2], wr[3]);
            __syncthreads();
            {
                const int next = k0 + GB_K;
                if (next < k_end || c + 1 < c_end) fetch(next < k_end ? next : (c + 1) * GB_CHUNK);
            }
#pragma unroll
            for (int kk = 0; kk < GB_K; kk += 4) {
                const float4 b = *reinterpret_cast<const float4*>(&ws[tn][kk]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float4 a = *reinterpret_cast<const float4*>(&xs[tm + i][kk]);
                    acc[i] = fmaf(a.x, b.x, acc[i]);
                    acc[i] = fmaf(a.y, b.y, acc[i]);
                    acc[i] = fmaf(a.z, b.z, acc[i]);
                    acc[i] = fmaf(a.w, b.w, acc[i]);
                }
            }
            __syncthreads();
        }
        const int n = n0 + tn;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + tm + i;
            if (part) {
                if (m < M && n < N) part[((size_t)c * M + m) * N + n] = acc[i];
            } else {
                total[i] = __fadd_rn(total[i], acc[i]);
            }
        }
    }
    if (part) return;
    const int n = n0 + tn;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + tm + i;
        if (m < M && n < N) out[(size_t)m * N + n] = from_f32<TO>(total[i]);
    }
}

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
    if (per > 0) {
        LC_CHECK(workspace, "gemm: M=%d N=%d K=%d needs a workspace", M, N, K);
        dim3 grid((N + GB_N - 1) / GB_N, few ? 1 : (M + GB_M - 1) / GB_M, (chunks + per - 1) / per);
        if (few)
            gemm_generic_few_kernel<TX, TW, TO><<<grid, 256, 0, stream>>>((const TX*)x, (const TW*)w, (TO*)out, M,
                                                                          N, K, workspace, per);
        else
            gemm_generic_kernel<TX, TW, TO><<<grid, 256, 0, stream>>>((const TX*)x, (const TW*)w, (TO*)out, M, N,
                                                                      K, workspace, per);
        LC_LAUNCH_CHECK("gemm_generic");
        const size_t MN = (size_t)M * N;
        gemm_generic_sum_kernel<TO><<<(int)((MN + 255) / 256 < 4096 ? (MN + 255) / 256 : 4096), 256, 0, stream>>>(
            workspace, (TO*)out, MN, chunks);
        LC_LAUNCH_CHECK("gemm_generic_sum");
        return 0;
    }
    dim3 grid((N + GB_N - 1) / GB_N, few ? 1 : (M + GB_M - 1) / GB_M);
    if (few)
        gemm_generic_few_kernel<TX, TW, TO><<<grid, 256, 0, stream>>>((const TX*)x, (const TW*)w, (TO*)out, M, N,
                                                                      K, nullptr, 0);
    else
        gemm_generic_kernel<TX, TW, TO><<<grid, 256, 0, stream>>>((const TX*)x, (const TW*)w, (TO*)out, M, N, K,
                                                                  nullptr, 0);
    LC_LAUNCH_CHECK("gemm_generic");
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
