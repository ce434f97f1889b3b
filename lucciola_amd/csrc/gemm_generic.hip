// out[M, N] = x[M, K] . w[N, K]^T for any sizes and any mix of float32 / bfloat16 operands,
// accumulated with float32 FMAs (no matrix-core instruction, so that with float32 operands it
// is a true 32-bit product).  The weight layout is the checkpoint's: [out_features,
// in_features] row-major, applied as y = x . W^T without bias (reference:
// src/kernels/linear.cu:24-27, one thread per output element; here LDS-tiled 64x64x16 with a
// 4x4 register tile per thread).
#include "common.h"

namespace lc {

constexpr int GB_M = 64, GB_N = 64, GB_K = 16;

template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TX* __restrict__ x,
                                                           const TW* __restrict__ w,
                                                           TO* __restrict__ out, int M, int N,
                                                           int K) {
    __shared__ float xs[GB_K][GB_M + 4];
    __shared__ float ws[GB_K][GB_N + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * GB_M, n0 = blockIdx.x * GB_N;
    const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
    float acc[4][4] = {};

    // loader mapping: 64 rows x 16 k; thread loads 4 consecutive k of one row
    const int lrow = tid / 4, lk = (tid % 4) * 4;
    for (int k0 = 0; k0 < K; k0 += GB_K) {
        {
            const int m = m0 + lrow;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int k = k0 + lk + j;
                xs[lk + j][lrow] = (m < M && k < K) ? to_f32(x[(size_t)m * K + k]) : 0.f;
            }
            const int n = n0 + lrow;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int k = k0 + lk + j;
                ws[lk + j][lrow] = (n < N && k < K) ? to_f32(w[(size_t)n * K + k]) : 0.f;
            }
        }
        __syncthreads();
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
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + tm + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tn + j;
            if (n < N) out[(size_t)m * N + n] = from_f32<TO>(acc[i][j]);
        }
    }
}

template <typename TX, typename TW, typename TO>
static int launch_generic(const void* x, const void* w, void* out, int M, int N, int K,
                          hipStream_t stream) {
    dim3 grid((N + GB_N - 1) / GB_N, (M + GB_M - 1) / GB_M);
    gemm_generic_kernel<TX, TW, TO><<<grid, 256, 0, stream>>>((const TX*)x, (const TW*)w,
                                                              (TO*)out, M, N, K);
    LC_LAUNCH_CHECK("gemm_generic");
    return 0;
}

}  // namespace lc

using namespace lc;

LC_API int lc_gemm_generic(const void* x, int x_dt, const void* w, int w_dt, void* out, int out_dt,
                           int M, int N, int K, hipStream_t stream) {
    LC_CHECK(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    if (M == 0) return 0;
    LC_CHECK(x && w && out, "gemm: null pointer");
    LC_CHECK((size_t)((M + GB_M - 1) / GB_M) <= 65535, "gemm: M=%d is too large", M);
    const int key = x_dt * 4 + w_dt * 2 + out_dt;
    switch (key) {
        case 0: return launch_generic<float, float, float>(x, w, out, M, N, K, stream);
        case 2: return launch_generic<float, bf16, float>(x, w, out, M, N, K, stream);
        case 4: return launch_generic<bf16, float, float>(x, w, out, M, N, K, stream);
        case 5: return launch_generic<bf16, float, bf16>(x, w, out, M, N, K, stream);
        case 6: return launch_generic<bf16, bf16, float>(x, w, out, M, N, K, stream);
        case 7: return launch_generic<bf16, bf16, bf16>(x, w, out, M, N, K, stream);
        default:
            LC_CHECK(false, "gemm: unsupported dtypes x=%d w=%d out=%d", x_dt, w_dt, out_dt);
    }
    return 0;
}
