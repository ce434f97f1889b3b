// Shared helpers of the gfx950 kernels: element types, 64-lane reductions, error reporting.
//
// The reference's helpers assume 32-lane warps (include/kernels/util.h:5-41: WARP_SIZE 32,
// __shfl_*_sync masks of 0xffffffff); a CDNA4 wavefront has 64 lanes and every reduction
// here is written for that.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lc {

constexpr int kWave = 64;

// Element type tags that cross the C boundary.
enum : int { DT_F32 = 0, DT_BF16 = 1 };

typedef __bf16 bf16;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return static_cast<float>(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return static_cast<bf16>(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// Sum over a workgroup of up to 1024 threads; `scratch` holds one float per wave (16 floats).
// Every thread gets the total.  The order of the additions is fixed by the thread layout.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int nwaves = (blockDim.x + kWave - 1) / kWave;
    v = wave_sum(v);
    __syncthreads();  // scratch may still be read from an earlier call
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < nwaves; ++w) total += scratch[w];
    return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int nwaves = (blockDim.x + kWave - 1) / kWave;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = scratch[0];
    for (int w = 1; w < nwaves; ++w) total = fmaxf(total, scratch[w]);
    return total;
}

// Error text of the last failed call on this thread; entry points return 0 on success.
void set_error(const char* fmt, ...);

#define LC_CHECK(cond, ...)                 \
    do {                                    \
        if (!(cond)) {                      \
            ::lc::set_error(__VA_ARGS__);   \
            return 1;                       \
        }                                   \
    } while (0)

#define LC_LAUNCH_CHECK(what)                                                     \
    do {                                                                          \
        hipError_t e__ = hipGetLastError();                                       \
        if (e__ != hipSuccess) {                                                  \
            ::lc::set_error("%s: launch failed: %s", what, hipGetErrorString(e__)); \
            return 2;                                                             \
        }                                                                         \
    } while (0)

}  // namespace lc

#define LC_API extern "C" __attribute__((visibility("default")))
