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

// four consecutive elements as floats, in one load
__device__ __forceinline__ void load4(float (&dst)[4], const float* p) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
}
__device__ __forceinline__ void load4(float (&dst)[4], const bf16* p) {
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
    const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
    for (int j = 0; j < 4; ++j) dst[j] = static_cast<float>(v[j]);
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

// ---------------------------------------------------------------------------------------------
// A head of 128 bfloat16 entries held by a group of 16 neighbouring lanes (lane j of the group
// has entries 8 j .. 8 j + 7): RMSNorm over the head and half-split rotary embedding without
// leaving the registers.  Lanes talk through DPP moves inside their row of 16; all 16 lanes of
// a group must be active.  Used by the q/k norm + rotary kernel and by the decode attention's
// own prologue, which therefore agree to the bit.
typedef __bf16 head_chunk __attribute__((ext_vector_type(8)));

template <int CTRL> __device__ __forceinline__ float row_move(float v) {   // a DPP move inside a row of 16
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over the 16 lanes of a row; the pairs are added in the same order in every lane, so all
// lanes end with the same bits.
__device__ __forceinline__ float row16_sum(float v, int j) {
    v += row_move<0xB1>(v);                                   // lane ^ 1
    v += row_move<0x4E>(v);                                   // lane ^ 2
    const float up = row_move<0x124>(v), down = row_move<0x12C>(v);   // rotations by 4 and by 12
    // which of the two rotations brought lane j ^ 4 depends on the direction of the rotation:
    // the lane index itself is sent along to tell
    const int from_up = __builtin_bit_cast(int, row_move<0x124>(__builtin_bit_cast(float, j)));
    v += (from_up == (j ^ 4)) ? up : down;                    // lane ^ 4
    v += row_move<0x128>(v);                                  // lane ^ 8
    return v;
}

// What head128_norm_rope needs beside the raw entries, for the lane that holds entries 8 j to
// 8 j + 7 of a head of 128: the norm's weights there (w: all 128, or null) and the cosines and sines
// of the entries' pairs (cs: the position's row of the rotary table, 64 cosines, then 64 sines, or
// null), both 16-byte aligned.  A function of its own so that a caller can ask for them before the
// raw entries are there.
struct Head128Constants {
    float w[8], c[8], s[8];
    bool normed, rotated;
};
__device__ __forceinline__ Head128Constants head128_constants(int j, const float* __restrict__ w,
                                                              const float* __restrict__ cs) {
    Head128Constants k;
    k.normed = w != nullptr;
    k.rotated = cs != nullptr;
    // w and cs are 16-byte aligned: four entries a load
    typedef float float4v __attribute__((ext_vector_type(4)));
    const int i0 = 8 * (j & 7);
    float4v w0 = {1.f, 1.f, 1.f, 1.f}, w1 = w0, c0 = w0, c1 = w0, s0 = {0.f, 0.f, 0.f, 0.f}, s1 = s0;
    if (w) {
        w0 = *reinterpret_cast<const float4v*>(w + 8 * j);
        w1 = *reinterpret_cast<const float4v*>(w + 8 * j + 4);
    }
    if (cs) {
        c0 = *reinterpret_cast<const float4v*>(cs + i0);
        c1 = *reinterpret_cast<const float4v*>(cs + i0 + 4);
        s0 = *reinterpret_cast<const float4v*>(cs + 64 + i0);
        s1 = *reinterpret_cast<const float4v*>(cs + 64 + i0 + 4);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        k.w[e] = w0[e]; k.w[4 + e] = w1[e];
        k.c[e] = c0[e]; k.c[4 + e] = c1[e];
        k.s[e] = s0[e]; k.s[4 + e] = s1[e];
    }
    return k;
}

// x: the lane's 8 entries (raw).  Entry i pairs with entry i + 64.
__device__ __forceinline__ head_chunk head128_norm_rope(head_chunk x, int j, const Head128Constants& k,
                                                        float eps) {
    float f[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = static_cast<float>(x[e]);
    if (k.normed) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) ss = __fmaf_rn(f[e], f[e], ss);
        ss = row16_sum(ss, j);
        const float inv = rsqrtf(ss / 128.f + eps);
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = __fmul_rn(__fmul_rn(f[e], inv), k.w[e]);
    }
    if (k.rotated) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float other = row_move<0x128>(f[e]);        // the partner entry, 64 further on or back
            // first half: a c - b s (a own, b partner); second half: a s + b c (b own, a partner)
            const float own_c = __fmul_rn(f[e], k.c[e]), other_s = __fmul_rn(other, k.s[e]);
            f[e] = (j < 8) ? __fsub_rn(own_c, other_s) : __fadd_rn(other_s, own_c);
        }
    }
    head_chunk out;
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = static_cast<bf16>(f[e]);
    return out;
}

// The same with the weights (or null) and the table's row (or null) where they lie.
__device__ __forceinline__ head_chunk head128_norm_rope(head_chunk x, int j, const float* __restrict__ w,
                                                        float eps, const float* __restrict__ cs) {
    return head128_norm_rope(x, j, head128_constants(j, w, cs), eps);
}

// Waits with a count of the wave's own: at most N of its youngest memory loads (vmcnt), or LDS and
// scalar-memory operations (lgkmcnt), may still be in flight; the other counters are left alone.
template <int N> __device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));
}
template <int N> __device__ __forceinline__ void wait_lgkmcnt() {
    __builtin_amdgcn_s_waitcnt(0xC07F | (N << 8));
}

// Compute units of the GPU.  They only steer how work is laid over the device (tile plans, the
// number of shares); no result depends on them.
int device_cus();

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
