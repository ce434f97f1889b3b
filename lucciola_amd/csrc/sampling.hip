// Picking the next token from float32 logits: greedy, and temperature sampling by inverse CDF.
//
// Greedy: the reference's argmax (src/kernels/argmax.cu:23-58: one workgroup per row, ties by
// thread order); here the lowest index wins.  Temperature sampling is absent from the
// reference: p = softmax(logits / temperature) in float32, token = first index whose
// cumulative probability exceeds u * sum, with u in [0, 1) given per row by the caller.
//
// A row of the vocabulary is cut into SP_BLOCKS fixed parts, one workgroup each, so that a
// few rows still fill the GPU.  Every sum runs over the same parts in the same order whatever
// else is in the batch: a row's result depends only on that row, its temperature and its u.
//   pass 1  per (row, part): maximum and its lowest index
//   pass 2  per (row, part), sampled rows only: sum of exp((x - max) / T) over the part
//   pass 3  per row: pick (greedy: the best part's index; sampled: the part that holds
//           u * total, then the first index inside it whose running sum passes the target)
#include "common.h"
#include "no_alloc.h"

#include <mutex>

namespace lc {

constexpr int SP_THREADS = 256;
constexpr int SP_BLOCKS = 32;

// The workspace of lc_sample_static.  In host code this name is only a stand-in for the
// symbol: the array's address on a device comes from hipGetSymbolAddress (static_scratch()),
// and only that pointer is ever given to a kernel.
static __device__ __align__(256) __attribute__((used)) float scratch[LC_SAMPLE_STATIC_MAX_ROWS * SP_BLOCKS * 3];

constexpr int SP_MAX_DEVICES = 64;
static float* scratch_ptr[SP_MAX_DEVICES];      // per device: each GPU has its own copy of the array
static std::mutex scratch_mutex;

// The address of `scratch` on the current device, looked up at the first call there.
static int static_scratch(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    LC_CHECK(e == hipSuccess, "sample_static: hipGetDevice failed: %s", hipGetErrorString(e));
    LC_CHECK(dev >= 0 && dev < SP_MAX_DEVICES, "sample_static: device %d is beyond the %d this library keeps",
             dev, SP_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        float* p = nullptr;
        e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        LC_CHECK(e == hipSuccess && p, "sample_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        scratch_ptr[dev] = p;
    }
    *out = scratch_ptr[dev];
    return 0;
}

__device__ __forceinline__ void part_range(int V, int part, int& begin, int& end) {
    const int per = (V + SP_BLOCKS - 1) / SP_BLOCKS;
    begin = min(part * per, V);
    end = min(begin + per, V);
}

// ws_max [R, SP_BLOCKS], ws_idx [R, SP_BLOCKS]
__global__ __launch_bounds__(SP_THREADS) void sample_max_kernel(const float* __restrict__ logits,
                                                                float* __restrict__ ws_max,
                                                                int* __restrict__ ws_idx, int V) {
    __shared__ float vals[SP_THREADS];
    __shared__ int idxs[SP_THREADS];
    const int row = blockIdx.y, part = blockIdx.x, tid = threadIdx.x;
    int begin, end;
    part_range(V, part, begin, end);
    const float* x = logits + (size_t)row * V;
    float best = -INFINITY;
    int best_i = V;
    for (int i = begin + tid; i < end; i += SP_THREADS) {
        const float v = x[i];
        if (best_i == V || v > best) { best = v; best_i = i; }   // i rises: ties keep the lower
    }
    vals[tid] = best;
    idxs[tid] = best_i;
    __syncthreads();
    for (int s = SP_THREADS / 2; s > 0; s >>= 1) {
        if (tid < s) {
            const float ov = vals[tid + s];
            const int oi = idxs[tid + s];
            if (oi < V && (idxs[tid] == V || ov > vals[tid] || (ov == vals[tid] && oi < idxs[tid]))) {
                vals[tid] = ov;
                idxs[tid] = oi;
            }
        }
        __syncthreads();
    }
    if (tid == 0) {
        ws_max[row * SP_BLOCKS + part] = vals[0];
        ws_idx[row * SP_BLOCKS + part] = idxs[0];
    }
}

__device__ __forceinline__ float row_max(const float* ws_max, const int* ws_idx, int row, int V,
                                         int* arg) {
    float b = -INFINITY;
    int bi = V;
    for (int k = 0; k < SP_BLOCKS; ++k) {
        const int i = ws_idx[row * SP_BLOCKS + k];
        const float v = ws_max[row * SP_BLOCKS + k];
        if (i < V && (bi == V || v > b)) { b = v; bi = i; }     // parts rise: ties keep the lower
    }
    if (arg) *arg = bi;
    return b;
}

// ws_sum [R, SP_BLOCKS]: sum of exp((x - max) / T) over the part, threads' shares added in order
__global__ __launch_bounds__(SP_THREADS) void sample_sum_kernel(const float* __restrict__ logits,
                                                                const float* __restrict__ temperature,
                                                                const float* __restrict__ ws_max,
                                                                const int* __restrict__ ws_idx,
                                                                float* __restrict__ ws_sum, int V) {
    __shared__ float vals[SP_THREADS];
    const int row = blockIdx.y, part = blockIdx.x, tid = threadIdx.x;
    const float temp = temperature[row];
    if (!(temp > 0.f)) return;
    int begin, end;
    part_range(V, part, begin, end);
    const float* x = logits + (size_t)row * V;
    const float m = row_max(ws_max, ws_idx, row, V, nullptr);
    const float inv_t = 1.f / temp;
    // each thread owns a contiguous piece of the part
    const int per = (end - begin + SP_THREADS - 1) / SP_THREADS;
    const int b = min(begin + tid * per, end), e = min(b + per, end);
    float s = 0.f;
    for (int i = b; i < e; ++i) s += expf((x[i] - m) * inv_t);
    vals[tid] = s;
    __syncthreads();
    if (tid == 0) {
        float total = 0.f;
        for (int k = 0; k < SP_THREADS; ++k) total += vals[k];
        ws_sum[row * SP_BLOCKS + part] = total;
    }
}

__global__ __launch_bounds__(SP_THREADS) void sample_pick_kernel(const float* __restrict__ logits,
                                                                 const float* __restrict__ temperature,
                                                                 const float* __restrict__ uniform,
                                                                 const float* __restrict__ ws_max,
                                                                 const int* __restrict__ ws_idx,
                                                                 const float* __restrict__ ws_sum,
                                                                 int* __restrict__ out, int V) {
    __shared__ float vals[SP_THREADS];
    __shared__ float s_run, s_target;
    __shared__ int s_owner;
    const int row = blockIdx.x, tid = threadIdx.x;
    int arg;
    const float m = row_max(ws_max, ws_idx, row, V, &arg);
    const float temp = temperature ? temperature[row] : 0.f;
    if (!(temp > 0.f)) {
        if (tid == 0) out[row] = arg;
        return;
    }
    const float* x = logits + (size_t)row * V;
    const float inv_t = 1.f / temp;
    // the part that holds the target
    float total = 0.f;
    for (int k = 0; k < SP_BLOCKS; ++k) total += ws_sum[row * SP_BLOCKS + k];
    const float target = uniform[row] * total;
    float run = 0.f;
    int part = SP_BLOCKS - 1;
    for (int k = 0; k < SP_BLOCKS; ++k) {
        const float s = ws_sum[row * SP_BLOCKS + k];
        if (run + s > target) { part = k; break; }
        run += s;
    }
    int begin, end;
    part_range(V, part, begin, end);
    while (end == begin && part > 0) { --part; part_range(V, part, begin, end); }
    // the threads' pieces of that part, as pass 2 summed them
    const int per = (end - begin + SP_THREADS - 1) / SP_THREADS;
    const int b = min(begin + tid * per, end), e = min(b + per, end);
    float s = 0.f;
    for (int i = b; i < e; ++i) s += expf((x[i] - m) * inv_t);
    vals[tid] = s;
    __syncthreads();
    if (tid == 0) {
        int owner = SP_THREADS - 1;
        float r = run;
        for (int k = 0; k < SP_THREADS; ++k) {
            if (r + vals[k] > target) { owner = k; break; }
            r += vals[k];
        }
        s_owner = owner;
        s_run = r;
        s_target = target;
    }
    __syncthreads();
    if (tid == s_owner) {
        float r = s_run;
        int pick = -1;
        for (int i = b; i < e; ++i) {
            r += expf((x[i] - m) * inv_t);
            if (r > s_target) { pick = i; break; }
        }
        if (pick < 0) pick = e > b ? e - 1 : arg;   // rounding left the target past the end
        out[row] = pick;
    }
}

// ids[i] = sampled[source[i]] where source[i] >= 0: the tokens a step sampled go into the next
// step's batch on the device, without a round trip through the host.
__global__ void feed_tokens_kernel(int* __restrict__ ids, const int* __restrict__ source,
                                   const int* __restrict__ sampled, int T, int S) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= T) return;
    int s = source[i];
    if (s >= 0 && s < S) ids[i] = sampled[s];
}

}  // namespace lc

using namespace lc;

// Floats of workspace a call needs for R rows.
LC_API int lc_sample_workspace(int R) { return R * SP_BLOCKS * 3; }

static int sample_into(const float* logits, const float* temperature, const float* uniform, int* out,
                       float* workspace, int R, int V, hipStream_t stream) {
    float* ws_max = workspace;
    int* ws_idx = reinterpret_cast<int*>(workspace + (size_t)R * SP_BLOCKS);
    float* ws_sum = workspace + (size_t)2 * R * SP_BLOCKS;
    sample_max_kernel<<<dim3(SP_BLOCKS, R), SP_THREADS, 0, stream>>>(logits, ws_max, ws_idx, V);
    LC_LAUNCH_CHECK("sample_max");
    if (temperature) {
        sample_sum_kernel<<<dim3(SP_BLOCKS, R), SP_THREADS, 0, stream>>>(logits, temperature, ws_max,
                                                                         ws_idx, ws_sum, V);
        LC_LAUNCH_CHECK("sample_sum");
    }
    sample_pick_kernel<<<R, SP_THREADS, 0, stream>>>(logits, temperature, uniform, ws_max, ws_idx,
                                                     ws_sum, out, V);
    LC_LAUNCH_CHECK("sample_pick");
    return 0;
}

// temperature and uniform may be null (all rows greedy).  workspace: lc_sample_workspace(R)
// 4-byte words.
LC_API int lc_sample(const float* logits, const float* temperature, const float* uniform, int* out,
                     float* workspace, int R, int V, hipStream_t stream) {
    LC_CHECK(R >= 0 && V > 0, "sample: bad sizes R=%d V=%d", R, V);
    if (R == 0) return 0;
    LC_CHECK(logits && out && workspace, "sample: null pointer");
    LC_CHECK(!temperature || uniform, "sample: temperatures without uniform numbers");
    LC_CHECK(R <= 65535, "sample: too many rows (%d)", R);
    return sample_into(logits, temperature, uniform, out, workspace, R, V, stream);
}

// lc_sample without a workspace from the caller and without any allocation (no_alloc.h): the
// workspace is the library's own array on the current device.  Overlapping calls on one GPU
// race on that array.
LC_API int lc_sample_static(const float* logits, const float* temperature, const float* uniform,
                            int* out, int R, int V, hipStream_t stream) {
    LC_CHECK(R >= 0 && V > 0, "sample_static: bad sizes R=%d V=%d", R, V);
    LC_CHECK(R <= LC_SAMPLE_STATIC_MAX_ROWS, "sample_static: %d rows are more than the %d the library's "
             "own workspace holds (use lc_sample with a workspace of the caller's)", R, LC_SAMPLE_STATIC_MAX_ROWS);
    if (R == 0) return 0;
    LC_CHECK(logits && out, "sample_static: null pointer");
    LC_CHECK(!temperature || uniform, "sample_static: temperatures without uniform numbers");
    float* workspace = nullptr;
    if (int rc = static_scratch(&workspace)) return rc;
    return sample_into(logits, temperature, uniform, out, workspace, R, V, stream);
}

LC_API int lc_sample_static_max_rows(void) { return LC_SAMPLE_STATIC_MAX_ROWS; }

// ids [T] of a batch: where source[i] >= 0 the id is taken from sampled[source[i]] (S rows of an
// earlier lc_sample on the same stream); other ids stay.
LC_API int lc_feed_tokens(int* ids, const int* source, const int* sampled, int T, int S,
                          hipStream_t stream) {
    LC_CHECK(T >= 0 && S >= 0, "feed_tokens: bad sizes T=%d S=%d", T, S);
    if (T == 0 || S == 0) return 0;
    LC_CHECK(ids && source && sampled, "feed_tokens: null pointer");
    feed_tokens_kernel<<<(T + 255) / 256, 256, 0, stream>>>(ids, source, sampled, T, S);
    LC_LAUNCH_CHECK("feed_tokens");
    return 0;
}
