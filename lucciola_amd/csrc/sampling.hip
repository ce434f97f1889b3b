// Picking the next token from float32 logits: greedy, and temperature sampling by inverse CDF.
//
// Greedy: the reference's argmax (src/kernels/argmax.cu:23-58) breaks ties by thread order;
// here the lowest index wins.  Temperature sampling is absent from the reference: p =
// softmax(logits / temperature) in float32, token = first index whose cumulative probability
// exceeds u * sum, with u in [0, 1) given per row by the caller.  A row's result depends only
// on that row, its temperature and its u.
#include "common.h"

namespace lc {

constexpr int SP_THREADS = 256;

// One workgroup per row.  temperature <= 0 selects greedy for that row.
__global__ __launch_bounds__(SP_THREADS) void sample_kernel(const float* __restrict__ logits,
                                                            const float* __restrict__ temperature,
                                                            const float* __restrict__ uniform,
                                                            int* __restrict__ out, int V) {
    __shared__ float vals[SP_THREADS];
    __shared__ int idxs[SP_THREADS];
    __shared__ float scratch[16];
    __shared__ int chosen;
    const int row = blockIdx.x, tid = threadIdx.x;
    const float* x = logits + (size_t)row * V;
    const int chunk = (V + SP_THREADS - 1) / SP_THREADS;
    const int begin = min(tid * chunk, V), end = min(begin + chunk, V);

    // maximum and its lowest index (each thread owns a contiguous range of the vocabulary)
    float best = -INFINITY;
    int best_i = V;
    for (int i = begin; i < end; ++i) {
        const float v = x[i];
        if (v > best || best_i == V) { best = v; best_i = i; }
    }
    vals[tid] = best;
    idxs[tid] = best_i;
    __syncthreads();
    if (tid == 0) {
        float b = vals[0];
        int bi = idxs[0];
        for (int k = 1; k < SP_THREADS; ++k)
            if (idxs[k] < V && (bi == V || vals[k] > b)) { b = vals[k]; bi = idxs[k]; }
        vals[0] = b;
        chosen = bi;
    }
    __syncthreads();
    const float temp = temperature ? temperature[row] : 0.f;
    if (!(temp > 0.f)) {
        if (tid == 0) out[row] = chosen;
        return;
    }
    const float m = vals[0];
    const float inv_t = 1.f / temp;
    __syncthreads();

    float part = 0.f;
    for (int i = begin; i < end; ++i) part += expf((x[i] - m) * inv_t);
    vals[tid] = part;
    __syncthreads();
    if (tid == 0) {
        float total = 0.f;
        for (int k = 0; k < SP_THREADS; ++k) total += vals[k];
        const float target = uniform[row] * total;
        // the range that holds the target
        float run = 0.f;
        int owner = SP_THREADS - 1;
        for (int k = 0; k < SP_THREADS; ++k) {
            if (run + vals[k] > target) { owner = k; break; }
            run += vals[k];
        }
        scratch[0] = run;
        scratch[1] = target;
        idxs[0] = owner;
    }
    __syncthreads();
    if (tid == idxs[0]) {
        float run = scratch[0];
        const float target = scratch[1];
        int pick = -1;
        for (int i = begin; i < end; ++i) {
            run += expf((x[i] - m) * inv_t);
            if (run > target) { pick = i; break; }
        }
        if (pick < 0) pick = end > begin ? end - 1 : chosen;  // rounding left the target past the end
        out[row] = pick;
    }
}

}  // namespace lc

using namespace lc;

// temperature and uniform may be null (all rows greedy).
LC_API int lc_sample(const float* logits, const float* temperature, const float* uniform, int* out,
                     int R, int V, hipStream_t stream) {
    LC_CHECK(R >= 0 && V > 0, "sample: bad sizes R=%d V=%d", R, V);
    if (R == 0) return 0;
    LC_CHECK(logits && out, "sample: null pointer");
    LC_CHECK(!temperature || uniform, "sample: temperatures without uniform numbers");
    sample_kernel<<<R, SP_THREADS, 0, stream>>>(logits, temperature, uniform, out, V);
    LC_LAUNCH_CHECK("sample");
    return 0;
}
