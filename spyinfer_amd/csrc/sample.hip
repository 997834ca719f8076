// Token choice on the device: first maximum (greedy), or the inverse CDF of softmax(logits / T)
// over ascending token ids at a given uniform number u.  One block per row of logits.
#include "common.h"
#include <math.h>

#define SM_THREADS 1024

__global__ __launch_bounds__(SM_THREADS) void sample_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                            const float* __restrict__ uniform, int* __restrict__ out, int V) {
    __shared__ float red[16];
    __shared__ float best_v[16];
    __shared__ int best_i[16];
    __shared__ float part[SM_THREADS];
    __shared__ int chosen;
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* x = logits + (size_t)r * V;
    const float temp = temperature[r];
    // each thread owns a contiguous run of ids, so that sums walk the ids in ascending order
    const int chunk = (V + SM_THREADS - 1) / SM_THREADS;
    const int b = min(V, tid * chunk), e = min(V, b + chunk);
    float mv = -INFINITY;
    int mi = 0x7fffffff;
    for (int i = b; i < e; ++i) {
        const float v = x[i];
        if (v > mv || (mi == 0x7fffffff && !(v < mv))) { mv = v; mi = i; }   // first maximum; a NaN row still yields an id
    }
    // wave: keep the greater value, on ties the lower id
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(mv, o, 64);
        const int oi = __shfl_xor(mi, o, 64);
        if (ov > mv || (ov == mv && oi < mi)) { mv = ov; mi = oi; }
    }
    if ((tid & 63) == 0) { best_v[tid >> 6] = mv; best_i[tid >> 6] = mi; }
    __syncthreads();
    mv = best_v[0]; mi = best_i[0];
    for (int w = 1; w < SM_THREADS / 64; ++w)
        if (best_v[w] > mv || (best_v[w] == mv && best_i[w] < mi)) { mv = best_v[w]; mi = best_i[w]; }
    if (!(temp > 0.f)) {
        if (tid == 0) out[r] = mi == 0x7fffffff ? 0 : mi;
        return;
    }
    const float inv_t = 1.0f / temp;
    float s = 0.f;
    for (int i = b; i < e; ++i) s += expf((x[i] - mv) * inv_t);
    part[tid] = s;
    const float total = block_sum(s, red);
    if (tid == 0) chosen = -1;
    __syncthreads();
    const float target = uniform[r] * total;
    // exclusive prefix of the per-thread sums, in id order (one wave scans the 1024 partial sums)
    if (tid < 64) {
        float run = 0.f;
        for (int i = 0; i < tid * (SM_THREADS / 64); ++i) run += part[i];   // prefix before this lane's 16 partials
        for (int i = tid * (SM_THREADS / 64); i < (tid + 1) * (SM_THREADS / 64); ++i) {
            const float nxt = run + part[i];
            const int bi = min(V, i * chunk), ei = min(V, bi + chunk);
            if (bi < ei && target >= run && target < nxt && chosen < 0) {
                // this run of ids holds the target: walk it
                float acc = run;
                int pick = ei - 1;
                for (int j = bi; j < ei; ++j) {
                    acc += expf((x[j] - mv) * inv_t);
                    if (target < acc) { pick = j; break; }
                }
                atomicCAS(&chosen, -1, pick);
            }
            run = nxt;
        }
    }
    __syncthreads();
    if (tid == 0) out[r] = chosen >= 0 ? chosen : (mi == 0x7fffffff ? 0 : mi);
}

extern "C" int spy_sample(const float* logits, const float* temperature, const float* uniform, int* out, int R, int V, hipStream_t st) {
    SPY_REQUIRE(R > 0 && V > 0, "spy_sample: empty operand");
    sample_kernel<<<R, SM_THREADS, 0, st>>>(logits, temperature, uniform, out, V);
    SPY_CHECK_LAUNCH("spy_sample");
    return 0;
}
