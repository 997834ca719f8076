// Token choice on the device: first maximum (greedy), or the inverse CDF of softmax(logits / T)
// over ascending token ids at a given uniform number u.
// Two kernels: (1) every row is cut into SM_CHUNKS contiguous chunks of ids, one block per chunk
// finds the chunk's first maximum and, for T > 0, its sum of exp((x - chunk max) / T);
// (2) one wave per row merges the chunks in id order, finds the chunk that holds u * total and
// walks it.  All sums run over ascending ids, so the choice is a function of (logits, T, u) alone.
#include "common.h"
#include "no_alloc.h"
#include <math.h>
#include <mutex>

#define SM_CHUNKS 64
#define SM_THREADS 256

__device__ __forceinline__ void better(float& v, int& i, float ov, int oi) {
    // the greater value wins, on ties the lower id; an id is "unset" as INT_MAX; a NaN never wins
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

__global__ __launch_bounds__(SM_THREADS) void sample_chunks_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                                   float* __restrict__ pmax, int* __restrict__ pidx,
                                                                   float* __restrict__ psum, int V) {
    __shared__ float sv[SM_THREADS / 64];
    __shared__ int si[SM_THREADS / 64];
    __shared__ float red[SM_THREADS / 64];
    const int c = blockIdx.x, r = blockIdx.y, tid = threadIdx.x;
    const int chunk = (V + SM_CHUNKS - 1) / SM_CHUNKS;
    const int b = min(V, c * chunk), e = min(V, b + chunk);
    const float* x = logits + (size_t)r * V;
    float mv = -INFINITY;
    int mi = 0x7fffffff;
    for (int i = b + tid; i < e; i += SM_THREADS) better(mv, mi, x[i], i);
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(mv, o, 64);
        const int oi = __shfl_xor(mi, o, 64);
        better(mv, mi, ov, oi);
    }
    if ((tid & 63) == 0) { sv[tid >> 6] = mv; si[tid >> 6] = mi; }
    __syncthreads();
    mv = sv[0]; mi = si[0];
    for (int w = 1; w < SM_THREADS / 64; ++w) better(mv, mi, sv[w], si[w]);
    const float temp = temperature[r];
    float s = 0.f;
    if (temp > 0.f && mi != 0x7fffffff) {
        const float inv_t = 1.0f / temp;
        for (int i = b + tid; i < e; i += SM_THREADS) s += expf((x[i] - mv) * inv_t);
        s = block_sum(s, red);
    }
    if (tid == 0) {
        pmax[r * SM_CHUNKS + c] = mv;
        pidx[r * SM_CHUNKS + c] = mi;
        psum[r * SM_CHUNKS + c] = s;
    }
}

__global__ __launch_bounds__(64) void sample_pick_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                         const float* __restrict__ uniform, const float* __restrict__ pmax,
                                                         const int* __restrict__ pidx, const float* __restrict__ psum,
                                                         int* __restrict__ out, int V) {
    __shared__ float mass[SM_CHUNKS];
    __shared__ float lsum[64];
    const int r = blockIdx.x, lane = threadIdx.x;
    float mv = pmax[r * SM_CHUNKS + lane];
    int mi = pidx[r * SM_CHUNKS + lane];
    const float cmax = mv;
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(mv, o, 64);
        const int oi = __shfl_xor(mi, o, 64);
        better(mv, mi, ov, oi);
    }
    const int greedy = mi == 0x7fffffff ? 0 : mi;
    const float temp = temperature[r];
    if (!(temp > 0.f)) {
        if (lane == 0) out[r] = greedy;
        return;
    }
    const float inv_t = 1.0f / temp;
    // mass of each chunk relative to the row maximum
    mass[lane] = (cmax == -INFINITY) ? 0.f : psum[r * SM_CHUNKS + lane] * expf((cmax - mv) * inv_t);
    __syncthreads();
    float total = 0.f;
    for (int c = 0; c < SM_CHUNKS; ++c) total += mass[c];
    const float target = uniform[r] * total;
    int chosen_chunk = -1;
    float before = 0.f;
    {
        float run = 0.f;
        for (int c = 0; c < SM_CHUNKS; ++c) {
            const float nxt = run + mass[c];
            if (chosen_chunk < 0 && mass[c] > 0.f && target < nxt) { chosen_chunk = c; before = run; }
            run = nxt;
        }
    }
    if (chosen_chunk < 0) {          // rounding pushed the target to the very end: the row's maximum stands in
        if (lane == 0) out[r] = greedy;
        return;
    }
    const int chunk = (V + SM_CHUNKS - 1) / SM_CHUNKS;
    const int b = min(V, chosen_chunk * chunk), e = min(V, b + chunk);
    const float* x = logits + (size_t)r * V;
    // every lane sums a contiguous run of the chunk, then the runs are walked in order
    const int per = (e - b + 63) / 64;
    const int lb = min(e, b + lane * per), le = min(e, lb + per);
    float s = 0.f;
    for (int i = lb; i < le; ++i) s += expf((x[i] - mv) * inv_t);
    lsum[lane] = s;
    __syncthreads();
    if (lane == 0) {
        float run = before;
        int pick = -1, last_pos = -1;
        for (int w = 0; w < 64 && pick < 0; ++w) {
            const float nxt = run + lsum[w];
            if (lsum[w] > 0.f) {
                const int wb = min(e, b + w * per), we = min(e, wb + per);
                if (target < nxt) {
                    float acc = run;
                    for (int i = wb; i < we; ++i) {
                        const float p = expf((x[i] - mv) * inv_t);
                        acc += p;
                        if (p > 0.f) last_pos = i;
                        if (target < acc) { pick = i; break; }
                    }
                    if (pick < 0) pick = last_pos;   // the run's sum and its walk rounded apart
                } else {
                    last_pos = we - 1;
                }
            }
            run = nxt;
        }
        out[r] = pick >= 0 ? pick : (last_pos >= 0 ? last_pos : greedy);
    }
}

extern "C" int64_t spy_sample_workspace(int R) { return (int64_t)R * SM_CHUNKS * 3; }

// Both kernels; ``ws`` holds spy_sample_workspace(R) floats of device memory.
static int launch_sample(const char* name, const float* logits, const float* temperature, const float* uniform, int* out, int R, int V,
                         float* ws, hipStream_t st) {
    float* pmax = ws;
    int* pidx = reinterpret_cast<int*>(ws + (size_t)R * SM_CHUNKS);
    float* psum = ws + (size_t)2 * R * SM_CHUNKS;
    sample_chunks_kernel<<<dim3(SM_CHUNKS, R), SM_THREADS, 0, st>>>(logits, temperature, pmax, pidx, psum, V);
    sample_pick_kernel<<<R, 64, 0, st>>>(logits, temperature, uniform, pmax, pidx, psum, out, V);
    SPY_CHECK_LAUNCH(name);
    return 0;
}

extern "C" int spy_sample(const float* logits, const float* temperature, const float* uniform, int* out, int R, int V, float* ws,
                          hipStream_t st) {
    SPY_REQUIRE(R > 0 && V > 0, "spy_sample: empty operand");
    SPY_REQUIRE(R <= 65535, "spy_sample: too many rows");
    SPY_REQUIRE(ws, "spy_sample: no workspace");
    return launch_sample("spy_sample", logits, temperature, uniform, out, R, V, ws, st);
}

// ---- the variant that allocates nothing (no_alloc.h) ------------------------------------------------------------
// The workspace of the two kernels as an array of the library: every GPU that runs the library has its own copy at
// its own address.  In host code the array's name is only a handle for hipGetSymbolAddress, never a device pointer.
static __device__ __align__(256) float scratch[(size_t)SPY_SAMPLE_STATIC_MAX_ROWS * SM_CHUNKS * 3];

#define SPY_MAX_DEVICES 64
static std::mutex g_scratch_lock;
static float* g_scratch_ptr[SPY_MAX_DEVICES];      // the array's address on each device, asked for once per device

// The current device's copy of ``scratch``; nullptr (and the error recorded) if it cannot be had.
static float* scratch_of_current_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= SPY_MAX_DEVICES) {
        spy_fail("spy_sample_static: no current device (%s)", e != hipSuccess ? hipGetErrorString(e) : "index out of range");
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        float* ptr = nullptr;
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            spy_fail("spy_sample_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

extern "C" int spy_sample_static(const float* logits, const float* temperature, const float* uniform, int* out, int R, int V,
                                 hipStream_t st) {
    SPY_REQUIRE(R > 0 && V > 0, "spy_sample_static: empty operand");
    SPY_REQUIRE(R <= SPY_SAMPLE_STATIC_MAX_ROWS, "spy_sample_static: %d rows, the library's scratch array holds %d at most", R,
                SPY_SAMPLE_STATIC_MAX_ROWS);
    SPY_REQUIRE(logits && temperature && uniform && out, "spy_sample_static: null operand");
    float* ws = scratch_of_current_device();
    if (!ws) return 1;
    // nothing to clear: sample_chunks_kernel writes all 3 * R * SM_CHUNKS elements that sample_pick_kernel reads
    return launch_sample("spy_sample_static", logits, temperature, uniform, out, R, V, ws, st);
}
