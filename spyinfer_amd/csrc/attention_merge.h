// Merging the partial results of attention over parts of the keys (shared by the attention kernels).
// A part of a 16-row unit is { O[16][DMAX] unnormalised, m[16] (natural-log domain), l[16] } in float32 at
// ws[((unit * n_kv + hk) * splits + part) * 16 * (DMAX + 2)].
#pragma once
#include "common.h"
#include <math.h>

// Where element (row m, column n) lies when at most 16 * tiles rows are kept in MFMA operand order for a product that
// reads them next: [n / 32 steps][tiles][64 lanes][8], lane 16 g + m % 16 of tile m / 16 holding columns 32 s + 8 g ...
__device__ __forceinline__ size_t attention_out_operand_order(int m, int n, int tiles) {
    return ((((size_t)(n >> 5) * tiles + (m >> 4)) * 64 + ((n & 31) >> 3) * 16 + (m & 15)) * 8) + (n & 7);
}

// Merge the parts of each (tile, kv head): O = sum_i O_i e^(m_i - M) / sum_i l_i e^(m_i - M).
// out_tiles > 0: the output goes out in operand order for that many row tiles (see above) instead of [T, n_q d].
// SINGLE: every entry is one token with one tile (tile t is entry t, query token t): nothing of the step's description
// is read, one memory round trip less before the parts can be asked for.
// The kernel is a chain of memory round trips with little to do between them, so every thread asks for all it needs of
// a stage at once: the parts' maxima and sums by 16 threads per part, then a thread's elements of four parts at a time.
template <int DMAX, bool SINGLE = false>
__global__ __launch_bounds__(256) void attention_merge_kernel(bf16_t* __restrict__ out, const float* __restrict__ ws,
                                                              const int* __restrict__ cu_q, const int* __restrict__ tile_entry,
                                                              const int* __restrict__ tile_row0, int n_q, int n_kv, int d, int splits,
                                                              int units_per_tile, int out_tiles = 0) {
    __shared__ float wgt[64 * 16];     // weight of part i for row r: [i][r], up to 64 parts
    __shared__ float pm[64 * 16], pl[64 * 16];
    __shared__ float inv_l[16];
    // a unit is 16 rows; a tile of the attention kernel that wrote the parts has units_per_tile of them
    const int unit = blockIdx.x, hk = blockIdx.y, tid = threadIdx.x;
    const int tile = unit / units_per_tile;
    const int G = n_q / n_kv;
    const int s = SINGLE ? tile : tile_entry[tile];
    const int row0 = SINGLE ? 0 : tile_row0[tile] + 16 * (unit - tile * units_per_tile);
    const int q0 = SINGLE ? s : cu_q[s];
    const int nrows = SINGLE ? G : (cu_q[s + 1] - q0) * G;
    constexpr int PART = 16 * (DMAX + 2);
    const float* base = ws + ((size_t)unit * n_kv + hk) * splits * PART;
    if (row0 >= nrows) return;
    for (int e = tid; e < splits * 16; e += 256) {
        const float* w = base + (size_t)(e >> 4) * PART + 16 * DMAX + (e & 15);
        pm[e] = w[0];
        pl[e] = w[16];
    }
    __syncthreads();
    if (tid < 16) {
        float M = -INFINITY;
        for (int i = 0; i < splits; ++i) M = fmaxf(M, pm[i * 16 + tid]);
        float L = 0.f;
        for (int i = 0; i < splits; ++i) {
            const float mi = pm[i * 16 + tid];
            const float e = (mi == -INFINITY) ? 0.f : __expf(mi - M);
            wgt[i * 16 + tid] = e;
            L += pl[i * 16 + tid] * e;
        }
        inv_l[tid] = L > 0.f ? 1.0f / L : 0.f;
    }
    __syncthreads();
    const int valid = min(16, nrows - row0);
    for (int e = tid; e < valid * d; e += 256) {
        const int r = e / d, dd = e - r * d;
        const int row = row0 + r;
        const float* src = base + r * DMAX + dd;
        float o = 0.f;
        for (int i0 = 0; i0 < splits; i0 += 4) {
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = i0 + j < splits ? src[(size_t)(i0 + j) * PART] : 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (i0 + j < splits) o += v[j] * wgt[(i0 + j) * 16 + r];      // parts in ascending order, as before
        }
        const int tq = row / G, head = hk * G + row % G;
        const size_t at = out_tiles ? attention_out_operand_order(q0 + tq, head * d + dd, out_tiles) : ((size_t)(q0 + tq) * n_q + head) * d + dd;
        out[at] = f32_to_bf16(o * inv_l[r]);
    }
}
