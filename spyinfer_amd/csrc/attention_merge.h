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
template <int DMAX>
__global__ __launch_bounds__(256) void attention_merge_kernel(bf16_t* __restrict__ out, const float* __restrict__ ws,
                                                              const int* __restrict__ cu_q, const int* __restrict__ tile_entry,
                                                              const int* __restrict__ tile_row0, int n_q, int n_kv, int d, int splits,
                                                              int units_per_tile, int out_tiles = 0) {
    __shared__ float wgt[64 * 16];     // weight of part i for row r: [i][r], up to 64 parts
    __shared__ float inv_l[16];
    // a unit is 16 rows; a tile of the attention kernel that wrote the parts has units_per_tile of them
    const int unit = blockIdx.x, hk = blockIdx.y, tid = threadIdx.x;
    const int tile = unit / units_per_tile;
    const int s = tile_entry[tile], row0 = tile_row0[tile] + 16 * (unit - tile * units_per_tile);
    const int G = n_q / n_kv;
    const int q0 = cu_q[s];
    const int nrows = (cu_q[s + 1] - q0) * G;
    const float* base = ws + ((size_t)unit * n_kv + hk) * splits * (16 * (DMAX + 2));
    if (row0 >= nrows) return;
    if (tid < 16) {
        float M = -INFINITY;
        for (int i = 0; i < splits; ++i) M = fmaxf(M, base[(size_t)i * (16 * (DMAX + 2)) + 16 * DMAX + tid]);
        float L = 0.f;
        for (int i = 0; i < splits; ++i) {
            const float* w = base + (size_t)i * (16 * (DMAX + 2));
            const float mi = w[16 * DMAX + tid];
            const float e = (mi == -INFINITY) ? 0.f : __expf(mi - M);
            wgt[i * 16 + tid] = e;
            L += w[16 * DMAX + 16 + tid] * e;
        }
        inv_l[tid] = L > 0.f ? 1.0f / L : 0.f;
    }
    __syncthreads();
    const int valid = min(16, nrows - row0);
    for (int e = tid; e < valid * d; e += 256) {
        const int r = e / d, dd = e - r * d;
        const int row = row0 + r;
        float o = 0.f;
        for (int i = 0; i < splits; ++i) o += base[(size_t)i * (16 * (DMAX + 2)) + r * DMAX + dd] * wgt[i * 16 + r];
        const int tq = row / G, head = hk * G + row % G;
        const size_t at = out_tiles ? attention_out_operand_order(q0 + tq, head * d + dd, out_tiles) : ((size_t)(q0 + tq) * n_q + head) * d + dd;
        out[at] = f32_to_bf16(o * inv_l[r]);
    }
}

