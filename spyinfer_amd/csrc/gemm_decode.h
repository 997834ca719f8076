// What the decode products' source files share: vector types, the epilogues' codes, the operand order, the arguments
// of a call.
#pragma once
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define GD_CHUNK 128
#define EPI_STORE 0
#define EPI_GATED 1
#define EPI_RESID 2

// Where element (row m, column n) of a matrix of MT row tiles lies in operand order, in elements:
// [N/32 steps][MT row tiles][64 lanes][8], lane 16 g + r of step s holding x[r][32 s + 8 g ..] of its row tile.
__device__ __forceinline__ size_t operand_order(int m, int n, int MT = 1) {
    return ((((size_t)(n >> 5) * MT + (m >> 4)) * 64 + ((n & 31) >> 3) * 16 + (m & 15)) * 8) + (n & 7);
}

// This thread's share of the parts of the rows' sums of squares, for MT row tiles: parts slot, slot + GROUPS, ... of row
// 16 mt + r.  The first 256 parts are asked for at once (one memory round trip; a loop that adds as it loads has one
// per turn) and added in the order of the parts.
template <int MT, int GROUPS>
__device__ __forceinline__ void gd_ss_share(const float* __restrict__ ss_in, int n_parts, int slot, int r, float (&out)[MT]) {
    constexpr int NPV = 256 / GROUPS, MP = 16 * MT;
    float pv[NPV][MT];
#pragma unroll
    for (int i = 0; i < NPV; ++i) {
        const int p = slot + GROUPS * i;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) pv[i][mt] = p < n_parts ? ss_in[p * MP + 16 * mt + r] : 0.f;
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) out[mt] = 0.f;
#pragma unroll
    for (int i = 0; i < NPV; ++i)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) out[mt] += pv[i][mt];
    for (int p = 256 + slot; p < n_parts; p += GROUPS)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) out[mt] += ss_in[p * MP + 16 * mt + r];
}

// The residual epilogue for one lane's four columns n .. n + 3 of row m: h = h_old + v goes back to the stream (float32),
// bf16(h * w_next) to the next product's input (row-major, or in operand order for MT row tiles), and the four lanes of
// a row add their shares of sum(h^2); lane group 0 writes the row's part to ss_part_row[m].  Rows beyond M write nothing
// to the stream and the part 0.  wn: the next norm's weight for the four columns, two bfloat16 per word.
template <bool OT>
__device__ __forceinline__ void gd_residual_epilogue(const f32x4_t& v, const f32x4_t& h_old, uint2 wn, float* __restrict__ resid_out,
                                                     bf16_t* __restrict__ xw_out, float* __restrict__ ss_part_row, int m, int n, int g,
                                                     int M, int N, int MT) {
    float s = 0.f;
    if (m < M) {
        f32x4_t h = h_old;
#pragma unroll
        for (int i = 0; i < 4; ++i) { h[i] += v[i]; s += h[i] * h[i]; }
        *reinterpret_cast<f32x4_t*>(resid_out + (size_t)m * N + n) = h;
        uint2 o;
        o.x = pack_bf16x2(h[0] * __uint_as_float(wn.x << 16), h[1] * __uint_as_float(wn.x & 0xffff0000u));
        o.y = pack_bf16x2(h[2] * __uint_as_float(wn.y << 16), h[3] * __uint_as_float(wn.y & 0xffff0000u));
        *reinterpret_cast<uint2*>(xw_out + (OT ? operand_order(m, n, MT) : (size_t)m * N + n)) = o;
    }
    s += __shfl_xor(s, 16, 64);
    s += __shfl_xor(s, 32, 64);
    if (g == 0) ss_part_row[m] = s;
}

struct GdArgs {
    const bf16_t* x; const bf16_t* w; void* c; float* resid; bf16_t* xw_out; const bf16_t* w_next; float* ss_out; const float* ss_in;
    int n_parts; float eps; int M, N, K; bool xt, ot; hipStream_t st;
    void* ws; long long ws_bytes;          // the device's workspace of the products that split K over blocks (or none)
};

// Compute units of the current device (asked for once per device).
int gd_compute_units();

// The product whose blocks walk runs of column tiles (gemm_decode_wide.hip): true if it has launched the call.
bool gd_wide_try(const GdArgs& a, int epi, bool scaled, bool f32_out);

// The product with K split over blocks (gemm_decode_splitk.hip): true if it has launched the call.
bool gd_splitk_try(const GdArgs& a, int epi, bool scaled, bool f32_out);
long long gd_splitk_workspace_bytes();
