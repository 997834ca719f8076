// The decode product whose blocks walk runs of column tiles: the kernel and its launch, shared by the two source files that
// build it for the stored product (gemm_decode_wide.hip) and for the gated product (gemm_decode_wide_gated.hip); two
// files so that they compile side by side.
#pragma once
#include "gemm_decode.h"
#include <math.h>

// For 17 to 128 rows and matrices of many columns (the gated product, the output head): what bounds the kernel with a
// column tile per block (gemm_decode.hip) is not the matrix' way from memory but the L2's throughput, through which every block also pulls all of X (with MT row
// tiles that is MT times the bytes of its tile of W).  Here one block per CU walks a run of neighbouring column tiles,
// CT at a time, against the same X fragments in registers: X's traffic falls to MT / CT (MT / 2 CT for the gated
// product, whose gate and up tiles share them as well).  The waves of a block split K in interleaved chunks; operands are loaded a
// step of 32 of K at a time, ahead of the products that use them; the waves' sums of the group's
// column tiles are added through LDS in two rounds, in a fixed order, and the four waves that end up with them run the
// epilogue, each for every fourth (column tile, row tile) unit.  Store and gated epilogues only.
// GW: waves per block.  8 up to four row tiles; 4 beyond (65 to 128 rows), where a wave's sums of a group take up to 192
// registers and a SIMD has one wave with all 512 of its registers.
template <int EPI, bool SCALED, typename TC, int MT, int CT, bool XT, bool OT, int GW = 8>
__global__ __launch_bounds__(GW * 64, 1) void gemm_decode_wide_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ Wt, TC* __restrict__ C, const float* __restrict__ ss_in,
    int n_parts, float eps, int M, int N, int K) {
    static_assert(EPI == EPI_STORE || EPI == EPI_GATED, "the wide kernel has no residual epilogue");
    static_assert(GW == 8 || GW == 4, "four or eight waves");
    static_assert((EPI == EPI_GATED ? 2 : 1) * CT * MT <= (GW == 8 ? 24 : 48), "the accumulators of a group must fit the registers");
    constexpr int GATES = EPI == EPI_GATED ? 2 : 1;
    constexpr int NT = GATES * CT;
    constexpr int MP = 16 * MT;
    constexpr int PAIRS = CT * MT;                       // (column tile, row tile) units of the epilogue
    // the waves' sums meet in two rounds: waves 4..7 (if there are eight) hand all of theirs to waves 0..3, then each of
    // these four takes every fourth unit from the other three, PB units at a time (72 KB of LDS at most).  The second
    // round's buffer lies inside the first's.
    constexpr int PB = PAIRS * 3 * GATES <= 72 ? PAIRS : 72 / (3 * GATES) / 4 * 4;
    constexpr int RED_TILES = (GW == 8 && 4 * NT * MT > PB * 3 * GATES) ? 4 * NT * MT : PB * 3 * GATES;
    __shared__ f32x4_t red[RED_TILES * 64];
    __shared__ float ss_red[GW * 4 * MP];
    __shared__ float row_scale[MP];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;

    // This thread's share of the rows' sums of squares, all of it under way at once (one round trip before the matrix'
    // first loads); the waves' shares meet after the first group's products.
    float ss_part[MT];
    if (SCALED) gd_ss_share<MT, GW * 4>(ss_in, n_parts, wave * 4 + g, r, ss_part);

    // this block's run of column tiles: the tiles dealt evenly over the blocks
    const int tiles = N / 16;
    const int t_begin = (int)((long long)tiles * blockIdx.x / gridDim.x), t_end = (int)((long long)tiles * (blockIdx.x + 1) / gridDim.x);
    const size_t chunk_stride = (size_t)(GATES * tiles) * 4096;
    unsigned xoff[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        xoff[mt] = XT ? (unsigned)mt * 1024u + 16u * lane : (unsigned)min(16 * mt + r, M - 1) * (unsigned)K * 2u + 16u * g;
    }
    const char* xbase = reinterpret_cast<const char*>(X);
    const int nfull = K / GD_CHUNK;
    const int my_steps = wave < nfull ? 4 * ((nfull - wave + GW - 1) / GW) : 0;      // steps of 32 of K: this wave's chunks

    for (int t0 = t_begin; t0 < t_end; t0 += CT) {
        const int here = min(CT, t_end - t0);            // tiles of this group (the run's last group may have fewer)
        f32x4_t acc[NT][MT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        const char* wbase = reinterpret_cast<const char*>(Wt) + (size_t)t0 * 4096 + 16u * lane;
        // One step at a time, the next step's operands asked for before this step's products: a wave has loads under
        // way while its matrix unit works (against half a chunk loaded and then multiplied: 1-2 %).
        {
            bf16x8_t a0[NT], b0[MT], a1[NT], b1[MT];
#define GDW_LOAD(A, B, STEP)                                                                                         \
            {                                                                                                        \
                const int c_ = wave + GW * ((STEP) >> 2), h_ = (STEP) & 3;                                           \
                const char* wb = wbase + (size_t)c_ * chunk_stride;                                                  \
                const char* xb = xbase + (size_t)c_ * (XT ? 4 * MT * 1024 : GD_CHUNK * 2);                           \
                _Pragma("unroll") for (int nt = 0; nt < NT; ++nt) {                                                  \
                    /* a tile that the group does not have reads the group's first tile again (its sums are dropped) */ \
                    const int ct = nt % CT < here ? nt % CT : 0;                                                     \
                    A[nt] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(                            \
                        wb + (size_t)((nt / CT) * tiles + ct) * 4096 + 1024 * h_));                                  \
                }                                                                                                    \
                _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                                    \
                    B[mt] = *reinterpret_cast<const bf16x8_t*>(xb + xoff[mt] + (XT ? MT * 1024 : 64) * h_);          \
            }
#define GDW_MFMA(A, B)                                                                                               \
            _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                                        \
                _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                                    \
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[nt], B[mt], acc[nt][mt], 0, 0, 0);
            // Every load is unconditional (rows of X beyond M: the last row's address, or the operand order's padding; their
            // sums are not stored) and the last steps, which ask for nothing more, are peeled from the loops: a load under a
            // condition makes the compiler count the loads in flight as the fewest there may be, and one that the last turn
            // skips makes it wait for all of them in every turn.  The scheduling barriers keep it from sinking the loads
            // below the products.
#define GDW_FENCE __builtin_amdgcn_sched_barrier(0);
            if constexpr (GW == 4 && NT + MT <= 12) {
                // a wave that has a SIMD's registers to itself keeps three steps' operands under way instead of one (four
                // waves with one step each would have too few bytes in flight to keep the memory busy), where four steps'
                // operands fit the 256 registers that loads can write
                bf16x8_t a2[NT], b2[MT], a3[NT], b3[MT];
                if (my_steps > 0) {                             // (a multiple of 4)
                    GDW_LOAD(a0, b0, 0) GDW_LOAD(a1, b1, 1) GDW_LOAD(a2, b2, 2)
                    int st = 0;
                    for (; st + 4 < my_steps; st += 4) {
                        GDW_LOAD(a3, b3, st + 3) GDW_FENCE
                        GDW_MFMA(a0, b0) GDW_FENCE
                        GDW_LOAD(a0, b0, st + 4) GDW_FENCE
                        GDW_MFMA(a1, b1) GDW_FENCE
                        GDW_LOAD(a1, b1, st + 5) GDW_FENCE
                        GDW_MFMA(a2, b2) GDW_FENCE
                        GDW_LOAD(a2, b2, st + 6) GDW_FENCE
                        GDW_MFMA(a3, b3) GDW_FENCE
                    }
                    GDW_LOAD(a3, b3, st + 3) GDW_FENCE
                    GDW_MFMA(a0, b0) GDW_FENCE
                    GDW_MFMA(a1, b1) GDW_FENCE
                    GDW_MFMA(a2, b2) GDW_FENCE
                    GDW_MFMA(a3, b3)
                }
            } else {
                // (three steps' operands where they fit beside the sums, two under way while one is multiplied, were slower:
                // the gated product at 24 / 32 / 48 rows 34.2 / 34.1 / 36.3 us against 33.7 / 33.6 / 35.4)
                if (my_steps > 0) {                             // (a multiple of 4)
                    GDW_LOAD(a0, b0, 0)
                    int st = 0;
                    for (; st + 2 < my_steps; st += 2) {
                        GDW_LOAD(a1, b1, st + 1) GDW_FENCE
                        GDW_MFMA(a0, b0) GDW_FENCE
                        GDW_LOAD(a0, b0, st + 2) GDW_FENCE
                        GDW_MFMA(a1, b1) GDW_FENCE
                    }
                    GDW_LOAD(a1, b1, st + 1) GDW_FENCE
                    GDW_MFMA(a0, b0) GDW_FENCE
                    GDW_MFMA(a1, b1)
                }
            }
#undef GDW_FENCE
#undef GDW_LOAD
#undef GDW_MFMA
        }
        // ---- round one: the upper four waves' sums to the lower four -------------------------------------------------
        if (SCALED && t0 == t_begin) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) ss_red[(wave * 4 + g) * MP + 16 * mt + r] = ss_part[mt];
        }
        if (GW == 8 && wave >= 4) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) red[(((wave - 4) * NT + nt) * MT + mt) * 64 + lane] = acc[nt][mt];
        }
        if (GW == 8 || (SCALED && t0 == t_begin)) __syncthreads();
        // (the rows' scales: by a wave that has nothing to add now, if there is one)
        const int t_scale = (int)threadIdx.x - (GW == 8 ? 256 : 0);
        if (SCALED && t0 == t_begin && t_scale >= 0 && t_scale < MP) {
            float s = 0.f;
            for (int i = 0; i < GW * 4; ++i) s += ss_red[i * MP + t_scale];
            row_scale[t_scale] = 1.0f / sqrtf(s / (float)K + eps);
        }
        if (GW == 8 && wave < 4) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[nt][mt] += red[((wave * NT + nt) * MT + mt) * 64 + lane];
        }
        if (GW == 8 || (SCALED && t0 == t_begin)) __syncthreads();
        // ---- round two: unit p = ct MT + mt (its gate and its up tile) belongs to wave p % 4 --------------------------
#pragma unroll
        for (int p0 = 0; p0 < PAIRS; p0 += PB) {
            if (wave < 4) {
#pragma unroll
                for (int p = p0; p < p0 + PB && p < PAIRS; ++p) {
                    const int owner = p & 3;
                    if (wave != owner) {
                        const int slot = wave < owner ? wave : wave - 1;
#pragma unroll
                        for (int gt = 0; gt < GATES; ++gt) red[(((p - p0) * 3 + slot) * GATES + gt) * 64 + lane] = acc[gt * CT + p / MT][p % MT];
                    }
                }
            }
            __syncthreads();
            if (wave < 4) {
#pragma unroll
                for (int p = p0; p < p0 + PB && p < PAIRS; ++p) {
                    if (wave != (p & 3)) continue;
                    const int ct = p / MT, mt = p % MT;
                    f32x4_t v = acc[ct][mt], up = acc[(GATES - 1) * CT + ct][mt];
#pragma unroll
                    for (int slot = 0; slot < 3; ++slot) {
                        v += red[(((p - p0) * 3 + slot) * GATES + 0) * 64 + lane];
                        if (EPI == EPI_GATED) up += red[(((p - p0) * 3 + slot) * GATES + GATES - 1) * 64 + lane];
                    }
                    const int n = (t0 + ct) * 16 + 4 * g, m = 16 * mt + r;
                    if (ct >= here || m >= M) continue;
                    const float scale = SCALED ? row_scale[m] : 1.f;
                    TC* out = C + (OT ? operand_order(m, n, MT) : (size_t)m * N + n);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float y = v[i] * scale;
                        if (EPI == EPI_GATED) { const float u = up[i] * scale; y = (y / (1.0f + expf(-y))) * u; }
                        out[i] = from_f32<TC>(y);
                    }
                }
            }
            __syncthreads();                              // the buffer is free for the next units, or the next group
        }
    }
}

constexpr int GD_WIDE_MIN_ROWS = 9;     // rows from which the kernel that walks column tiles is taken

// Column tiles per group of the wide kernel for blocks that walk `per` tiles each with MT row tiles: the CT that moves the
// fewest bytes through L2, X once per group (MT units per step) and W once per tile (GATES units).
static int wide_ct(int per, int MT, int gates, int max_ct) {
    int best = 1, best_cost = 1 << 30;
    for (int ct = 1; ct <= max_ct; ++ct) {
        if (ct == 5 || ct == 7 || (ct > 8 && ct != 12)) continue;   // (not built)
        const int cost = ((per + ct - 1) / ct) * MT + per * gates;
        if (cost < best_cost) { best = ct; best_cost = cost; }
    }
    return best;
}

constexpr int GD_GW4_FROM = 5;        // (four waves from three row tiles on, measured at 40 to 64 rows: gate/up 41-43 us against 35-37)
constexpr int GD_GW4_STORE_FROM = 3;  // (the stored product, whose four-wave blocks take up to twelve column tiles at a time: the output head of
                                      // 151936 x 4096 at 48 / 64 / 96 rows 253 / 267 / 288 us against 266 / 283 / 307 with eight waves and six tiles)

// The most column tiles of a group: its accumulators (GATES * CT * MT tiles of four registers) leave room for its
// operands up to 24 tiles, 48 for a wave that has a SIMD to itself.
template <int GATES, int MT, int GW>
constexpr int wide_max_ct() {
    constexpr int room = (GW == 8 ? 24 : 48) / (GATES * MT), most = GW == 4 ? 12 : 6;
    return room < most ? room : most;
}

// (MIN_CT: the fewest column tiles of a group that this call may ask for; smaller groups are not built for it)
template <int EPI, bool SCALED, typename TC, int MT, bool XT, bool OT, int GW, int MIN_CT = 1>
static bool gd_launch_wide_with(const GdArgs& a, int ct, int blocks) {
    constexpr int MAX_CT = wide_max_ct<EPI == EPI_GATED ? 2 : 1, MT, GW>();
#define GD_WIDE_CASE(C)                                                                                               \
    if constexpr (C <= MAX_CT && C >= MIN_CT) {                                                                       \
        if (ct == C) {                                                                                                \
            gemm_decode_wide_kernel<EPI, SCALED, TC, MT, C, XT, OT, GW><<<blocks, GW * 64, 0, a.st>>>(                    \
                a.x, a.w, (TC*)a.c, a.ss_in, a.n_parts, a.eps, a.M, a.N, a.K);                                        \
            return true;                                                                                              \
        }                                                                                                             \
    }
    GD_WIDE_CASE(2) GD_WIDE_CASE(3) GD_WIDE_CASE(4) GD_WIDE_CASE(6) GD_WIDE_CASE(8) GD_WIDE_CASE(12)
#undef GD_WIDE_CASE
    return false;                                              // one tile at a time: the kernel with a tile per block stands
}

template <int EPI, bool SCALED, typename TC, int MT, bool XT, bool OT>
static bool gd_launch_wide(const GdArgs& a) {
    // (only the combination that a decode step has, a normed input in operand order, to keep the library's build short)
    if constexpr (EPI == EPI_RESID || !SCALED || !XT) return false;
    else {
        constexpr int GATES = EPI == EPI_GATED ? 2 : 1;
        // beyond four row tiles (the stored product: beyond two): four waves with a SIMD's registers each
        constexpr bool FOUR = MT >= (EPI == EPI_STORE ? GD_GW4_STORE_FROM : GD_GW4_FROM);
        const int cus = gd_compute_units(), tiles = a.N / 16;
        // fewer than two tiles per CU: one tile per block, two blocks per CU (beyond four row tiles the gated product has
        // no other kernel: it walks here whatever the width, two column tiles at a time at least)
        const bool only = MT > 4 && EPI == EPI_GATED;
        if (tiles < 2 * cus && !only) return false;
        const int per = (tiles + cus - 1) / cus;
        const int blocks = tiles < cus ? tiles : cus;
        if constexpr (FOUR) {
            int ct = wide_ct(per, MT, GATES, wide_max_ct<GATES, MT, 4>());
            if (only && ct < 2) ct = 2;
            return gd_launch_wide_with<EPI, SCALED, TC, MT, XT, OT, 4>(a, ct, blocks);
        } else {
            const int ct = wide_ct(per, MT, GATES, wide_max_ct<GATES, MT, 8>());
            // The gated product at three and four row tiles: four waves where their larger groups take a block's run in
            // fewer turns, each turn a pass over X (five gate/up pairs a block with 17408 x 5120: one group of six
            // against groups of three and two, 67.8 against 77.9 us at 64 rows; with three pairs a block, 12288 x 4096,
            // one group either way, eight waves are faster: 35-37 against 41-43 us)
            if constexpr (EPI == EPI_GATED && MT >= 3 && sizeof(TC) == 2) {
                const int ct4 = wide_ct(per, MT, GATES, wide_max_ct<GATES, MT, 4>());
                if (ct4 >= 4 && (per + ct4 - 1) / ct4 < (per + ct - 1) / ct)
                    return gd_launch_wide_with<EPI, SCALED, TC, MT, XT, OT, 4, 4>(a, ct4, blocks);
            }
            return gd_launch_wide_with<EPI, SCALED, TC, MT, XT, OT, 8>(a, ct, blocks);
        }
    }
}

// Which calls walk: the stored and the gated product of a normed input in operand order (what a decode step has), from
// 17 rows on for matrices with two column tiles per compute unit and more, beyond 64 rows the gated product of any
// width; and the stored product (the output head) from 9 rows on: with a column tile per block its blocks pull as many
// bytes of X through L2 as of W at 16 rows (251 us; walking six tiles at a time 222; up to 8 rows the kernel with a tile
// per block stays, 187-194 against 206-211 us).
template <int EPI, typename TC, bool OT>
static bool wide_rows(const GdArgs& a) {
    if (EPI == EPI_STORE && a.M >= GD_WIDE_MIN_ROWS && a.M <= 16) return gd_launch_wide<EPI, true, TC, 1, true, OT>(a);
    if (a.M > 96) return gd_launch_wide<EPI, true, TC, 8, true, OT>(a);
    if (a.M > 64) return gd_launch_wide<EPI, true, TC, 6, true, OT>(a);
    if (a.M > 48) return gd_launch_wide<EPI, true, TC, 4, true, OT>(a);
    if (a.M > 32) return gd_launch_wide<EPI, true, TC, 3, true, OT>(a);
    if (a.M > 16) return gd_launch_wide<EPI, true, TC, 2, true, OT>(a);
    return false;
}

