// Decode-time products (at most 16 rows) with the neighbouring small kernels folded in, so that a decode
// step launches fewer kernels (each costs 5-7 us here however little it does):
//
//   EPI_RESID the result is added to the residual stream h in place (float32); the block also writes
//             bf16(h_new * w_next), the next RMS norm's input already multiplied by that norm's weight, and
//             its part of every row's sum(h_new^2).
//   SCALED    the input is such a bf16(h * w) with the parts of sum(h^2); they are summed in a fixed order
//             and the result of the product is multiplied by rsqrt(sum / K + eps) in float32.  Together:
//             x . W^T with x = norm(h), the scale applied after the sum instead of before it.  The one
//             rounding of the operand to bfloat16 happens before the scale, which changes nothing in its
//             relative size.
//   EPI_GATED W = [gate | up] tiles, the block stores silu(gate) * up.
//   XT / OT   the input X / the bfloat16 output that the next product reads (bf16(h w) of EPI_RESID, the result of
//             EPI_GATED) in MFMA operand order instead of row-major: [K/32 steps][64 lanes][8], lane 16 g + r of step s
//             holding x[r][32 s + 8 g ..] for the 16 rows of the tile (rows beyond M hold anything).  An operand is then
//             one load of 1 KiB in one piece, as for W, instead of 16 pieces of 64 bytes: 5-12 % at 16 rows.
//   EPI_STORE the block stores the result (bfloat16 or float32).
//
// W comes as a copy in the order the kernel reads it (ops.tile_weight): [K/128 chunks][N/16 tiles][4 steps][64 lanes][8],
// lane 16 g + r of step j of chunk c of tile t holding W[16 t + r][128 c + 32 j + 8 g ..]: the MFMA operand of a wave
// is one load of 1 KiB in one piece, and, chunks being outermost, the tiles that all blocks read at one time lie next
// to each other in memory (with tiles outermost the blocks' addresses differ by multiples of the tile size and crowd
// on a part of the memory channels: 8-10 % slower).  One 16-row tile (two for EPI_GATED: gate tile t and up tile
// N/16 + t) per block; its waves split K in interleaved chunks and add through LDS in a fixed order.
#include "gemm_decode.h"
#include <math.h>

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

constexpr int GD_WAVES_GATED = 4;     // waves of a block of the gated product with a pair of column tiles per block

// H3: a block has three halves of column tiles (24 columns) instead of one tile: tile t whole and the lower half of
// tile t + 1, or the upper half of tile t and tile t + 1 whole, in turn.  For a matrix of one and a half column tiles per
// compute unit (qkv of 6144 columns on 256 units) every unit then streams the same number of bytes; with a tile per
// block half of the units stream two tiles and the others one.  A half tile is the lanes r < 8 (or r >= 8) of every
// fragment of W, 128 bytes in one piece each, and the columns 4 g + i of the lane groups g < 2 (g >= 2) of the result.
// The stored product only.
// HT: 0, or the number of half tiles of a block, 3 or 5 (two and a half tiles per unit: qkv of 10240 columns).
template <int EPI, bool SCALED, typename TC, int GD_WAVES, bool XT, bool OT, int HT = 0>
__global__ __launch_bounds__(GD_WAVES * 64) void gemm_decode_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ Wt, TC* __restrict__ C, float* __restrict__ resid_out,
    bf16_t* __restrict__ xw_out, const bf16_t* __restrict__ w_next, float* __restrict__ ss_out, const float* __restrict__ ss_in,
    int n_parts, float eps, int M, int N, int K) {
    constexpr bool H3 = HT != 0;
    static_assert(!H3 || (EPI == EPI_STORE && (HT == 3 || HT == 5)), "three or five halves of column tiles, the stored product only");
    constexpr int NT = H3 ? (HT + 1) / 2 : (EPI == EPI_GATED ? 2 : 1);
    __shared__ float red[(GD_WAVES - 1) * NT * 64 * 4];
    __shared__ float ss_red[GD_WAVES * 4 * 16];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int tile0 = H3 ? (HT * (int)blockIdx.x) >> 1 : (int)blockIdx.x;     // the block's (first) column tile
    const bool lower = (blockIdx.x & 1) == 0;                                   // H3: tile0 whole and half of the next, or the reverse
    const int n_base = tile0 * 16;
    const bool x_ok = r < M;                       // lanes whose row of X does not exist load nothing

    // Loads whose values are needed only after the product are issued now, so that they are on their way while
    // the matrix streams: every thread's share of the parts of sum(h^2) of row r (the first 256 parts; more are
    // summed here), and for the residual epilogue wave 0's piece of the stream and of the next norm's weight.
    constexpr int NPV = 256 / (GD_WAVES * 4);
    float pv[NPV], part = 0.f;
    if (SCALED) {
#pragma unroll
        for (int i = 0; i < NPV; ++i) {
            const int p = wave * 4 + g + GD_WAVES * 4 * i;
            pv[i] = p < n_parts ? ss_in[p * 16 + r] : 0.f;
        }
        for (int p = 256 + wave * 4 + g; p < n_parts; p += GD_WAVES * 4) part += ss_in[p * 16 + r];
    }
    f32x4_t h_old = {0.f, 0.f, 0.f, 0.f};
    uint2 wn = {0u, 0u};
    if (EPI == EPI_RESID && wave == 0 && x_ok) {
        h_old = *reinterpret_cast<const f32x4_t*>(resid_out + (size_t)r * N + n_base + 4 * g);
        wn = *reinterpret_cast<const uint2*>(w_next + n_base + 4 * g);
    }

    f32x4_t acc[NT], acc2[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) { acc[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f}; acc2[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f}; }
    const size_t chunk_stride = (size_t)((EPI == EPI_GATED ? 2 : 1) * N / 16) * 4096;         // bytes of one chunk of all tiles
    const char* wbase = reinterpret_cast<const char*>(Wt) + (size_t)tile0 * 4096;
    unsigned woff[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) woff[nt] = (H3 ? (unsigned)nt : (unsigned)(nt * N / 16)) * 4096u + 16u * lane;
    // halves: the lanes of a fragment of tile nt that this block reads (its first tile's upper half only, or its last
    // tile's lower half only)
    bool w_on[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) w_on[nt] = !H3 || (nt == 0 ? (lower || r >= 8) : (nt == NT - 1 ? (!lower || r < 8) : true));
    const char* xbase = reinterpret_cast<const char*>(X);
    const unsigned xoff = XT ? 16u * lane : (unsigned)min(r, M - 1) * (unsigned)K * 2u + 16u * g;

    bf16x8_t a0[NT][4], a1[NT][4], b0[4], b1[4];
#define GD_LOAD(A, B, CHUNK)                                                                             \
    {                                                                                                    \
        const char* wb_ = wbase + (size_t)(CHUNK) * chunk_stride;                                        \
        const char* xb_ = xbase + (size_t)(CHUNK) * (XT ? 4096 : GD_CHUNK * 2) + xoff;                   \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                                  \
            _Pragma("unroll") for (int nt = 0; nt < NT; ++nt) {                                          \
                if (!H3) A[nt][j] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wb_ + woff[nt] + 1024 * j));      \
                else A[nt][j] = w_on[nt] ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wb_ + woff[nt] + 1024 * j)) \
                                         : bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};                                                       \
            }                                                                                            \
            B[j] = x_ok ? *reinterpret_cast<const bf16x8_t*>(xb_ + (XT ? 1024 : 64) * j) : bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0}; \
        }                                                                                                \
    }
#define GD_MFMA(A, B, ACC)                                                                               \
    _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                        \
        _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                                \
            ACC[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[nt][j], B[j], ACC[nt], 0, 0, 0);

    const int nfull = K / GD_CHUNK;                 // K is a multiple of 128
    // Two chunks per round, all of their loads issued back to back before the products.  (A ring that keeps two chunks
    // under way all the time, the next asked for as soon as a chunk's registers are free, with unconditional loads and
    // waits that count what is in flight, was measured slower up to 8 rows: qkv 10.6 against 10.3 us, o 8.0 against 7.5,
    // gate/up 33.2 against 32.5, down 20.3 against 17.5, the output head 216 against 191; the memory serves the bursts of
    // 24 loads a wave better than the same loads twelve at a time between products.)
    int c = wave;
    for (; c + GD_WAVES < nfull; c += 2 * GD_WAVES) {
        GD_LOAD(a0, b0, c)
        GD_LOAD(a1, b1, c + GD_WAVES)
        GD_MFMA(a0, b0, acc)
        GD_MFMA(a1, b1, acc2)
    }
    if (c < nfull) {
        GD_LOAD(a0, b0, c)
        GD_MFMA(a0, b0, acc)
    }
#undef GD_LOAD
#undef GD_MFMA
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] += acc2[nt];

    if (SCALED) {
#pragma unroll
        for (int i = 0; i < NPV; ++i) part += pv[i];
        ss_red[(wave * 4 + g) * 16 + r] = part;
    }
    // ---- add the waves' tiles, in a fixed order ---------------------------------------------------------------
    if (wave > 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[(((wave - 1) * NT + nt) * 4 + i) * 64 + lane] = acc[nt][i];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 1; w < GD_WAVES; ++w)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[nt][i] += red[(((w - 1) * NT + nt) * 4 + i) * 64 + lane];
    if (SCALED) {
        float s = 0.f;
        for (int i = 0; i < GD_WAVES * 4; ++i) s += ss_red[i * 16 + r];
        const float scale = 1.0f / sqrtf(s / (float)K + eps);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[nt][i] *= scale;
    }

    // lane (m = r, g) holds C[m][n_base + 4 g + i]
    const int m = r, n = n_base + 4 * g;
    if (EPI == EPI_RESID) {
        gd_residual_epilogue<OT>(acc[0], h_old, wn, resid_out, xw_out, ss_out + blockIdx.x * 16, m, n, g, M, N, 1);
        return;
    }
    if (m >= M) return;
    if constexpr (H3) {
        // tile0: all columns (lower) or those of its upper half; the next tile: its lower half, or all
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const bool mine = nt == 0 ? (lower || g >= 2) : (nt == NT - 1 ? (!lower || g < 2) : true);
            if (!mine) continue;
            TC* out = C + (size_t)m * N + n + 16 * nt;
#pragma unroll
            for (int i = 0; i < 4; ++i) out[i] = from_f32<TC>(acc[nt][i]);
        }
        return;
    }
    TC* out = C + (OT ? operand_order(m, n) : (size_t)m * N + n);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float v = acc[0][i];
        if (EPI == EPI_GATED) { const float up = acc[NT - 1][i]; v = (v / (1.0f + expf(-v))) * up; }
        out[i] = from_f32<TC>(v);
    }
}

// The same for 17 to 64 rows: MT row tiles of X per tile of W, one chunk per round (the operands of MT row tiles take
// the registers that a second chunk would).  X and the outputs in operand order have MT row tiles per step; the parts
// of sum(h^2) have 16 MT rows each: ss[n][16 MT].
// CT: column tiles of 16 per block.  Every block reads all of X, from L2, and with MT row tiles that is MT times the
// bytes of its W tile: with two column tiles the X fragments in registers serve both, and X's traffic halves.
// H3 (with CT = 2, the stored product): three halves of column tiles per block, as in gemm_decode_kernel.
template <int EPI, bool SCALED, typename TC, int MT, int CT, int GD_WAVES, bool XT, bool OT, bool H3 = false, int NCH = 0>
__global__ __launch_bounds__(GD_WAVES * 64) void gemm_decode_rows_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ Wt, TC* __restrict__ C, float* __restrict__ resid_out,
    bf16_t* __restrict__ xw_out, const bf16_t* __restrict__ w_next, float* __restrict__ ss_out, const float* __restrict__ ss_in,
    int n_parts, float eps, int M, int N, int K) {
    static_assert(!H3 || (EPI == EPI_STORE && CT == 2), "halves of column tiles: the stored product, two tiles a block");
    constexpr int NT = (EPI == EPI_GATED ? 2 : 1) * CT;      // W tiles per block: [gate tiles | up tiles] for the gated product
    constexpr int MP = 16 * MT;
    __shared__ f32x4_t red[(GD_WAVES - 1) * NT * MT * 64];
    __shared__ float ss_red[GD_WAVES * 4 * MP];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;

    // What is needed only after the product is asked for now: this thread's share of the rows' sums of squares (all of
    // it under way at once), and for the residual epilogue the piece of the stream and of the next norm's weight of
    // the wave that will run it (row tile mt belongs to wave mt).
    float ss_part[MT];
    if (SCALED) gd_ss_share<MT, GD_WAVES * 4>(ss_in, n_parts, wave * 4 + g, r, ss_part);
    f32x4_t h_old = {0.f, 0.f, 0.f, 0.f};
    uint2 wn = {0u, 0u};
    if (EPI == EPI_RESID && wave < MT && 16 * wave + r < M) {
        static_assert(EPI != EPI_RESID || CT == 1, "the residual epilogue has one column tile per block");
        h_old = *reinterpret_cast<const f32x4_t*>(resid_out + (size_t)(16 * wave + r) * N + blockIdx.x * 16 + 4 * g);
        wn = *reinterpret_cast<const uint2*>(w_next + blockIdx.x * 16 + 4 * g);
    }

    f32x4_t acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const size_t chunk_stride = (size_t)((EPI == EPI_GATED ? 2 : 1) * N / 16) * 4096;
    const int tile0 = H3 ? (3 * (int)blockIdx.x) >> 1 : (int)blockIdx.x * CT;       // the block's first column tile
    const bool lower = (blockIdx.x & 1) == 0;                // H3: tile0 whole and the lower half of the next, or the reverse
    const bool w_on[2] = {!H3 || lower || r >= 8, !H3 || !lower || r < 8};
    const char* wbase = reinterpret_cast<const char*>(Wt) + (size_t)tile0 * 4096;
    unsigned woff[NT], xoff[MT];
    bool x_ok[MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) woff[nt] = (unsigned)((nt / CT) * (N / 16) + nt % CT) * 4096u + 16u * lane;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        x_ok[mt] = 16 * mt + r < M;
        xoff[mt] = XT ? (unsigned)mt * 1024u + 16u * lane : (unsigned)min(16 * mt + r, M - 1) * (unsigned)K * 2u + 16u * g;
    }
    const char* xbase = reinterpret_cast<const char*>(X);
    const int nfull = K / GD_CHUNK;
#define GDR_LOAD(A, B, CHUNK)                                                                                        \
    {                                                                                                                \
        const char* wb = wbase + (size_t)(CHUNK) * chunk_stride;                                                     \
        const char* xb = xbase + (size_t)(CHUNK) * (XT ? 4 * MT * 1024 : GD_CHUNK * 2);                              \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                                              \
            _Pragma("unroll") for (int nt = 0; nt < NT; ++nt) {                                                      \
                if (!H3) A[nt][j] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wb + woff[nt] + 1024 * j));                    \
                else A[nt][j] = w_on[nt & 1] ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wb + woff[nt] + 1024 * j))          \
                                             : bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};                                                                 \
            }                                                                                                        \
            _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                                        \
                B[mt][j] = x_ok[mt] ? *reinterpret_cast<const bf16x8_t*>(xb + xoff[mt] + (XT ? MT * 1024 : 64) * j)  \
                                    : bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};                                              \
        }                                                                                                            \
    }
#define GDR_MFMA(A, B)                                                                                               \
    _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                                    \
        _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                                            \
            _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                                        \
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[nt][j], B[mt][j], acc[nt][mt], 0, 0, 0);
    // (two chunks per round, and the next chunk's operands asked for before this chunk's products, were measured at two
    // to four row tiles: no gain either)
    if constexpr (NCH > 0) {
        // NCH chunks per wave exactly (the host has checked K = 128 NCH waves), all in straight-line code.  A ring of RW
        // chunks of W is under way while one is multiplied (all of the wave's W if it has no more), so that a compute unit
        // keeps enough of the matrix in flight to cover the memory's latency: a loop that loads a chunk and then multiplies
        // has a round trip to memory per chunk and streams at a third of the memory's rate.  X, which comes from L2, is
        // asked for two chunks ahead, and ahead of the W asked for in the same turn: loads come back in the order they
        // were issued, so an X piece behind a W piece waits for memory with it.  Every load is unconditional (rows of X
        // beyond M: the last row's address, or the operand order's padding; their sums are not stored), and scheduling
        // barriers keep the compiler from sinking the loads below the products.
        constexpr int RW = NCH * NT <= 4 ? NCH : (NT == 1 ? 4 : 2);
        bf16x8_t a[RW][NT][4], b[2][MT][4];
#define GDR_LOAD_W(A, I)                                                                                             \
    {                                                                                                                \
        const char* wb = wbase + (size_t)(wave + (I) * GD_WAVES) * chunk_stride;                                     \
        _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                                \
            _Pragma("unroll") for (int nt = 0; nt < NT; ++nt) {                                                      \
                if (!H3) A[nt][j] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wb + woff[nt] + 1024 * j));            \
                else A[nt][j] = w_on[nt & 1] ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wb + woff[nt] + 1024 * j))  \
                                             : bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};                                                         \
            }                                                                                                        \
    }
#define GDR_LOAD_X(B, I)                                                                                             \
    {                                                                                                                \
        const char* xb = xbase + (size_t)(wave + (I) * GD_WAVES) * (XT ? 4 * MT * 1024 : GD_CHUNK * 2);              \
        _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                                \
            _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                                        \
                B[mt][j] = *reinterpret_cast<const bf16x8_t*>(xb + xoff[mt] + (XT ? MT * 1024 : 64) * j);            \
    }
#pragma unroll
        for (int i = 0; i < RW; ++i) {
            GDR_LOAD_W(a[i], i)
            if (i < 2) GDR_LOAD_X(b[i], i)
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            GDR_MFMA(a[i % RW], b[i & 1])
            __builtin_amdgcn_sched_barrier(0);
            if (i + 2 < NCH) GDR_LOAD_X(b[i & 1], i + 2)
            if (i + RW < NCH) GDR_LOAD_W(a[i % RW], i + RW)
            __builtin_amdgcn_sched_barrier(0);
        }
#undef GDR_LOAD_X
#undef GDR_LOAD_W
    } else {
        for (int c = wave; c < nfull; c += GD_WAVES) {
            bf16x8_t a[NT][4], b[MT][4];
            GDR_LOAD(a, b, c)
            GDR_MFMA(a, b)
        }
    }
#undef GDR_LOAD
#undef GDR_MFMA
    // ---- add the waves' sums in a fixed order: row tile mt is summed, and its epilogue run, by wave mt ------------------
    static_assert(MT <= GD_WAVES, "a wave per row tile");
    if (SCALED) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) ss_red[(wave * 4 + g) * MP + 16 * mt + r] = ss_part[mt];
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (wave == mt) continue;
        const int slot = wave < mt ? wave : wave - 1;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) red[((slot * NT + nt) * MT + mt) * 64 + lane] = acc[nt][mt];
    }
    __syncthreads();
    if (wave >= MT) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (wave != mt) continue;
#pragma unroll
        for (int w = 0; w < GD_WAVES - 1; ++w)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[nt][mt] += red[((w * NT + nt) * MT + mt) * 64 + lane];
        const int m = 16 * mt + r;
        float scale = 1.f;
        if (SCALED) {
            float s = 0.f;
            for (int i = 0; i < GD_WAVES * 4; ++i) s += ss_red[i * MP + m];
            scale = 1.0f / sqrtf(s / (float)K + eps);
        }
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const int tile = tile0 + ct, n = tile * 16 + 4 * g;
            if (H3 && !(ct == 0 ? (lower || g >= 2) : (!lower || g < 2))) continue;      // the other block's half of the tile
            if (SCALED) {
#pragma unroll
                for (int i = 0; i < 4; ++i) { acc[ct][mt][i] *= scale; if (EPI == EPI_GATED) acc[CT + ct][mt][i] *= scale; }
            }
            if (EPI == EPI_RESID) {
                gd_residual_epilogue<OT>(acc[ct][mt], h_old, wn, resid_out, xw_out, ss_out + tile * MP, m, n, g, M, N, MT);
                continue;
            }
            if (m >= M) continue;
            TC* out = C + (OT ? operand_order(m, n, MT) : (size_t)m * N + n);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float v = acc[ct][mt][i];
                if (EPI == EPI_GATED) { const float up = acc[CT + ct][mt][i]; v = (v / (1.0f + expf(-v))) * up; }
                out[i] = from_f32<TC>(v);
            }
        }
    }
}

// Blocks of 8 waves, one per 16 columns; the gated product (two tiles per block, usually three blocks per CU)
// takes blocks of GD_WAVES_GATED waves so that all of them are resident at once.
int gd_compute_units() {
    static int cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (!cached[dev]) {
        int n = 0;
        cached[dev] = (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) ? n : 256;
    }
    return cached[dev];
}

// false: this combination is not built for the call's number of rows (beyond 64 rows only what a decode step has is built)
template <int EPI, bool SCALED, typename TC, bool XT, bool OT>
static bool gd_launch2(const GdArgs& a) {
    constexpr int W = EPI == EPI_GATED ? GD_WAVES_GATED : 8;
#define GD_ARGS a.x, a.w, (TC*)a.c, a.resid, a.xw_out, a.w_next, a.ss_out, a.ss_in, a.n_parts, a.eps, a.M, a.N, a.K
    // Two column tiles per block where that leaves enough blocks (measured, 64 rows: qkv of 6144 columns 26.8 -> 20.5
    // us; with 4096 columns, 128 blocks, 15.4 -> 19.4 us; the gated product 53 -> 61 us: its block has one wave per SIMD then)
    const bool two = EPI == EPI_STORE && a.N % 32 == 0 && a.N / 32 >= 192;
    // one and a half column tiles per compute unit: three halves of tiles per block (the stored product of a normed input)
    bool halves_rows = false;
    if constexpr (EPI == EPI_STORE && SCALED && XT && !OT && sizeof(TC) == 2) {
        const int cus_ = gd_compute_units();
        halves_rows = a.N % 48 == 0 && (a.N / 24) % cus_ == 0 && (a.N / 16) % cus_ != 0;
    }
    // beyond four row tiles: blocks of eight waves (a wave per row tile runs the epilogue), one column tile; built for
    // what a decode step has: inputs in operand order, the residual product of a plain input with its output in operand
    // order, the stored product of a normed input
    constexpr bool TALL = XT && ((EPI == EPI_RESID && !SCALED && OT) || (EPI == EPI_STORE && SCALED));
    // With up to eight chunks of K per wave, and three row tiles or more, the chunks run in straight-line code behind a ring of
    // loads (measured, 4096 x 4096 and 6144 x 4096: 10.9 / 12.1 us against 11.7 / 13.5 and 14.8 / 16.3 against 15.5 / 17.8 at 48
    // / 64 rows; at 24 and 32 rows the loop is as fast or faster: 8.9 / 9.8 and 12.2 / 13.2 against 9.4 / 9.4 and 13.6 / 13.6).
    // What bounds these products from three row tiles on is the L2's throughput: every block pulls all of X through it.
    const int nch = (EPI != EPI_GATED && a.K % (GD_CHUNK * W) == 0 && a.K / (GD_CHUNK * W) <= 8) ? a.K / (GD_CHUNK * W) : 0;
    if (a.M <= 16) {
        // one and a half column tiles per compute unit: three halves of tiles per block
        bool halves = false;
        if constexpr (EPI == EPI_STORE && SCALED && XT && !OT && sizeof(TC) == 2) {
            const int cus = gd_compute_units();
            const bool uneven = (a.N / 16) % cus != 0;
            if (uneven && a.N % 48 == 0 && (a.N / 24) % cus == 0) {
                gemm_decode_kernel<EPI, SCALED, TC, W, XT, OT, 3><<<a.N / 24, W * 64, 0, a.st>>>(GD_ARGS);
                halves = true;
            } else if (uneven && a.N % 80 == 0 && (a.N / 40) % cus == 0) {
                gemm_decode_kernel<EPI, SCALED, TC, W, XT, OT, 5><<<a.N / 40, W * 64, 0, a.st>>>(GD_ARGS);
                halves = true;
            }
        }
        if (!halves) gemm_decode_kernel<EPI, SCALED, TC, W, XT, OT><<<a.N / 16, W * 64, 0, a.st>>>(GD_ARGS);
    }
#define GD_ROWS_N(MT, CT, H3, BLOCKS, NCH) gemm_decode_rows_kernel<EPI, SCALED, TC, MT, CT, W, XT, OT, H3, NCH><<<BLOCKS, W * 64, 0, a.st>>>(GD_ARGS)
#define GD_ROWS_PICK(MT, CT, H3, BLOCKS)                                                                             \
    if constexpr (EPI != EPI_GATED && MT >= 3) {                                                                     \
        switch (nch) {                                                                                               \
        case 4: GD_ROWS_N(MT, CT, H3, BLOCKS, 4); break;                                                             \
        case 5: GD_ROWS_N(MT, CT, H3, BLOCKS, 5); break;                                                             \
        case 8: GD_ROWS_N(MT, CT, H3, BLOCKS, 8); break;                                                             \
        default: GD_ROWS_N(MT, CT, H3, BLOCKS, 0);                                                                   \
        }                                                                                                            \
    } else GD_ROWS_N(MT, CT, H3, BLOCKS, 0)
#define GD_ROWS_ONE(MT) GD_ROWS_PICK(MT, 1, false, a.N / 16)
#define GD_ROWS(MT)                                                                                                  \
    if constexpr (EPI == EPI_STORE) {                                                                                \
        if (halves_rows) { GD_ROWS_PICK(MT, 2, true, a.N / 24); }                                                    \
        else if (two) { GD_ROWS_PICK(MT, 2, false, a.N / 32); }                                                      \
        else GD_ROWS_ONE(MT);                                                                                        \
    } else GD_ROWS_ONE(MT)
#define GD_ROWS_TALL(MT)                                                                                             \
    if constexpr (TALL) gemm_decode_rows_kernel<EPI, SCALED, TC, MT, 1, 8, XT, OT><<<a.N / 16, 512, 0, a.st>>>(GD_ARGS); \
    else return false;
    else if (a.M <= 32) { GD_ROWS(2); }
    else if (a.M <= 48) { GD_ROWS(3); }
    else if (a.M <= 64) { GD_ROWS(4); }
    else if (a.M <= 96) { GD_ROWS_TALL(6) }
    else { GD_ROWS_TALL(8) }
#undef GD_ROWS_TALL
#undef GD_ROWS
#undef GD_ROWS_ONE
#undef GD_ROWS_PICK
#undef GD_ROWS_N
#undef GD_ARGS
    return true;
}

template <int EPI, bool SCALED, typename TC>
static bool gd_launch(const GdArgs& a) {
    constexpr bool CAN_OT = EPI != EPI_STORE && sizeof(TC) == 2;      // operand order is for bfloat16 that a product reads next
    if (a.xt) return (CAN_OT && a.ot) ? gd_launch2<EPI, SCALED, TC, true, CAN_OT>(a) : gd_launch2<EPI, SCALED, TC, true, false>(a);
    return (CAN_OT && a.ot) ? gd_launch2<EPI, SCALED, TC, false, CAN_OT>(a) : gd_launch2<EPI, SCALED, TC, false, false>(a);
}

// Bytes of the device's workspace for the products that split K over blocks: zeroed once by the caller, then handed to
// every call on that device (ws; none: those products are not taken).  Calls on one device that overlap race on it.
extern "C" int64_t spy_gemm_decode_workspace() { return gd_splitk_workspace_bytes(); }

// x: bfloat16 [M, K], M <= 128; MP = 16 times the row tiles the kernel is built with (M rounded up to 16 up to 64 rows, 96
// or 128 beyond).  scaled != 0: x = bf16(h * w_norm) and ss_in
// [n_parts, MP] holds the parts of sum(h^2); the result is multiplied by rsqrt(sum / K + eps).
// epi 0: C [M, N] (c_dtype);  epi 1: W = [gate | up], C [M, N] = silu(gate) * up;  epi 2: resid [M, N] += result,
// xw_out [M, N] = bf16(resid * w_next), ss_out [N / 16, MP] = every block's part of the rows' sums of squares.
// x_tiled / out_tiled: X / the bfloat16 output for the next product (xw_out of epi 2, C of epi 1) are in operand order.
extern "C" int spy_gemm_decode(const void* X, int scaled, const float* ss_in, int n_parts, float eps, const void* Wt, int epi,
                               void* C, int c_dtype, float* resid, void* xw_out, const void* w_next, float* ss_out, int M, int N,
                               int K, int x_tiled, int out_tiled, void* ws, int64_t ws_bytes, hipStream_t st) {
    SPY_REQUIRE(M > 0 && M <= 128, "spy_gemm_decode: M = %d rows (1..128 allowed)", M);
    SPY_REQUIRE(N > 0 && N % 16 == 0 && K > 0 && K % 128 == 0, "spy_gemm_decode: N = %d must be a multiple of 16 and K = %d of 128", N, K);
    SPY_REQUIRE(epi >= 0 && epi <= 2, "spy_gemm_decode: unknown epilogue %d", epi);
    SPY_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)Wt % 16) == 0, "spy_gemm_decode: operands must be 16-byte aligned");
    SPY_REQUIRE(!scaled || (ss_in && n_parts > 0), "spy_gemm_decode: the scale needs the parts of the sums of squares");
    SPY_REQUIRE(epi != EPI_RESID || (resid && ss_out && xw_out && w_next && ((uintptr_t)resid % 16) == 0 &&
                                     ((uintptr_t)xw_out % 8) == 0 && ((uintptr_t)w_next % 8) == 0),
                "spy_gemm_decode: the residual epilogue needs the stream, the next norm's weight and its outputs");
    SPY_REQUIRE(epi == EPI_RESID || (C && ((uintptr_t)C % 16) == 0), "spy_gemm_decode: no output");
    SPY_REQUIRE((long long)N * 256 + 8192 < (1ll << 32), "spy_gemm_decode: N = %d is too large for 32-bit offsets inside a chunk", N);
    SPY_REQUIRE(!out_tiled || (N % 32 == 0 && (epi == EPI_RESID || (epi == EPI_GATED && c_dtype == SPY_BF16))),
                "spy_gemm_decode: operand order is for the bfloat16 output of the gated and the residual epilogue, N a multiple of 32");
    GdArgs a = {(const bf16_t*)X, (const bf16_t*)Wt, C, resid, (bf16_t*)xw_out, (const bf16_t*)w_next, ss_out, ss_in, n_parts, eps, M, N, K,
                x_tiled != 0, out_tiled != 0, st, ws, (long long)ws_bytes};
    const bool f32 = c_dtype == SPY_F32;
    if (gd_splitk_try(a, epi, scaled != 0, f32) || gd_wide_try(a, epi, scaled != 0, f32)) {
        SPY_CHECK_LAUNCH("spy_gemm_decode");
        return 0;
    }
    bool built;
    if (epi == EPI_RESID) built = scaled ? gd_launch<EPI_RESID, true, bf16_t>(a) : gd_launch<EPI_RESID, false, bf16_t>(a);
    else if (epi == EPI_GATED) {
        if (scaled) built = f32 ? gd_launch<EPI_GATED, true, float>(a) : gd_launch<EPI_GATED, true, bf16_t>(a);
        else built = f32 ? gd_launch<EPI_GATED, false, float>(a) : gd_launch<EPI_GATED, false, bf16_t>(a);
    } else {
        if (scaled) built = f32 ? gd_launch<EPI_STORE, true, float>(a) : gd_launch<EPI_STORE, true, bf16_t>(a);
        else built = f32 ? gd_launch<EPI_STORE, false, float>(a) : gd_launch<EPI_STORE, false, bf16_t>(a);
    }
    SPY_REQUIRE(built, "spy_gemm_decode: %d rows: beyond 64 rows the product is built for inputs in operand order only, as the stored or "
                "gated product of a normed input or the residual product of a plain input with its output in operand order", M);
    SPY_CHECK_LAUNCH("spy_gemm_decode");
    return 0;
}
