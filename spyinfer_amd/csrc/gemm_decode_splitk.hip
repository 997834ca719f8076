// Decode products of 33 to 128 rows for matrices with about one column tile of 16 per compute unit (o, down, qkv).
//
// With a column tile per block every block pulls all of X through L2, MT row tiles against one tile of W: MT times the
// bytes of W, and the L2's throughput bounds the product, not the matrix' way from memory.  Sharing the X fragments
// between several column tiles of a block (as for the gated product) leaves too few blocks here.  So K is split over
// blocks as well: block (column group cg, part ks) has CT neighbouring column tiles and the chunks [nfull ks / KS,
// nfull (ks + 1) / KS) of K; it reads 1 / KS of X against CT tiles of W, and X's traffic falls from MT to MT / CT
// times W's.  The block's 8 waves split its chunks and add through LDS in a fixed order, in two rounds, after which
// four waves have the block's sums, each every fourth (column tile, row tile) unit; they write them to the workspace.
// The block that finishes a column group last (a counter per group) adds the group's KS parts in the order of ks and
// runs the epilogue, so the result does not depend on which block that is.  It leaves the counter at zero for the
// next call.
//
// The dies' L2s are not coherent with each other inside a kernel, and the fences that make them so (write back and
// invalidate the whole L2) cost about 30 us per call here.  So the parts are written through the caches (stores of
// system scope), waited for before the block's barrier and its count, and read past the caches (loads of system
// scope); the counter is an atomic of device scope.  Everything else is read and written as usual.
//
// The workspace (counters, then the parts) belongs to the device and is shared by all calls: it starts zeroed, and
// calls that overlap on two streams of one device race.
#include "gemm_decode.h"
#include <math.h>

#define SK_COUNTER_BYTES 16384            // 4096 column groups at most
#define SK_MAX_TILES_PER_BLOCK 32         // CT * MT at most
#define SK_MAX_PARTS 8                    // parts of K at most

// GW: waves per block, 8 up to four row tiles, 4 beyond (a wave then has a SIMD's registers to itself).
template <int EPI, bool SCALED, typename TC, int MT, int CT, bool XT, bool OT, int GW = 8>
__global__ __launch_bounds__(GW * 64, 1) void gemm_decode_splitk_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ Wt, TC* __restrict__ C, float* __restrict__ resid_out,
    bf16_t* __restrict__ xw_out, const bf16_t* __restrict__ w_next, float* __restrict__ ss_out, const float* __restrict__ ss_in,
    int n_parts, float eps, int M, int N, int K, int KS, unsigned* counters, float* parts) {
    static_assert(EPI == EPI_STORE || EPI == EPI_RESID, "store and residual epilogues");
    static_assert(GW == 8 || GW == 4, "four or eight waves");
    static_assert(CT * MT <= (GW == 8 ? 16 : SK_MAX_TILES_PER_BLOCK), "the sums must fit the registers and the workspace");
    constexpr int MP = 16 * MT;
    constexpr int PAIRS = CT * MT;                       // (column tile, row tile) units: p = ct MT + mt, owned by wave p % 4
    constexpr int MINE = (PAIRS + 3) / 4;                // units of a wave at most
    // the waves' sums meet in two rounds: waves 4..7 hand all of theirs to waves 0..3, then each of these four takes
    // every fourth unit from the other three.  The second round's buffer lies inside the first's.
    __shared__ f32x4_t red[(GW == 8 ? 4 : 3) * PAIRS * 64];
    __shared__ float ss_red[SCALED ? GW * 4 * MP : 1];
    __shared__ float row_scale[SCALED ? MP : 1];
    __shared__ unsigned is_last;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    // neighbouring blocks, which go to different dies, have different parts of K: a die's L2 then holds 1 / KS of X
    const int cg = blockIdx.x / KS, ks = blockIdx.x % KS;
    const int tiles = N / 16;
    const int t0 = cg * CT;
    const int here = min(CT, tiles - t0);              // the last group may have fewer tiles

    // What the epilogue needs beside the sums is asked for now, by every block (any may be the last of its group, and
    // that one's chain of round trips is long enough: parts out, count, parts in): the old values of the stream and the
    // next norm's weight for this wave's units, and this thread's share of the rows' sums of squares.
    f32x4_t h_old[MINE];
    uint2 wn[MINE];
    if (EPI == EPI_RESID && wave < 4) {
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) {
            if ((p & 3) != wave) continue;
            const int ct = p / MT, m = 16 * (p % MT) + r, n = (t0 + ct) * 16 + 4 * g;
            const bool ok = ct < here && m < M;
            h_old[p / 4] = ok ? *reinterpret_cast<const f32x4_t*>(resid_out + (size_t)m * N + n) : f32x4_t{0.f, 0.f, 0.f, 0.f};
            wn[p / 4] = ct < here ? *reinterpret_cast<const uint2*>(w_next + n) : uint2{0u, 0u};
        }
    }
    float ss_part[MT];
    if (SCALED) gd_ss_share<MT, GW * 4>(ss_in, n_parts, wave * 4 + g, r, ss_part);

    const size_t chunk_stride = (size_t)tiles * 4096;
    unsigned xoff[MT];                // (rows beyond M: the last row's address, or the operand order's padding)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        xoff[mt] = XT ? (unsigned)mt * 1024u + 16u * lane : (unsigned)min(16 * mt + r, M - 1) * (unsigned)K * 2u + 16u * g;
    }
    const char* xbase = reinterpret_cast<const char*>(X);
    const int nfull = K / GD_CHUNK;
    const int c_begin = (int)((long long)nfull * ks / KS), c_end = (int)((long long)nfull * (ks + 1) / KS);
    const int my_steps = c_begin + wave < c_end ? 4 * ((c_end - c_begin - wave + GW - 1) / GW) : 0;   // steps of 32 of K

    f32x4_t acc[CT][MT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[ct][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const char* wbase = reinterpret_cast<const char*>(Wt) + (size_t)t0 * 4096 + 16u * lane;
    {
        // A ring of four steps' operands: three steps are under way while one is multiplied, so that a compute unit keeps
        // enough of the matrix in flight to cover the memory's latency (with one step under way the product of 64 rows
        // streamed at half the memory's rate).  What keeps the ring full in the compiled code: every load is
        // unconditional (rows of X beyond M are read from the last row, or from the padding of the operand order; their
        // sums are never stored), and the last four steps, which ask for nothing more, are peeled from the loop.  A load
        // under a condition makes the compiler count the loads in flight as the fewest there may be, and a load that the
        // loop's last turn skips makes it wait for all of them in every turn.
        bf16x8_t a0[CT], b0[MT], a1[CT], b1[MT], a2[CT], b2[MT], a3[CT], b3[MT];
#define SK_LOAD(A, B, STEP)                                                                                          \
        {                                                                                                            \
            const int c_ = c_begin + wave + GW * ((STEP) >> 2), h_ = (STEP) & 3;                                     \
            const char* wb = wbase + (size_t)c_ * chunk_stride;                                                      \
            const char* xb = xbase + (size_t)c_ * (XT ? 4 * MT * 1024 : GD_CHUNK * 2);                               \
            _Pragma("unroll") for (int ct = 0; ct < CT; ++ct) {                                                      \
                /* a tile that the group does not have reads the group's first tile again (its sums are dropped) */  \
                const int t = ct < here ? ct : 0;                                                                    \
                A[ct] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wb + (size_t)t * 4096 + 1024 * h_)); \
            }                                                                                                        \
            _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                                        \
                B[mt] = *reinterpret_cast<const bf16x8_t*>(xb + xoff[mt] + (XT ? MT * 1024 : 64) * h_);              \
        }
#define SK_MFMA(A, B)                                                                                                \
        _Pragma("unroll") for (int ct = 0; ct < CT; ++ct)                                                            \
            _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                                        \
                acc[ct][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[ct], B[mt], acc[ct][mt], 0, 0, 0);
        if (my_steps > 0) {                                 // (a multiple of 4)
            SK_LOAD(a0, b0, 0) SK_LOAD(a1, b1, 1) SK_LOAD(a2, b2, 2)
            int st = 0;
            // (the scheduling barriers keep the compiler from sinking the loads below the products, which would let the
            // queue of loads run empty once per turn)
#define SK_FENCE __builtin_amdgcn_sched_barrier(0);
            for (; st + 4 < my_steps; st += 4) {
                SK_LOAD(a3, b3, st + 3) SK_FENCE
                SK_MFMA(a0, b0) SK_FENCE
                SK_LOAD(a0, b0, st + 4) SK_FENCE
                SK_MFMA(a1, b1) SK_FENCE
                SK_LOAD(a1, b1, st + 5) SK_FENCE
                SK_MFMA(a2, b2) SK_FENCE
                SK_LOAD(a2, b2, st + 6) SK_FENCE
                SK_MFMA(a3, b3) SK_FENCE
            }
            SK_LOAD(a3, b3, st + 3) SK_FENCE
            SK_MFMA(a0, b0) SK_FENCE
            SK_MFMA(a1, b1) SK_FENCE
            SK_MFMA(a2, b2) SK_FENCE
            SK_MFMA(a3, b3)
#undef SK_FENCE
        }
#undef SK_LOAD
#undef SK_MFMA
    }
    // ---- round one: the upper four waves' sums to the lower four ------------------------------------------------------
    if (SCALED) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) ss_red[(wave * 4 + g) * MP + 16 * mt + r] = ss_part[mt];
    }
    if (GW == 8 && wave >= 4) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) red[(((wave - 4) * CT + ct) * MT + mt) * 64 + lane] = acc[ct][mt];
    }
    if (GW == 8 || SCALED) __syncthreads();
    const int t_scale = (int)threadIdx.x - (GW == 8 ? 256 : 0);        // (a wave that has nothing to add now, if there is one)
    if (SCALED && t_scale >= 0 && t_scale < MP) {
        float s = 0.f;
        for (int i = 0; i < GW * 4; ++i) s += ss_red[i * MP + t_scale];
        row_scale[t_scale] = 1.0f / sqrtf(s / (float)K + eps);
    }
    if (GW == 8 && wave < 4) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[ct][mt] += red[((wave * CT + ct) * MT + mt) * 64 + lane];
    }
    if (GW == 8 || SCALED) __syncthreads();
    // ---- round two: unit p to wave p % 4 ---------------------------------------------------------------------------------
    if (wave < 4) {
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) {
            const int owner = p & 3;
            if (wave != owner) red[(p * 3 + (wave < owner ? wave : wave - 1)) * 64 + lane] = acc[p / MT][p % MT];
        }
    }
    __syncthreads();
    // ---- the block's sums to the workspace: parts [block][unit][4][64 lanes] ----------------------------------------------
    if (wave < 4) {
        float* const mine = parts + (size_t)blockIdx.x * PAIRS * 256 + lane;
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) {
            if ((p & 3) != wave) continue;
            f32x4_t v = acc[p / MT][p % MT];
#pragma unroll
            for (int slot = 0; slot < 3; ++slot) v += red[(p * 3 + slot) * 64 + lane];
#pragma unroll
            for (int i = 0; i < 4; ++i) __hip_atomic_store(mine + (p * 4 + i) * 64, v[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        // ORDER (as at the attention's merge of key parts): no release/acquire pair, which this compiler turns into a
        // write-back and invalidation of the whole L2 (30 us a call).  Instead: the stores of system scope write through
        // every cache and have reached memory when vmcnt has counted them, which this wait is for; the barrier puts all
        // waves' waits before thread 0's increment, an atomic of device scope that all dies execute at one place; the last block's loads of system scope
        // read past the caches, after the barrier behind the increment.  Ordinary stores or loads here would be wrong.
        __builtin_amdgcn_s_waitcnt(0);                     // the stores have arrived before the block counts itself done
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned before = __hip_atomic_fetch_add(&counters[cg], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last = before == (unsigned)KS - 1u;
        // every block of the group has counted: zero for the next call
        if (before == (unsigned)KS - 1u) __hip_atomic_store(&counters[cg], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!is_last || wave >= 4) return;
    // ---- the last block of the group: the parts in the order of ks, then the epilogue of this wave's units ------------------
    // (all of this wave's share of the parts is asked for before any of it is used: one memory round trip, where a loop
    // that adds as it loads has one per part)
    float pv[MINE][SK_MAX_PARTS][4];
#pragma unroll
    for (int p = 0; p < PAIRS; ++p) {
        if ((p & 3) != wave) continue;
        const float* q = parts + ((size_t)cg * KS * PAIRS + p) * 256 + lane;
#pragma unroll
        for (int k = 0; k < SK_MAX_PARTS; ++k)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                pv[p / 4][k][i] = k < KS ? __hip_atomic_load(q + (size_t)k * PAIRS * 256 + i * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) : 0.f;
    }
#pragma unroll
    for (int p = 0; p < PAIRS; ++p) {
        if ((p & 3) != wave) continue;
        const int ct = p / MT, mt = p % MT;
        if (ct >= here) continue;
        f32x4_t v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < SK_MAX_PARTS; ++k)
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] += pv[p / 4][k][i];
        const int tile = t0 + ct, n = tile * 16 + 4 * g, m = 16 * mt + r;
        if (SCALED) {
            const float scale = row_scale[m];
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] *= scale;
        }
        if (EPI == EPI_RESID) {
            gd_residual_epilogue<OT>(v, h_old[p / 4], wn[p / 4], resid_out, xw_out, ss_out + tile * MP, m, n, g, M, N, MT);
            continue;
        }
        if (m >= M) continue;
        TC* out = C + (size_t)m * N + n;
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i] = from_f32<TC>(v[i]);
    }
}

long long gd_splitk_workspace_bytes() {
    return SK_COUNTER_BYTES + (long long)gd_compute_units() * SK_MAX_TILES_PER_BLOCK * 1024;
}

constexpr int SK_MIN_CHUNKS = 12;    // chunks of K that a part has at least (three for every two waves of eight)
constexpr int SK_MIN_FILL = 85;      // per cent of the compute units that must get a block (qkv of 7168 x 5120, 448 tiles, in 224
                                     // blocks: 32.7 against 41.4 us at 96 rows)
constexpr int SK_EVEN_FILL = 85;     // per cent of the blocks' turns that a tile per block must fill to stand up to 32 rows
constexpr int SK_STORE_FROM = 64;    // rows beyond which the stored product splits K

// Column tiles per block and parts of K: the pair that gives the most compute units a block, a part with at least 12
// chunks of K for its 8 waves (with one chunk per wave the way of the parts through memory costs more than X's traffic:
// the o product of 4096 x 4096 at 64 rows took 17.3 us in four parts against 15.1 with a column tile per block; with 13
// chunks a part, 5120 x 5120 in three parts, 20.1 against 28.3; down, 4096 x 12288, 27.6 against 35.1, and qkv,
// 6144 x 4096 in two parts, 18.6 against 19.3); among equals the most column tiles.
static void sk_shape(int tiles, int nfull, int cus, int* ct_out, int* ks_out) {
    int best_ct = 0, best_ks = 0, best_blocks = 0;
    for (int ct = 4; ct >= 3; --ct) {
        const int groups = (tiles + ct - 1) / ct;
        int ks = cus / groups;
        if (ks > nfull / SK_MIN_CHUNKS) ks = nfull / SK_MIN_CHUNKS;
        if (ks > SK_MAX_PARTS) ks = SK_MAX_PARTS;
        if (ks < 2 || groups * ks * 100 < cus * SK_MIN_FILL) continue;
        if (groups * ks > best_blocks) { best_blocks = groups * ks; best_ct = ct; best_ks = ks; }
    }
    *ct_out = best_ct;
    *ks_out = best_ks;
}

template <int EPI, bool SCALED, typename TC, int MT, bool XT, bool OT>
static bool sk_launch(const GdArgs& a) {
    const int cus = gd_compute_units(), tiles = a.N / 16, nfull = a.K / GD_CHUNK;
    int ct = 0, ks = 0;
    sk_shape(tiles, nfull, cus, &ct, &ks);
    if (ct == 0) return false;
    const int groups = (tiles + ct - 1) / ct;
    if (groups * 4 > SK_COUNTER_BYTES || (long long)groups * ks > cus) return false;
    if (a.ws_bytes < gd_splitk_workspace_bytes()) return false;
    unsigned* counters = reinterpret_cast<unsigned*>(a.ws);
    float* parts = reinterpret_cast<float*>(reinterpret_cast<char*>(a.ws) + SK_COUNTER_BYTES);
    constexpr int GW = MT > 4 ? 4 : 8;
#define SK_CASE(C)                                                                                                      \
    if (ct == C) {                                                                                                      \
        gemm_decode_splitk_kernel<EPI, SCALED, TC, MT, C, XT, OT, GW><<<groups * ks, GW * 64, 0, a.st>>>(                \
            a.x, a.w, (TC*)a.c, a.resid, a.xw_out, a.w_next, a.ss_out, a.ss_in, a.n_parts, a.eps, a.M, a.N, a.K, ks, counters, parts); \
        return true;                                                                                                    \
    }
    SK_CASE(3) SK_CASE(4)
#undef SK_CASE
    return false;
}

template <int EPI, bool SCALED, typename TC, bool XT, bool OT>
static bool sk_rows(const GdArgs& a) {
    if constexpr (XT) {                                   // (beyond 64 rows: inputs in operand order only)
        if (a.M > 96) return sk_launch<EPI, SCALED, TC, 8, XT, OT>(a);
        if (a.M > 64) return sk_launch<EPI, SCALED, TC, 6, XT, OT>(a);
    }
    if (a.M > 64) return false;
    if (a.M > 48) return sk_launch<EPI, SCALED, TC, 4, XT, OT>(a);
    if (a.M > 32) return sk_launch<EPI, SCALED, TC, 3, XT, OT>(a);
    if constexpr (EPI == EPI_RESID) {                     // (one and two row tiles: the residual product only)
        if (a.M > 16) return sk_launch<EPI, SCALED, TC, 2, XT, OT>(a);
        return sk_launch<EPI, SCALED, TC, 1, XT, OT>(a);
    }
    return false;
}

// Built for the combinations that a decode step has: the residual product of a plain input (row-major or in operand
// order) with its output in operand order, and the stored bfloat16 product of a normed input in operand order.
bool gd_splitk_try(const GdArgs& a, int epi, bool scaled, bool f32_out) {
    if (a.ws == nullptr || a.M > 128 || a.N % 16 != 0 || a.K % GD_CHUNK != 0) return false;
    const int cus = gd_compute_units(), tiles = a.N / 16;
    if (tiles >= 2 * cus) return false;                             // many columns: the kernels that walk column tiles
    // Up to 32 rows the kernels with a column tile per block are as fast where their blocks fill the compute units evenly
    // (256 tiles: down, 4096 x 12288, 23.5 against 23.6 us at 32 rows).  Where the last turn of blocks is short (320 tiles
    // on 256 compute units: some units stream two tiles, the others one), equal parts for all pay from the first row on:
    // down of 5120 x 25600 55.9 / 65.6 / 77.0 us at 8 / 16 / 24 rows with a tile per block, against 50.7 at 40 rows here.
    // (Fewer tiles than units and few rows: no unit streams two tiles, and the parts' way through memory costs what the
    // idle units would save: down of 2560 x 9728, 160 tiles, 13.5 against 12.4 us at 8 rows, 13.4 against 14.9 at 16.)
    if (a.M <= 32) {
        const int turns = (tiles + cus - 1) / cus;
        if (tiles * 100 >= turns * cus * SK_EVEN_FILL || (a.M <= 8 && turns == 1)) return false;
    }
    if (epi == EPI_RESID && !scaled && a.ot) {
        return a.xt ? sk_rows<EPI_RESID, false, bf16_t, true, true>(a) : sk_rows<EPI_RESID, false, bf16_t, false, true>(a);
    }
    // (the stored product, qkv of 6144 x 4096, 384 tiles: up to 8 rows a tile per block takes 11.4 us against 12.6 in two parts,
    // 13.0 against 12.7 at 16; from 17 to 64 rows the kernel with two column tiles per block is as fast or faster,
    // 15.2 against 17.3 us at 33 rows, 16.1 against 17.6 at 48, 18.2 against 18.1 at 64; beyond, 31.1 against 24.2 at 80)
    if (epi == EPI_STORE && scaled && a.xt && !f32_out && !a.ot && a.M > SK_STORE_FROM) return sk_rows<EPI_STORE, true, bf16_t, true, false>(a);
    return false;
}
