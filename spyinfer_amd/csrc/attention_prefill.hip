// Paged attention on MFMA for entries with many query rows (prompt portions): a block works on 128 rows of one entry
// and one kv head, as 8 waves of one 16-row MFMA tile each (head sizes 64 and 128) or 4 waves of two tiles each (the
// other head sizes).  Rows are (token, query head of the group) pairs as in attention_mfma.hip.  Keys and values of
// 64 keys at a time are gathered through the block table into LDS once per block (prefetched into registers while
// the previous 64 keys are worked on) and shared by the 8 row tiles; with two row tiles per wave every K and V
// fragment that a wave reads from LDS serves both.
//
// MFMA arrangement as in attention_mfma.hip: S^T = K . Q^T in two tiles whose key order leaves
// lane (q row, g) with the scores of 8 consecutive keys, which are exactly the 8 k-values that
// lane must supply of P^T in O^T += V^T . P^T.  In LDS the keys of a 32-key half are stored in the
// order the two S^T tiles read them (rows 0..15 tile a, 16..31 tile b), which makes the 16-byte
// reads of 16 lanes hit 16 different bank groups.
#include "common.h"
#include "attention_merge.h"
#include <math.h>

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define PF_KEYS 64       // keys staged per round
#define PF_DIES 8        // dies (XCDs) of the chip, each with its own L2; blocks go to them in turn
#define PF_SLACK 8.0f    // a score may exceed the running maximum by 2^8 before the maximum is raised

__device__ __forceinline__ bf16x8_t pf_zero8() { return bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0}; }

// DFULL: head_dim == DMAX, so no part of the head-dim loops is conditional and the compiler may move the LDS reads of
// a whole 32-key half ahead of its products.
// RT: 16-row tiles per wave.  2 (4 waves per block): every K and V fragment read from LDS serves two row tiles, but a
// SIMD has one wave per block and little to run while it waits.  1 (8 waves per block): two waves per SIMD and block.
// MINW: waves per SIMD that the registers must allow.  The 8-wave shape with 4 (128 registers, two blocks per CU) is
// the fastest shape for grids of more than one block per CU; with one block per CU it is 6 % faster with the
// registers of 2.
// PF_ROWS: rows per block, 128 or 256.  With 256 rows (8 waves of two row tiles) a round's keys and values are staged
// once for twice the rows: half the staging instructions and half the LDS reads per score of the 128-row shapes.
template <int DMAX, bool DFULL, int RT, int MINW, int PF_ROWS>
__global__ __launch_bounds__(PF_ROWS / RT * 4, MINW) void attention_prefill_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
    int P, int num_pages, const int* __restrict__ cu_q, const int* __restrict__ pos0, const int* __restrict__ kv_len,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ tile_entry, const int* __restrict__ tile_row0,
    int n_q, int n_kv, int d, float scale, int window, int log2p, int num_tiles, int splits, float* __restrict__ ws, int out_tiles) {
    constexpr int KK = DMAX / 32, DT = DMAX / 16;
    // 16 elements of padding per staged row: the products' 16-byte reads then have no bank conflicts (measured with
    // SQ_LDS_BANK_CONFLICT: 40 % of the LDS cycles with 8, none with 16; the kernel's time follows only by 0-3 %)
    constexpr int KLD = DMAX + 16;           // bf16 per staged key row
    constexpr int VLD = PF_KEYS + 16;        // bf16 per staged value row (one head dim, 64 keys)
    constexpr int NT = PF_ROWS / RT * 4;        // threads per block: a wave per 16 RT rows
    constexpr int NV = PF_KEYS * DMAX / 8 / NT; // 16-byte vectors per thread and operand per round
    __shared__ __attribute__((aligned(16))) bf16_t ks[PF_KEYS * KLD];
    __shared__ __attribute__((aligned(16))) bf16_t vs[DMAX * VLD];

    // A block works on two tiles, one after the other: tile b and tile n - 1 - b of a list that the host
    // has sorted by the number of keys a tile reads.  So every block has about the same work, which a
    // causal prompt's tiles alone (few keys early, many late) do not give.
    // Blocks go to the chip's 8 dies in turn, by their number in the grid, and each die has an L2 of its own.  So the
    // grid's numbers are dealt out again: a die gets a run of blocks that follow each other in (part, kv head, tile)
    // order, which read the same head's keys and values, and these stay in that die's L2 (with 8 kv heads a die has one
    // head; dealt out plainly, every die reads every head).  Measured, 32 query heads of 128 in 8 groups: 73.9 -> 71.1
    // us at 2048 tokens, 176 -> 168 at 4096, 618 -> 602 at 8192, 2376 -> 2320 at 16384.
    int bx, hk, part;
    {
        const int gx = gridDim.x, gy = gridDim.y, n = gx * gy * (int)gridDim.z;
        const int lin = blockIdx.x + gx * (blockIdx.y + gy * blockIdx.z);
        const int die = lin % PF_DIES, idx = lin / PF_DIES;
        const int per = (n + PF_DIES - 1) / PF_DIES, rem = n % PF_DIES;      // the first rem dies have per blocks, the others one fewer
        const int v = (rem == 0 || die < rem) ? die * per + idx : rem * per + (die - rem) * (per - 1) + idx;
        bx = v % gx;
        hk = (v / gx) % gy;
        part = v / (gx * gy);
    }
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, r16 = lane & 15, g = lane >> 4;
    // With key parts (splits > 1: few tiles, many keys, e.g. a late portion of a long prompt) a block has one
    // tile and the rounds of one part; the parts are merged by attention_merge_kernel.
    for (int which = 0; which < 2; ++which) {
    const int tile = which == 0 ? bx : num_tiles - 1 - bx;
    if (which == 1 && (splits > 1 || tile <= bx)) break;
    __syncthreads();                                   // the first tile's last readers of LDS are done
    const int s = tile_entry[tile];
    const int row0 = tile_row0[tile];
    const int G = n_q / n_kv;
    const int q0 = cu_q[s];
    const int nrows = (cu_q[s + 1] - q0) * G;
    const int p0 = pos0[s];
    const int kvl = kv_len[s];
    const int* bt = block_table + (size_t)s * max_blocks;
    const int d8 = d >> 3;

    // this lane's two query rows
    bool row_ok[RT];
    int tq[RT], head[RT], pos[RT], lo_row[RT];
    bf16x8_t bq[RT][KK];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int row = row0 + 16 * RT * wave + 16 * t + r16;
        row_ok[t] = row < nrows;
        tq[t] = row_ok[t] ? row / G : 0;
        head[t] = hk * G + (row_ok[t] ? row % G : 0);
        pos[t] = p0 + tq[t];
        lo_row[t] = window > 0 ? max(0, pos[t] - window + 1) : 0;
        const bf16_t* qp = q + ((size_t)(q0 + tq[t]) * n_q + head[t]) * d;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const int dofs = kk * 32 + 8 * g;
            bq[t][kk] = (row_ok[t] && dofs < d) ? *reinterpret_cast<const bf16x8_t*>(qp + dofs) : pf_zero8();
        }
    }
    // keys the block can see, and those this wave can see (wave-uniform)
    const int blk_last_row = min(nrows, row0 + PF_ROWS) - 1;
    const int hi = min(p0 + blk_last_row / G, kvl - 1);
    int lo = window > 0 ? max(0, p0 + row0 / G - window + 1) : 0;
    lo &= ~(PF_KEYS - 1);
    const int nblk = hi >= lo ? (hi - lo) / PF_KEYS + 1 : 0;
    const int w_first_row = row0 + 16 * RT * wave;
    const int w_last_row = min(nrows, w_first_row + 16 * RT) - 1;
    const int w_hi = w_last_row >= w_first_row ? p0 + w_last_row / G : -1;               // last key any row of the wave reads
    const int w_lo = window > 0 ? max(0, p0 + w_first_row / G - window + 1) : 0;           // first key any row of the wave reads
    const bool w_rows_full = w_first_row + 16 * RT - 1 < nrows;                             // all rows of the wave exist
    const int w_min_pos = p0 + w_first_row / G;                                            // keys up to here are before every row
    const int w_max_lo = window > 0 ? max(0, w_hi - window + 1) : 0;                       // keys from here on are in every window
    const float scale2 = scale * 1.4426950408889634f;                                      // scores times log2(e)

    f32x4_t acc[RT][DT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[t][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m[RT], l[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) { m[t] = -INFINITY; l[t] = 0.f; }

    bf16x8_t pk[NV], pv[NV];
    int kpg[NV], vpg[NV];        // pages of this thread's vectors, looked up one round ahead of the data
    // vector v = tid + NT i of a round:  K: key = v / d8, chunk = v % d8 (16 bytes of one key row)
    //                                     V: kgrp = v % 8, dd = v / 8     (8 keys of one head dim)
    // What does not change from round to round is worked out once: the local key, the offsets inside a
    // page and the places in LDS.  Pages are powers of two here, so a key's page is a shift away.
    // An address is  cache + page * (bytes of a page) + (what depends on the thread only) + (what depends on the round
    // only):  one 64-bit multiply-add per vector and round.  Inside a page, key c0 + k lies at ((c0 & (P - 1) & ~63) +
    // (k & (P - 1))): c0 is a multiple of 64 and pages are powers of two, so the two terms never carry into each other.
    int k_local[NV], v_local[NV], k_toff[NV], v_toff[NV], k_lds[NV], v_lds[NV];
    bool v_on[NV];
    const int pmask = P - 1;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = tid + NT * i;
        v_on[i] = v < PF_KEYS * d8;
        const int key = v_on[i] ? v / d8 : 0, ch = v_on[i] ? v % d8 : 0;
        k_local[i] = key;
        k_toff[i] = (key & pmask) * d + ch * 8;
        const int k32 = key & 31;
        // row order inside a 32-key half: tile a reads keys 8j + {0..3}, tile b keys 8j + {4..7}
        const int rho = (key & ~31) + (((k32 & 7) < 4) ? (4 * (k32 >> 3) + (k32 & 3)) : (16 + 4 * (k32 >> 3) + (k32 & 3)));
        k_lds[i] = rho * KLD + ch * 8;
        const int kg = v % (PF_KEYS / 8), dd = v / (PF_KEYS / 8);
        v_local[i] = 8 * kg;
        v_toff[i] = dd * P + ((8 * kg) & pmask);
        v_lds[i] = dd * VLD + 8 * kg;
    }
    const size_t page_elems = (size_t)n_kv * P * d;                 // elements of one page of K (and of V)
    const bf16_t* kc_h = kc + (size_t)hk * P * d;
    const bf16_t* vc_h = vc + (size_t)hk * d * P;
    // The page lookups of a round are issued together and a round early, so that a round costs one
    // memory round trip (the data), not one per vector.
#define PF_PAGES(C0)                                                                                          \
    _Pragma("unroll") for (int i = 0; i < NV; ++i) {                                                          \
        const int key = (C0) + k_local[i], key0 = (C0) + v_local[i];                                          \
        kpg[i] = (v_on[i] && key < kvl) ? bt[key >> log2p] : -1;                                              \
        vpg[i] = (v_on[i] && key0 < kvl) ? bt[key0 >> log2p] : -1;                                            \
    }
#define PF_PREFETCH(C0)                                                                                       \
    {                                                                                                         \
        const int in_page = (C0) & pmask & ~(PF_KEYS - 1);       /* of the round's first key; 0 for pages up to 64 */ \
        const bf16_t* kr = kc_h + (size_t)in_page * d;                                                        \
        const bf16_t* vr = vc_h + in_page;                                                                    \
        _Pragma("unroll") for (int i = 0; i < NV; ++i) {                                                      \
            pk[i] = pf_zero8();                                                                               \
            pv[i] = pf_zero8();                                                                               \
            if ((unsigned)kpg[i] < (unsigned)num_pages)                                                       \
                pk[i] = *reinterpret_cast<const bf16x8_t*>(kr + (size_t)(unsigned)kpg[i] * page_elems + k_toff[i]); \
            if ((unsigned)vpg[i] < (unsigned)num_pages)                                                       \
                pv[i] = *reinterpret_cast<const bf16x8_t*>(vr + (size_t)(unsigned)vpg[i] * page_elems + v_toff[i]); \
        }                                                                                                     \
    }                                                                                                         \
    if ((C0) + PF_KEYS > kvl) {                        /* slots beyond the request's keys hold anything */     \
        _Pragma("unroll") for (int i = 0; i < NV; ++i) {                                                      \
            const int valid = kvl - ((C0) + v_local[i]);                                                      \
            if (valid < 8) { _Pragma("unroll") for (int j = 0; j < 8; ++j) if (j >= valid) pv[i][j] = 0; }     \
        }                                                                                                     \
    }

    const int per_part = (nblk + splits - 1) / splits;
    const int b_first = part * per_part, b_last = min(nblk, b_first + per_part);
    // The query rows are waited for here, once.  Left pending into the loop, they make the compiler wait for every
    // outstanding load (vmcnt(0)) ahead of each round's first product, the round's own prefetch included.
    __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0); the other counters stay as they are
    if (b_first < b_last) {
        PF_PAGES(lo + PF_KEYS * b_first)
        PF_PREFETCH(lo + PF_KEYS * b_first)
        PF_PAGES(lo + PF_KEYS * (b_first + 1))
    }
    for (int b = b_first; b < b_last; ++b) {
        const int c0 = lo + PF_KEYS * b;
        __syncthreads();                               // the previous round's readers are done
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            if (v_on[i]) {
                *reinterpret_cast<bf16x8_t*>(ks + k_lds[i]) = pk[i];
                *reinterpret_cast<bf16x8_t*>(vs + v_lds[i]) = pv[i];
            }
        }
        __syncthreads();
        if (b + 1 < b_last) {
            PF_PREFETCH(c0 + PF_KEYS)
            PF_PAGES(c0 + 2 * PF_KEYS)
        }

#pragma unroll
        for (int half = 0; half < PF_KEYS / 32; ++half) {          // 32 keys at a time
            const int h0 = c0 + 32 * half;
            if (h0 > w_hi || h0 + 31 < w_lo) continue;             // no row of this wave reads these keys (wave-uniform)
            // ---- S^T = K . Q^T for both row tiles ------------------------------------------------
            f32x4_t sa[RT], sb[RT];
#pragma unroll
            for (int t = 0; t < RT; ++t) { sa[t] = f32x4_t{0.f, 0.f, 0.f, 0.f}; sb[t] = f32x4_t{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                if (DFULL || kk * 32 < d) {
                    // columns at and beyond d were never staged: they must read as zero, not as what LDS held before
                    const bool in_d = DFULL || kk * 32 + 8 * g < d;
                    const bf16x8_t ka = in_d ? *reinterpret_cast<const bf16x8_t*>(ks + (32 * half + r16) * KLD + kk * 32 + 8 * g) : pf_zero8();
                    const bf16x8_t kb = in_d ? *reinterpret_cast<const bf16x8_t*>(ks + (32 * half + 16 + r16) * KLD + kk * 32 + 8 * g) : pf_zero8();
#pragma unroll
                    for (int t = 0; t < RT; ++t) {
                        sa[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, bq[t][kk], sa[t], 0, 0, 0);
                        sb[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb, bq[t][kk], sb[t], 0, 0, 0);
                    }
                }
            }
            // ---- softmax: this lane has keys h0 + 8 g .. + 7 of its rows.  Scores are kept times log2(e),
            // so that the exponentials are single v_exp_f32; the result does not change. ---------------------
            // Most key blocks lie wholly before every row of the wave and inside every window: no masks then.
            const bool unmasked = w_rows_full && h0 + 31 <= w_min_pos && h0 >= w_max_lo && h0 + 31 < kvl;
            bf16x8_t pb[RT];
            float alpha[RT];
#pragma unroll
            for (int t = 0; t < RT; ++t) {
                float sc[8];                          // raw scores; the scale goes into the exponent's fma
#pragma unroll
                for (int j = 0; j < 8; ++j) sc[j] = j < 4 ? sa[t][j] : sb[t][j - 4];
                if (!unmasked) {
                    // (the empty statement keeps the masks' index arithmetic inside this branch: the compiler had moved
                    // it ahead of the branch, into the path of every block of keys)
                    int key0 = h0 + 8 * g;
                    asm volatile("" : "+v"(key0));
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int key = key0 + j;
                        const bool ok = row_ok[t] && key <= pos[t] && key >= lo_row[t] && key < kvl;
                        sc[j] = ok ? sc[j] : -INFINITY;
                    }
                }
                const float bmax = scale2 * fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
                // The running maximum m[t] (times log2 e) only has to bound the scores loosely: it is raised,
                // for the whole wave at once, only when some score exceeds it by more than 2^PF_SLACK.  Most
                // rounds then need neither the exchange between the four lanes of a row nor a rescale of O.
                alpha[t] = 1.f;
                if (__any(bmax > m[t] + PF_SLACK)) {
                    float rmax = fmaxf(bmax, __shfl_xor(bmax, 16, 64));
                    rmax = fmaxf(rmax, __shfl_xor(rmax, 32, 64));
                    const float m_new = fmaxf(m[t], rmax);
                    // a row that has seen no key yet keeps m = -inf; its exponent base is 0 then (all its p are 0)
                    alpha[t] = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m[t] - m_new);
                    l[t] *= alpha[t];
                    m[t] = m_new;
                }
                const float nbase = (m[t] == -INFINITY) ? 0.f : -m[t];
                float pj[8];
                float psum = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) { pj[j] = __builtin_amdgcn_exp2f(fmaf(sc[j], scale2, nbase)); psum += pj[j]; }
                typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
                const u32x4_t packed = {pack_bf16x2(pj[0], pj[1]), pack_bf16x2(pj[2], pj[3]), pack_bf16x2(pj[4], pj[5]), pack_bf16x2(pj[6], pj[7])};
                pb[t] = __builtin_bit_cast(bf16x8_t, packed);
                l[t] += psum;
            }
            // ---- O^T = O^T * alpha + V^T . P^T (the rescale is skipped while no row's maximum moves) -------
#pragma unroll
            for (int t = 0; t < RT; ++t) {
                if (__any(alpha[t] != 1.f)) {
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) acc[t][dt] *= alpha[t];
                }
            }
            if (DFULL) {
                // the value fragments are read two products ahead of their use; the scheduling barriers keep the compiler
                // from moving every read down to its product (it did, to save registers: 8 LDS round trips in a row)
                const bf16_t* vrow = vs + r16 * VLD + 32 * half + 8 * g;
                bf16x8_t vt[3];
                vt[0] = *reinterpret_cast<const bf16x8_t*>(vrow);
                vt[1] = *reinterpret_cast<const bf16x8_t*>(vrow + 16 * VLD);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    if (dt + 2 < DT) vt[(dt + 2) % 3] = *reinterpret_cast<const bf16x8_t*>(vrow + (dt + 2) * 16 * VLD);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int t = 0; t < RT; ++t) acc[t][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt[dt % 3], pb[t], acc[t][dt], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    if (dt * 16 < d) {
                        const bf16x8_t vt = *reinterpret_cast<const bf16x8_t*>(vs + (dt * 16 + r16) * VLD + 32 * half + 8 * g);
#pragma unroll
                        for (int t = 0; t < RT; ++t) acc[t][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt, pb[t], acc[t][dt], 0, 0, 0);
                    }
                }
            }
        }
    }
#undef PF_PREFETCH
#undef PF_PAGES
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        float lt = l[t];
        lt += __shfl_xor(lt, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
        if (splits > 1) {
            // this part's share of the 16-row unit: O unnormalised, m back in the natural-log domain, l
            const int unit = tile * (PF_ROWS / 16) + wave * RT + t;
            float* w = ws + (((size_t)unit * n_kv + hk) * splits + part) * (16 * (DMAX + 2));
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4_t*>(w + r16 * DMAX + dt * 16 + 4 * g) = acc[t][dt];
            if (g == 0) {
                w[16 * DMAX + r16] = m[t] * 0.6931471805599453f;
                w[16 * DMAX + 16 + r16] = lt;
            }
            continue;
        }
        if (!row_ok[t]) continue;
        const float inv = lt > 0.f ? 1.0f / lt : 0.f;
        bf16_t* op = out + ((size_t)(q0 + tq[t]) * n_q + head[t]) * d;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int dd = dt * 16 + 4 * g;
            if (dd < d) {
                uint2 w;
                w.x = pack_bf16x2(acc[t][dt][0] * inv, acc[t][dt][1] * inv);
                w.y = pack_bf16x2(acc[t][dt][2] * inv, acc[t][dt][3] * inv);
                // (four columns from a multiple of 4 never cross a group of 8: one store either way)
                if (out_tiles) *reinterpret_cast<uint2*>(out + attention_out_operand_order(q0 + tq[t], head[t] * d + dd, out_tiles)) = w;
                else *reinterpret_cast<uint2*>(op + dd) = w;
            }
        }
    }
    }   // which
}

extern "C" int64_t spy_attention_prefill_workspace(int num_tiles, int tile_rows, int n_kv, int d, int splits) {
    if (splits <= 1) return 0;
    return (int64_t)num_tiles * (tile_rows / 16) * n_kv * splits * 16 * ((d <= 64 ? 64 : 128) + 2);
}

// Tiles of 256 rows against tiles of 128, same measurement: 92 against 73 us at 2048 tokens (128 blocks: half the CUs
// idle), 125 against 133 at 3072, 170 against 195 at 4096, 607 against 675 at 8192, 2331 against 2565 at 16384 (0.94
// PFLOP/s); the caller picks the tile size by the number of blocks.  One tile per block instead of two, so that a grid
// of one block per CU becomes two per CU, was slower at every length (88 against 73 us at 2048 tokens).
// Measured on MI355X (256 CUs), 32 query heads of 128, microseconds per call for 2048 / 2304 / 3072 / 4096 / 8192
// tokens of one prompt (256 / 288 / 384 / 512 / 1024 blocks): 4 waves of two row tiles 85 / 115 / 148 / 193 / 717;
// 8 waves of one row tile with registers for one block per CU 65 / 130 / 165 / 217 / 807, with 128 registers (two
// blocks per CU) 69 / 98 / 129 / 185 / 677.  So: 8 waves always (full head sizes), the registers by the grid.
static long long cu_count() {
    static long long cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus = n;
    }
    return cus;
}

extern "C" int spy_attention_prefill(void* out, const void* q, const void* kc, const void* vc, int P, int num_pages, const int* cu_q,
                                     const int* pos0, const int* kv_len, const int* block_table, int max_blocks,
                                     const int* tile_entry, const int* tile_row0, int num_tiles, int tile_rows, int S, int T, int n_q,
                                     int n_kv, int d, float scale, int window, int splits, float* ws, int out_tiles, hipStream_t st) {
    SPY_REQUIRE(num_tiles > 0 && S > 0 && T > 0 && n_q > 0 && n_kv > 0 && num_pages > 0 && max_blocks > 0,
                "spy_attention_prefill: empty operand");
    SPY_REQUIRE(d % 16 == 0 && d >= 16 && d <= 128, "spy_attention_prefill: head_dim %d is not a multiple of 16 in 16..128", d);
    SPY_REQUIRE(P >= 8 && (P & (P - 1)) == 0, "spy_attention_prefill: page size %d is not a power of two >= 8", P);
    int log2p = 0;
    while ((1 << log2p) < P) ++log2p;
    SPY_REQUIRE(n_q % n_kv == 0, "spy_attention_prefill: n_q %d is not a multiple of n_kv %d", n_q, n_kv);
    SPY_REQUIRE(n_kv <= 65535, "spy_attention_prefill: too many kv heads");
    SPY_REQUIRE(splits >= 1 && splits <= 16, "spy_attention_prefill: %d key parts (1..16 allowed)", splits);
    SPY_REQUIRE(splits == 1 || ws, "spy_attention_prefill: key parts without a workspace");
    SPY_REQUIRE(tile_rows == 128 || (tile_rows == 256 && (d == 64 || d == 128)),
                "spy_attention_prefill: tiles of %d rows (128, or 256 for head sizes 64 and 128)", tile_rows);
    // out_tiles > 0: the output [T, n_q d] goes out in MFMA operand order for that many row tiles (attention_merge.h), for a
    // decode product that reads it next
    SPY_REQUIRE(out_tiles >= 0 && out_tiles <= 8 && (!out_tiles || (T <= 16 * out_tiles && (n_q * d) % 32 == 0 && d % 8 == 0)),
                "spy_attention_prefill: operand order is for at most 128 rows (%d here) of a width that is a multiple of 32", T);
    const dim3 grid(splits > 1 ? num_tiles : (num_tiles + 1) / 2, n_kv, splits);
    const dim3 mgrid(num_tiles * (tile_rows / 16), n_kv);
    const bool one_per_cu = (long long)grid.x * grid.y * grid.z <= cu_count();
#define PF_ARGS (bf16_t*)out, (const bf16_t*)q, (const bf16_t*)kc, (const bf16_t*)vc, P, num_pages, cu_q, pos0, kv_len, block_table,   \
                max_blocks, tile_entry, tile_row0, n_q, n_kv, d, scale, window, log2p, num_tiles, splits, ws, out_tiles
    // (head sizes other than 64 and 128 keep the 4-wave shape: with conditions in the head-dim loops the other needs too many registers)
#define PF_CASE(DM)                                                                                                              \
    if (tile_rows == 256) attention_prefill_kernel<DM, true, 2, 2, 256><<<grid, 512, 0, st>>>(PF_ARGS);                          \
    else if (d == DM) {                                                                                                          \
        if (one_per_cu) attention_prefill_kernel<DM, true, 1, 2, 128><<<grid, 512, 0, st>>>(PF_ARGS);                            \
        else attention_prefill_kernel<DM, true, 1, 4, 128><<<grid, 512, 0, st>>>(PF_ARGS);                                       \
    } else attention_prefill_kernel<DM, false, 2, 2, 128><<<grid, 256, 0, st>>>(PF_ARGS);                                        \
    if (splits > 1)                                                                                                              \
        attention_merge_kernel<DM><<<mgrid, 256, 0, st>>>((bf16_t*)out, ws, cu_q, tile_entry, tile_row0, n_q, n_kv, d, splits,    \
                                                          tile_rows / 16, out_tiles);
    if (d <= 64) { PF_CASE(64) } else { PF_CASE(128) }
#undef PF_CASE
#undef PF_ARGS
    SPY_CHECK_LAUNCH("spy_attention_prefill");
    return 0;
}
