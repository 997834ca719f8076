// Paged attention on MFMA for bfloat16: one block of AW waves per (16-row tile, kv head, part of
// the keys); the waves take the part's 32-key blocks in turn and merge through LDS at the end.
//
// Rows of a tile are (token, query head of the kv head's group) pairs of one batch entry, token
// major: row r -> token r / G, head hk * G + r % G.  So a decoded token fills G rows, a prompt
// portion of n tokens n * G rows, and one kernel serves single tokens, portions and their mix.
//
// Per block of 32 keys, with v_mfma_f32_16x16x32_bf16 (operand lane layout: lane % 16 = row or
// column, lane / 16 = which 8 of the 32 k values):
//   S^T = K . Q^T   two MFMA tiles (a, b).  Tile a takes keys c0 + 8(r/4) + r%4, tile b those + 4,
//                   so that lane (q row, g) ends up with the scores of keys c0 + 8g .. c0 + 8g + 7.
//   softmax         running maximum and sum per q row, float32; the maximum is combined over the
//                   four lanes of a row (g) with two lane exchanges.
//   O^T += V^T . P^T   P^T needs exactly those 8 keys per lane as its 8 k values: no data movement.
//                   V^T comes from the cache, where values lie [d][key] within a page: lane
//                   (d row, g) loads the 8 keys c0 + 8g .. +7 of row d with one 16-byte load.
// Keys lie [key][d] within a page: lane (key, g) loads 16 bytes K[key][32 kk + 8 g ..].
// With several parts per tile the partial (O, m, l) go to a workspace; the tile's last block merges them (given
// counters), or a second kernel does.  The parts of a tile are of one size, set by the grid, or (steps of single tokens)
// cut by the host from the lengths of all of the step's requests, a record per block: long requests in many parts,
// short ones whole, every compute unit about the same number of keys.
//
// FUSED (steps in which every entry is a single token, head_dim 64, 128 or 256, whole head rotated): the kernel reads
// the raw q, k, v of the step's product itself.  A query row's values lie in one lane and the three lanes beside it the
// way the rotation pairs them (dims j and j + d/2 are 32-wide chunks kk and kk + KK/2 of the same lane), so the
// per-head RMS norm costs two lane exchanges and the rotation none.  The entry's new key is prepared the same way
// by every lane for its own 8-value pieces, put in the place of the cache's row in the one block and round that reach
// its position, and stored to the cache from there; so is the new value.  No other block reads that position.
// (The merge by the last block uses no fence: with device-scope fences on both sides, each of which writes back and
// invalidates the whole L2, it took 26 us against 17 us at 8 requests.  What orders it instead is said at the site.)
#include "common.h"
#include "attention_merge.h"
#include <math.h>
#include <type_traits>

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

__device__ __forceinline__ bf16x8_t zero8() { return bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0}; }

#define AW 4   // waves per block

// What the fused variant needs beside the cache: the step's raw [q | k | v] rows, the norm weights, the rotation tables.
struct FusedQKV {
    const bf16_t* qkv;      // [T, (n_q + 2 n_kv) d]
    const void* qw;         // [d] or null (no norm)
    const void* kw;
    int w_dtype;
    float eps;
    const float* cos_t;     // [max_pos, d / 2], null: no rotation
    const float* sin_t;
    int max_pos;
    int store;              // 0: the new key and value are neither stored nor used (the cache of another call is read)
};

// This lane's pieces (dims 32 kk + 8 g + e) of a [d] weight vector.  A bfloat16 vector is asked for early and kept as it
// comes from memory, widened to float only where it is used: widening it at once would wait for it, a memory round trip
// at the kernel's start.  A float32 vector (a checkpoint that stores its norms so) is read where it is used.
template <int KK>
__device__ __forceinline__ void load_weight_pieces(bf16x8_t (&raw)[KK], const void* w, int dtype, int g) {
    if (dtype != SPY_F32) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) raw[kk] = *reinterpret_cast<const bf16x8_t*>(reinterpret_cast<const bf16_t*>(w) + kk * 32 + 8 * g);
    }
}
template <int KK>
__device__ __forceinline__ void widen_weight_pieces(float (&wv)[KK][8], const bf16x8_t (&raw)[KK], const void* w, int dtype, int g) {
    if (dtype == SPY_F32) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(reinterpret_cast<const float*>(w) + kk * 32 + 8 * g);
            const f32x4_t hi = *reinterpret_cast<const f32x4_t*>(reinterpret_cast<const float*>(w) + kk * 32 + 8 * g + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) { wv[kk][e] = lo[e]; wv[kk][e + 4] = hi[e]; }
        }
    } else {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
#pragma unroll
            for (int e = 0; e < 8; ++e) wv[kk][e] = bf16_to_f32((bf16_t)raw[kk][e]);
    }
}

// Raw head row -> normed and rotated, for this lane's pieces.  `x` holds the raw pieces; wv the norm weight's pieces
// (used if normed); cs, sn the cosines and sines of dims 32 kk + 8 g + e, kk < KK / 2 (used if rotated).
template <int KK>
__device__ __forceinline__ void norm_rotate(bf16x8_t (&x)[KK], bool normed, const float (&wv)[KK][8], float eps, bool rotated,
                                            const float (&cs)[KK / 2][8], const float (&sn)[KK / 2][8], int d) {
    float v[KK][8];
    float ss = 0.f;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
#pragma unroll
        for (int e = 0; e < 8; ++e) { v[kk][e] = bf16_to_f32((bf16_t)x[kk][e]); ss += v[kk][e] * v[kk][e]; }
    if (normed) {
        ss += __shfl_xor(ss, 16, 64);
        ss += __shfl_xor(ss, 32, 64);
        const float scale = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
#pragma unroll
            for (int e = 0; e < 8; ++e) v[kk][e] = (scale * v[kk][e]) * wv[kk][e];
    }
    if (rotated) {
        constexpr int HK = KK / 2;
#pragma unroll
        for (int kk = 0; kk < HK; ++kk)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float a = v[kk][e], b = v[kk + HK][e];
                v[kk][e] = a * cs[kk][e] - b * sn[kk][e];
                v[kk + HK][e] = a * sn[kk][e] + b * cs[kk][e];
            }
    }
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        const u32x4_t pk = {pack_bf16x2(v[kk][0], v[kk][1]), pack_bf16x2(v[kk][2], v[kk][3]), pack_bf16x2(v[kk][4], v[kk][5]),
                            pack_bf16x2(v[kk][6], v[kk][7])};
        x[kk] = __builtin_bit_cast(bf16x8_t, pk);
    }
}

// FULL (not 0): head_dim == DMAX.  The loads of keys and values then have no conditions (a page that does not exist is read as
// page 0 and what was read is masked: scores by position, values by the count of keys that exist and, under a window, by
// the page's absence), so the compiler knows how many loads are in flight and a wait is for the oldest only.
// FULL_STREAMED / FULL_KEPT: whether the values are read with the hint that they will not be read again (pages of up to 32
// keys) or without it (larger pages).
constexpr int FULL_STREAMED = 1, FULL_KEPT = 2;
template <int DMAX, bool FUSED, int FULL>
__global__ __launch_bounds__(AW * 64, (FUSED && DMAX <= 128) ? 2 : 1) void attention_mfma_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, bf16_t* kc, bf16_t* vc,
    int P, int num_pages, const int* __restrict__ cu_q, const int* __restrict__ pos0, const int* __restrict__ kv_len,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ tile_entry, const int* __restrict__ tile_row0,
    int n_q, int n_kv, int d, float scale, int window, int splits, float* __restrict__ ws, FusedQKV fz, int out_tiles,
    unsigned* counters, int log2p, const int* __restrict__ pieces) {
    constexpr int KK = DMAX / 32;   // 32-wide chunks of the head dim for Q.K
    constexpr int DT = DMAX / 16;   // 16-row tiles of the head dim for P.V
    extern __shared__ float lds[];   // the waves' O, m, l: AW (head sizes up to 128) or AW - 1 times (DT * 4 + 2) * 64 floats
    // Which (tile, kv head, part of the keys) this block has: its place in the grid, or (FUSED, `pieces` given) a record
    // of 8 ints that the host made for this block: { entry, kv head, first and end block of 32 keys, number of this
    // part, parts of the (entry, kv head), first workspace slot of its parts, the entry's keys }.  The host cuts every
    // entry's keys by what the whole step has to read, so that blocks have even shares whatever the entries' lengths
    // are; a record with entry -1 is a block without work.
    int tile = blockIdx.x, hk = blockIdx.y, sp = blockIdx.z;
    int pc_begin = 0, pc_end = 0, pc_slot = 0, pc_kvl = 0;
    const bool cut_by_host = FUSED && pieces != nullptr;
    if (cut_by_host) {
        const int4 r0 = *reinterpret_cast<const int4*>(pieces + (size_t)blockIdx.x * 8);
        const int4 r1 = *reinterpret_cast<const int4*>(pieces + (size_t)blockIdx.x * 8 + 4);
        if (r0.x < 0) return;
        tile = r0.x, hk = r0.y, pc_begin = r0.z, pc_end = r0.w;
        sp = r1.x, splits = r1.y, pc_slot = r1.z, pc_kvl = r1.w;
    }
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // uniform: loops over it stay scalar
    // a key's page and its place inside: a shift and a mask for pages that are a power of two (log2p >= 0), instead of
    // a division of two dozen instructions per lane, four of them per block of keys
    auto page_of = [&](int key) { return log2p >= 0 ? key >> log2p : key / P; };
    auto in_page = [&](int key) { return log2p >= 0 ? key & (P - 1) : key % P; };
    const int lane = threadIdx.x & 63, r16 = lane & 15, g = lane >> 4;
    // FUSED: every entry is one token and has one tile (the host has checked it), so tile t is entry t with query token t:
    // two dependent loads less before the first key can be asked for
    const int s = FUSED ? tile : tile_entry[tile];
    const int row0 = FUSED ? 0 : tile_row0[tile];
    const int G = n_q / n_kv;
    const int q0 = FUSED ? s : cu_q[s];
    const int n = FUSED ? 1 : cu_q[s + 1] - q0;
    const int nrows = n * G;
    // (the host's record brings the entry's length along: one round trip less before the pages can be asked for)
    const int p0 = cut_by_host ? pc_kvl - 1 : pos0[s];
    const int kvl = cut_by_host ? pc_kvl : kv_len[s];
    const int* bt = block_table + (size_t)s * max_blocks;

    // this lane's query row (as column of S^T and O^T)
    const int row = row0 + r16;
    const bool row_ok = row < nrows;
    const int tq = row_ok ? row / G : 0;
    const int head = hk * G + (row_ok ? row % G : 0);
    const int pos = p0 + tq;
    const int lo_row = window > 0 ? max(0, pos - window + 1) : 0;

    bf16x8_t bq[KK];
    {
        const bf16_t* qp = FUSED ? fz.qkv + ((size_t)(q0 + tq) * (n_q + 2 * n_kv) + head) * d : q + ((size_t)(q0 + tq) * n_q + head) * d;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const int dofs = kk * 32 + 8 * g;
            bq[kk] = (row_ok && dofs < d) ? *reinterpret_cast<const bf16x8_t*>(qp + dofs) : zero8();
        }
    }
    // keys this tile can see: from the first row's window start to the last row's position
    const int last_row = min(nrows, row0 + 16) - 1;
    const int hi = min(p0 + last_row / G, kvl - 1);
    int lo = window > 0 ? max(0, p0 + row0 / G - window + 1) : 0;
    lo &= ~31;
    const int nblk = hi >= lo ? (hi - lo) / 32 + 1 : 0;
    const int per = (nblk + splits - 1) / splits;
    const int b_begin = cut_by_host ? pc_begin : sp * per, b_end = min(nblk, cut_by_host ? pc_end : b_begin + per);

    f32x4_t acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    // FUSED: the entry's one new token lies at position p0 = kvl - 1; its query rows have that position too.  The block
    // whose keys reach it prepares the new key (every lane its pieces for its g, as for q) and takes the new value's
    // elements of its rows dd.
    // The kernel's start is a chain of memory round trips (about a microsecond each when the step's weights have swept
    // the caches), so loads are issued in the order of what they depend on, each group together and ahead of any wait:
    // what depends on the block alone (raw k and v, the norm weights; the raw query row is on its way already), then
    // what needs the entry's position (rotation table, pages), then the first keys (they need the pages); the norm and
    // the rotation are worked out while the keys are on their way.
    const int newpos = p0;
    bool has_new = false;
    bf16x8_t knew[KK];
    bf16_t vnew[DT];
    int new_page = -1;
    constexpr int HKF = FUSED ? KK / 2 : 1;
    float cs[HKF][8], sn[HKF][8];
    bf16x8_t wq_raw[FUSED ? KK : 1], wk_raw[FUSED ? KK : 1];
    const bool normed = FUSED && fz.qw != nullptr, rotated = FUSED && fz.cos_t != nullptr;
    if constexpr (FUSED) {
        if (fz.store) {
            const bf16_t* base = fz.qkv + (size_t)q0 * (n_q + 2 * n_kv) * d;
            const bf16_t* kp_raw = base + (size_t)(n_q + hk) * d;
            const bf16_t* vp_raw = base + (size_t)(n_q + n_kv + hk) * d;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) knew[kk] = *reinterpret_cast<const bf16x8_t*>(kp_raw + kk * 32 + 8 * g);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) vnew[dt] = vp_raw[dt * 16 + r16];
            if (normed) load_weight_pieces<KK>(wk_raw, fz.kw, fz.w_dtype, g);
        }
        if (normed) load_weight_pieces<KK>(wq_raw, fz.qw, fz.w_dtype, g);
        __builtin_amdgcn_sched_barrier(0);
        has_new = fz.store && n == 1 && newpos >= lo + 32 * b_begin && newpos < lo + 32 * b_end;
    }
    // A wave's loop is a chain of memory round trips, so they are overlapped: pages are looked up two blocks ahead (both
    // lookups together); the keys of the next block are asked for as soon as this block's S^T products have read the
    // key registers, and arrive while the softmax and the second product run; the values are asked for at the top of
    // their block and arrive behind the first product.
    int kpage = -1, vpage = -1, kpage_n = -1, vpage_n = -1;
#define AM_LOOKUP(B, KP, VP)                                                                                  \
    {                                                                                                         \
        KP = -1;                                                                                              \
        VP = -1;                                                                                              \
        if ((B) < b_end) {                                                                                    \
            const int c0_ = lo + 32 * (B);                                                                    \
            const int ka_ = c0_ + 8 * (r16 >> 2) + (r16 & 3), kv_ = c0_ + 8 * g;                              \
            if (ka_ < kvl) KP = bt[page_of(ka_)];                                                                \
            if (kv_ < kvl) VP = bt[page_of(kv_)];                                                                \
        }                                                                                                     \
    }
    bf16x8_t ka[KK], kb[KK];
    // tile a of block B has this lane's key lo + 32 B + 8 (r16 / 4) + r16 % 4; tile b is 4 keys on (same page: P % 8 == 0)
#define AM_LOAD_K(B, KP)                                                                                      \
    {                                                                                                         \
        const int key_ = lo + 32 * (B) + 8 * (r16 >> 2) + (r16 & 3);                                          \
        const bool ok_ = (KP) >= 0 && (KP) < num_pages;                                                       \
        const bf16_t* kp_ = kc + (((size_t)(ok_ ? (KP) : 0) * n_kv + hk) * P + in_page(key_)) * d;            \
        _Pragma("unroll") for (int kk = 0; kk < KK; ++kk) {                                                   \
            const int dofs = kk * 32 + 8 * g;                                                                 \
            if (FULL) {                                                                                       \
                ka[kk] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(kp_ + dofs));                                      \
                kb[kk] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(kp_ + 4 * d + dofs));                              \
            } else {                                                                                          \
                ka[kk] = zero8();                                                                             \
                kb[kk] = zero8();                                                                             \
                if (ok_ && dofs < d) {                                                                        \
                    ka[kk] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(kp_ + dofs));                                  \
                    if (key_ + 4 < kvl) kb[kk] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(kp_ + 4 * d + dofs));      \
                }                                                                                             \
            }                                                                                                 \
        }                                                                                                     \
    }
    AM_LOOKUP(b_begin + wave, kpage, vpage)
    AM_LOOKUP(b_begin + wave + AW, kpage_n, vpage_n)
    if constexpr (FUSED) {
        if (has_new) new_page = bt[page_of(newpos)];
        if (rotated) {
            const size_t trow = (size_t)min(newpos, fz.max_pos - 1) * (d / 2);
#pragma unroll
            for (int kk = 0; kk < HKF; ++kk) {
                const f32x4_t c0 = *reinterpret_cast<const f32x4_t*>(fz.cos_t + trow + kk * 32 + 8 * g);
                const f32x4_t c1 = *reinterpret_cast<const f32x4_t*>(fz.cos_t + trow + kk * 32 + 8 * g + 4);
                const f32x4_t s0 = *reinterpret_cast<const f32x4_t*>(fz.sin_t + trow + kk * 32 + 8 * g);
                const f32x4_t s1 = *reinterpret_cast<const f32x4_t*>(fz.sin_t + trow + kk * 32 + 8 * g + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) { cs[kk][e] = c0[e]; cs[kk][e + 4] = c1[e]; sn[kk][e] = s0[e]; sn[kk][e + 4] = s1[e]; }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    if (b_begin + wave < b_end) AM_LOAD_K(b_begin + wave, kpage)
    if constexpr (FUSED) {
        __builtin_amdgcn_sched_barrier(0);
        float wv[KK][8];
        if (normed) widen_weight_pieces<KK>(wv, wq_raw, fz.qw, fz.w_dtype, g);
        norm_rotate<KK>(bq, normed, wv, fz.eps, rotated, cs, sn, d);
        if (has_new) {
            if (normed) widen_weight_pieces<KK>(wv, wk_raw, fz.kw, fz.w_dtype, g);
            norm_rotate<KK>(knew, normed, wv, fz.eps, rotated, cs, sn, d);
            if (new_page < 0 || new_page >= num_pages) has_new = false;   // no page: nothing to store or to use
        }
    }
    // One block of 32 keys.  LAST: the wave's last block, which alone can hold keys beyond the request's and the step's
    // new key, and after which no keys are asked for; the blocks before it have no condition around their loads.
    auto block = [&](const int b, auto last_block) {
        constexpr bool LAST = decltype(last_block)::value;
        const int c0 = lo + 32 * b;
        const int key_a = c0 + 8 * (r16 >> 2) + (r16 & 3);      // tile a; tile b is key_a + 4
        const int key_v = c0 + 8 * g;                             // this lane's 8 keys of V
        const bool v_ok = vpage >= 0 && vpage < num_pages;
        const bf16_t* vp = vc + (((size_t)(v_ok ? vpage : 0) * n_kv + hk) * d) * P + in_page(key_v);
        bf16x8_t vt[DT];
        if constexpr (FULL == FULL_STREAMED) {
            // (a block's 32 keys of a dim are whole lines of pages of up to 32 keys: read once, not to be kept)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) vt[dt] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(vp + (size_t)(dt * 16 + r16) * P));
        } else if constexpr (FULL == FULL_KEPT) {
            // (of larger pages they are half a line or less, and the next block, which another wave of this block takes
            // at about the same time, reads the rest of it: kept, or memory would bring every line twice.  64 requests
            // of 8337 keys in pages of 64: 397 against 460 us; pages of 16: 357.  A template's value and not a branch:
            // the compiler makes one load of the two arms of a branch, without the hint)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) vt[dt] = *reinterpret_cast<const bf16x8_t*>(vp + (size_t)(dt * 16 + r16) * P);
        } else {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int dd = dt * 16 + r16;
                vt[dt] = (v_ok && dd < d) ? *reinterpret_cast<const bf16x8_t*>(vp + (size_t)dd * P) : zero8();
            }
        }
        if (FULL && window > 0 && !v_ok) {
            // The window's first block of 32 keys may begin in a page that the window has passed and the request has
            // given back: its keys are masked by their positions, but what page 0 holds in their values' place would
            // still be multiplied (by a weight of zero: harmless for numbers, not for a NaN or an infinity).
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) vt[dt] = zero8();
        }
        int kpage_nn, vpage_nn;
        AM_LOOKUP(b + 2 * AW, kpage_nn, vpage_nn)
        if (FUSED && LAST && has_new && newpos >= c0 && newpos < c0 + 32) {
            // the new key: the four lanes of its row take the prepared pieces; the lanes with r16 % 16 == its row store it
            const bool mine_a = key_a == newpos, mine_b = key_a + 4 == newpos;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                if (mine_a) ka[kk] = knew[kk];
                if (mine_b) kb[kk] = knew[kk];
            }
            if (mine_a || mine_b) {
                bf16_t* dst = kc + (((size_t)new_page * n_kv + hk) * P + in_page(newpos)) * d + 8 * g;
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) *reinterpret_cast<bf16x8_t*>(dst + kk * 32) = knew[kk];
            }
            // the new value: element newpos - key_v of the lanes whose 8 keys hold it
            const int jn = newpos - key_v;
            if (jn >= 0 && jn < 8) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (j == jn) vt[dt][j] = (short)vnew[dt];
                    vc[(((size_t)new_page * n_kv + hk) * d + dt * 16 + r16) * P + in_page(newpos)] = vnew[dt];
                }
            }
        }
        const int v_valid = min(8, kvl - key_v);                  // keys of the group that exist (slots beyond hold anything)
        // ---- S^T = K . Q^T ------------------------------------------------------------------
        f32x4_t sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            if (FULL || kk * 32 < d) {
                sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[kk], bq[kk], sa, 0, 0, 0);
                sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb[kk], bq[kk], sb, 0, 0, 0);
            }
        }
        // the key registers are free: the next block's keys
        if (!LAST) AM_LOAD_K(b + AW, kpage_n)
        kpage = kpage_n;
        vpage = vpage_n;
        kpage_n = kpage_nn;
        vpage_n = vpage_nn;
        if ((LAST || !FULL) && (FULL || v_ok) && v_valid < 8) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (j >= v_valid) vt[dt][j] = 0;
        }
        // ---- softmax over this lane's 8 keys of its q row --------------------------------------
        float sc[8];
        float bmax = -INFINITY;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int key = c0 + 8 * g + j;
            const float v = (j < 4 ? sa[j] : sb[j - 4]) * scale;
            const bool ok = row_ok && key <= pos && key >= lo_row && key < kvl;
            sc[j] = ok ? v : -INFINITY;
            bmax = fmaxf(bmax, sc[j]);
        }
        bmax = fmaxf(bmax, __shfl_xor(bmax, 16, 64));
        bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
        const float m_new = fmaxf(m, bmax);
        float alpha = 1.f;
        bf16x8_t pb = zero8();
        if (m_new != -INFINITY) {
            alpha = (m == -INFINITY) ? 0.f : __expf(m - m_new);
            float psum = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float pj = (sc[j] == -INFINITY) ? 0.f : __expf(sc[j] - m_new);
                psum += pj;
                pb[j] = (short)f32_to_bf16(pj);
            }
            l = l * alpha + psum;
            m = m_new;
        }
        // ---- O^T = O^T * alpha + V^T . P^T -----------------------------------------------------
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            if (FULL || dt * 16 < d) {
                acc[dt] *= alpha;
                acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt[dt], pb, acc[dt], 0, 0, 0);
            }
        }
    };
    {
        int b = b_begin + wave;
        for (; b + AW < b_end; b += AW) block(b, std::false_type{});
        if (b < b_end) block(b, std::true_type{});
    }
#undef AM_LOOKUP
#undef AM_LOAD_K
    // the four lanes of a row hold partial sums of l
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);

    // Merge the waves of the block.  Every wave puts its (O, m, l) into LDS, lane for lane (O as vectors of four), and
    // then merges and writes out its share of the head dim's tiles: DT / AW tiles of every wave's O.  (For head sizes
    // beyond 128 the four waves' sums do not fit the LDS that a block may ask for: there wave 0 merges them all.)
    constexpr int PER = DT * 4 + 2;
    constexpr bool SPREAD = DMAX <= 128;
    constexpr int MINE = SPREAD ? DT / AW : DT;       // tiles of the head dim that this wave merges
    static_assert(!SPREAD || DT % AW == 0, "the head dim's tiles are dealt evenly to the waves");
    const int dt0 = SPREAD ? wave * MINE : 0;
    f32x4_t mo[MINE];
    if (SPREAD) {
        float* mine = lds + (size_t)wave * PER * 64;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4_t*>(mine + (dt * 64 + lane) * 4) = acc[dt];
        mine[(DT * 4) * 64 + lane] = m;
        mine[(DT * 4 + 1) * 64 + lane] = l;
        __syncthreads();
        float mw[AW], lw[AW];
        float mn = -INFINITY;
#pragma unroll
        for (int w = 0; w < AW; ++w) {
            mw[w] = lds[((size_t)w * PER + DT * 4) * 64 + lane];
            lw[w] = lds[((size_t)w * PER + DT * 4 + 1) * 64 + lane];
            mn = fmaxf(mn, mw[w]);
        }
        l = 0.f;
#pragma unroll
        for (int i = 0; i < MINE; ++i) mo[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < AW; ++w) {                 // in the order of the waves, whichever wave adds
            const float a = (mw[w] == -INFINITY) ? 0.f : __expf(mw[w] - mn);
            l += lw[w] * a;
#pragma unroll
            for (int i = 0; i < MINE; ++i) {
                const f32x4_t o = *reinterpret_cast<const f32x4_t*>(lds + (((size_t)w * PER * 64) + ((dt0 + i) * 64 + lane) * 4));
                mo[i] += o * a;
            }
        }
        m = mn;
    } else {
        if (wave > 0) {
            float* mine = lds + (size_t)(wave - 1) * PER * 64;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) mine[(dt * 4 + i) * 64 + lane] = acc[dt][i];
            mine[(DT * 4) * 64 + lane] = m;
            mine[(DT * 4 + 1) * 64 + lane] = l;
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 1; w < AW; ++w) {
            const float* other = lds + (size_t)(w - 1) * PER * 64;
            const float mo_ = other[(DT * 4) * 64 + lane];
            const float lo_ = other[(DT * 4 + 1) * 64 + lane];
            const float mn = fmaxf(m, mo_);
            if (mn == -INFINITY) continue;
            const float a = (m == -INFINITY) ? 0.f : __expf(m - mn);
            const float bsc = (mo_ == -INFINITY) ? 0.f : __expf(mo_ - mn);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[dt][i] = acc[dt][i] * a + other[(dt * 4 + i) * 64 + lane] * bsc;
            l = l * a + lo_ * bsc;
            m = mn;
        }
#pragma unroll
        for (int i = 0; i < MINE; ++i) mo[i] = acc[i];
    }

    if (splits == 1) {
        if (!row_ok) return;
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        bf16_t* op = out + ((size_t)(q0 + tq) * n_q + head) * d;
#pragma unroll
        for (int i = 0; i < MINE; ++i) {
            const int dd = (dt0 + i) * 16 + 4 * g;
            if (dd < d) {
                uint2 w;
                w.x = pack_bf16x2(mo[i][0] * inv, mo[i][1] * inv);
                w.y = pack_bf16x2(mo[i][2] * inv, mo[i][3] * inv);
                // (four columns from a multiple of 4 never cross a group of 8: one store either way)
                if (out_tiles) *reinterpret_cast<uint2*>(out + attention_out_operand_order(q0 + tq, head * d + dd, out_tiles)) = w;
                else *reinterpret_cast<uint2*>(op + dd) = w;
            }
        }
        return;
    }
    // the first of this (tile, kv head)'s parts in the workspace: where the grid puts it, or where the host's record says
    const size_t slot0 = cut_by_host ? (size_t)pc_slot : ((size_t)tile * n_kv + hk) * splits;
    float* w = ws + (slot0 + sp) * (16 * (DMAX + 2));
    if (SPREAD && counters) {
        // The parts of a (tile, kv head) are merged here, by the block that finishes last (a counter per tile and head,
        // left at zero), instead of by a second kernel.  The dies' L2s are not coherent inside a kernel: the parts go
        // through the caches (stores of system scope, waited for before the block counts itself) and are read past them.
        // ORDER.  No release/acquire pair states that the parts are visible before the count: the HIP memory model would
        // ask for a release on the counter's increment and an acquire behind it, which this compiler turns into a
        // write-back and an invalidation of the whole L2 (the 9 us above).  What stands in for them is how gfx950 executes
        // these instructions: (1) an atomic store of system scope is a write-through store (sc0 sc1) that has reached
        // memory, past every L2, when the wave's vmcnt has counted it, and s_waitcnt(0) waits for that; (2) the barrier
        // behind it puts every wave's wait before thread 0's increment, and the increment is an atomic of device scope,
        // which all dies execute at one place beyond their L2s (it could not count across dies otherwise), so no block
        // sees the count before the stores it follows have arrived; (3) the last block's loads of
        // system scope miss L1 and L2 (sc0 sc1) and so read what memory holds, and they are issued after the barrier
        // that follows the increment's return.  Do not weaken any of the three (ordinary stores, no wait, ordinary
        // loads), and do not "strengthen" the atomics to release/acquire without measuring: it is correct and slow.
        // A part lies lane for lane: O[(dt 4 + i)][64 lanes], then m[16], l[16].
        __shared__ unsigned am_last;
#pragma unroll
        for (int i = 0; i < MINE; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) __hip_atomic_store(w + ((dt0 + i) * 4 + j) * 64 + lane, mo[i][j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        if (g == 0 && wave == 0) {
            __hip_atomic_store(w + 16 * DMAX + r16, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            __hip_atomic_store(w + 16 * DMAX + 16 + r16, l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned* c = counters + (size_t)tile * n_kv + hk;
            const unsigned before = __hip_atomic_fetch_add(c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            am_last = before == (unsigned)splits - 1u;
            if (before == (unsigned)splits - 1u) __hip_atomic_store(c, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (!am_last) return;
        // All that is read of the parts is asked for before any of it is used, eight parts at a time: one memory round
        // trip for up to eight parts (a loop that adds as it loads has one per part; sixteen at a time cost the step of
        // 8 requests, which has four parts, 1.2 us for the code's length).
        constexpr int MAXS = 32, BATCH = 8;                // (the caller keeps to 32 parts: 16 from the grid, 32 in the host's records)
        constexpr int PART = 16 * (DMAX + 2);
        const float* base = ws + slot0 * PART;
        float pm[MAXS], pl[MAXS];
#pragma unroll
        for (int i = 0; i < MAXS; ++i) {
            pm[i] = -INFINITY;
            pl[i] = 0.f;
            if (i < splits) {
                pm[i] = __hip_atomic_load(base + (size_t)i * PART + 16 * DMAX + r16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                pl[i] = __hip_atomic_load(base + (size_t)i * PART + 16 * DMAX + 16 + r16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
        }
        f32x4_t o[MINE];
#pragma unroll
        for (int i = 0; i < MINE; ++i) o[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        float mn = -INFINITY, L = 0.f;
#pragma unroll
        for (int i0 = 0; i0 < MAXS; i0 += BATCH) {
            if (i0 >= splits) break;
            float ov[BATCH][MINE][4];
#pragma unroll
            for (int i = 0; i < BATCH; ++i)
#pragma unroll
                for (int k = 0; k < MINE; ++k)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        ov[i][k][j] = i0 + i < splits ? __hip_atomic_load(base + (size_t)(i0 + i) * PART + ((dt0 + k) * 4 + j) * 64 + lane,
                                                                          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) : 0.f;
            if (i0 == 0) {
#pragma unroll
                for (int i = 0; i < MAXS; ++i) mn = fmaxf(mn, pm[i]);
            }
#pragma unroll
            for (int i = 0; i < BATCH; ++i) {              // in the order of the parts
                const float a = (pm[i0 + i] == -INFINITY) ? 0.f : __expf(pm[i0 + i] - mn);
                L += pl[i0 + i] * a;
#pragma unroll
                for (int k = 0; k < MINE; ++k)
#pragma unroll
                    for (int j = 0; j < 4; ++j) o[k][j] += a * ov[i][k][j];
            }
        }
        if (!row_ok) return;
        const float inv = L > 0.f ? 1.0f / L : 0.f;
        bf16_t* op = out + ((size_t)(q0 + tq) * n_q + head) * d;
#pragma unroll
        for (int i = 0; i < MINE; ++i) {
            const int dd = (dt0 + i) * 16 + 4 * g;
            if (dd < d) {
                uint2 w2;
                w2.x = pack_bf16x2(o[i][0] * inv, o[i][1] * inv);
                w2.y = pack_bf16x2(o[i][2] * inv, o[i][3] * inv);
                if (out_tiles) *reinterpret_cast<uint2*>(out + attention_out_operand_order(q0 + tq, head * d + dd, out_tiles)) = w2;
                else *reinterpret_cast<uint2*>(op + dd) = w2;
            }
        }
        return;
    }
    // partial result for the merge kernel: ws[((tile * n_kv + hk) * splits + sp)] = { O[16][DMAX], m[16], l[16] }
#pragma unroll
    for (int i = 0; i < MINE; ++i) {
        const int dd = (dt0 + i) * 16 + 4 * g;
        *reinterpret_cast<f32x4_t*>(w + r16 * DMAX + dd) = mo[i];
    }
    if (g == 0 && wave == 0) {
        w[16 * DMAX + r16] = m;
        w[16 * DMAX + 16 + r16] = l;
    }
}

static int dmax_of(int d) { return d <= 64 ? 64 : (d <= 128 ? 128 : 256); }

// Floats of one part's sums in the workspace (keys cut by the host: one part per record).
extern "C" int64_t spy_attention_mfma_part_workspace(int d) { return 16 * (dmax_of(d) + 2); }

extern "C" int64_t spy_attention_mfma_workspace(int num_tiles, int n_kv, int d, int splits) {
    if (splits <= 1) return 0;
    return (int64_t)num_tiles * n_kv * splits * 16 * (dmax_of(d) + 2);
}

// out_tiles > 0: the output [T, n_q d] goes out in MFMA operand order for that many row tiles (attention_merge.h), for a
// decode product that reads it next.
// qkv != null: the fused variant (see the top of the file).  Then q is not read, every entry must be a single token
// (T == S), head_dim 64, 128 or 256 with the whole head rotated (or no rotation: cos_t == null), and the new keys and
// values are written to kc and vc by this call (store != 0).
extern "C" int spy_attention_mfma(void* out, const void* q, void* kc, void* vc, int P, int num_pages, const int* cu_q,
                                  const int* pos0, const int* kv_len, const int* block_table, int max_blocks, const int* tile_entry,
                                  const int* tile_row0, int num_tiles, int S, int T, int n_q, int n_kv, int d, float scale,
                                  int window, int splits, float* ws, const void* qkv, const void* qw, const void* kw, int w_dtype,
                                  float eps, const float* cos_t, const float* sin_t, int max_pos, int store, int out_tiles,
                                  unsigned* counters, int n_counters, const int* pieces, int num_pieces, hipStream_t st) {
    SPY_REQUIRE(num_tiles > 0 && S > 0 && T > 0 && n_q > 0 && n_kv > 0 && num_pages > 0 && max_blocks > 0,
                "spy_attention_mfma: empty operand");
    SPY_REQUIRE(d % 16 == 0 && d >= 16 && d <= 256, "spy_attention_mfma: head_dim %d is not a multiple of 16 in 16..256", d);
    SPY_REQUIRE(P % 8 == 0, "spy_attention_mfma: page size %d is not a multiple of 8", P);
    SPY_REQUIRE(n_q % n_kv == 0, "spy_attention_mfma: n_q %d is not a multiple of n_kv %d", n_q, n_kv);
    SPY_REQUIRE(splits >= 1 && splits <= 64, "spy_attention_mfma: %d parts (1..64 allowed)", splits);
    SPY_REQUIRE(splits == 1 || ws, "spy_attention_mfma: parts without a workspace");
    SPY_REQUIRE(n_kv <= 65535, "spy_attention_mfma: too many kv heads");
    SPY_REQUIRE(out_tiles >= 0 && out_tiles <= 8 && (!out_tiles || (T <= 16 * out_tiles && (n_q * d) % 32 == 0 && d % 8 == 0)),
                "spy_attention_mfma: operand order is for at most 128 rows (%d here) of a width that is a multiple of 32", T);
    FusedQKV fz = {(const bf16_t*)qkv, qw, kw, w_dtype, eps, cos_t, sin_t, max_pos, store};
    if (qkv) {
        SPY_REQUIRE(T == S && num_tiles == S, "spy_attention_mfma: the fused variant takes single tokens only (%d tokens of %d entries)", T, S);
        SPY_REQUIRE(d == 64 || d == 128 || d == 256, "spy_attention_mfma: the fused variant takes head_dim 64, 128 or 256, not %d", d);
        SPY_REQUIRE((!cos_t) == (!sin_t) && (!cos_t || max_pos > 0), "spy_attention_mfma: rotation tables are incomplete");
        SPY_REQUIRE((!qw) == (!kw) && (!qw || w_dtype == SPY_F32 || w_dtype == SPY_BF16), "spy_attention_mfma: norm weights are incomplete");
        SPY_REQUIRE(n_q / n_kv <= 16, "spy_attention_mfma: the fused variant takes groups of at most 16 heads");
        SPY_REQUIRE(((uintptr_t)qkv % 16) == 0, "spy_attention_mfma: qkv must be 16-byte aligned");
    } else {
        SPY_REQUIRE(q, "spy_attention_mfma: no queries");
    }
    if (pieces) {
        // the keys cut by the host (see the kernel's top): one block per record, parts merged by their last block only
        SPY_REQUIRE(qkv && num_pieces > 0, "spy_attention_mfma: keys cut by the host are for the fused variant");
        SPY_REQUIRE(d <= 128 && counters && ws && (long long)num_tiles * n_kv <= n_counters && ((uintptr_t)pieces % 16) == 0,
                    "spy_attention_mfma: keys cut by the host need head_dim <= 128, a workspace and a counter per (entry, kv head) (%d x %d, %d counters)",
                    num_tiles, n_kv, n_counters);
    }
    int log2p = -1;                                        // pages of a power of two: shifts instead of divisions
    if ((P & (P - 1)) == 0) { log2p = 0; while ((1 << log2p) < P) ++log2p; }
    const dim3 grid = pieces ? dim3(num_pieces, 1, 1) : dim3(num_tiles, n_kv, splits);
    const dim3 mgrid(num_tiles, n_kv);
    // The parts merged by each (tile, kv head)'s last block instead of a second kernel: with counters (zeroed once by the
    // caller, one per tile and head, left at zero by every call; calls that overlap on one device race on them), up to
    // 16 parts (the grid's; the host's records may name up to 32 of an entry) and head sizes up to 128.
    unsigned* const cnt = (pieces || (counters && splits > 1 && splits <= 16 && d <= 128 && (long long)num_tiles * n_kv <= n_counters)) ? counters : nullptr;
#define ATT_LAUNCH(DM, FZ, FL)                                                                                                \
    attention_mfma_kernel<DM, FZ, FL><<<grid, AW * 64, (DM <= 128 ? AW : AW - 1) * ((DM / 16) * 4 + 2) * 64 * sizeof(float), st>>>(  \
        (bf16_t*)out, (const bf16_t*)q, (bf16_t*)kc, (bf16_t*)vc, P, num_pages, cu_q, pos0, kv_len, block_table, max_blocks,  \
        tile_entry, tile_row0, n_q, n_kv, d, scale, window, splits, ws, fz, out_tiles, cnt, log2p, pieces)
#define ATT_CASE(DM)                                                                                                          \
    if (qkv && P <= 32) ATT_LAUNCH(DM, true, FULL_STREAMED); else if (qkv) ATT_LAUNCH(DM, true, FULL_KEPT);                      \
    else if (d == DM && P <= 32) ATT_LAUNCH(DM, false, FULL_STREAMED); else if (d == DM) ATT_LAUNCH(DM, false, FULL_KEPT);       \
    else ATT_LAUNCH(DM, false, 0);                                                                                            \
    if (cnt) {}                                                                                                               \
    else if (splits > 1 && qkv)                                                                                               \
        attention_merge_kernel<DM, true><<<mgrid, 256, 0, st>>>((bf16_t*)out, ws, cu_q, tile_entry, tile_row0, n_q, n_kv, d, splits, 1, out_tiles); \
    else if (splits > 1)                                                                                                      \
        attention_merge_kernel<DM><<<mgrid, 256, 0, st>>>((bf16_t*)out, ws, cu_q, tile_entry, tile_row0, n_q, n_kv, d, splits, 1, out_tiles);
    switch (dmax_of(d)) {
        case 64: ATT_CASE(64) break;
        case 128: ATT_CASE(128) break;
        default: ATT_CASE(256) break;
    }
#undef ATT_CASE
#undef ATT_LAUNCH
    SPY_CHECK_LAUNCH("spy_attention_mfma");
    return 0;
}
