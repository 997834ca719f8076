// C[M, N] = X[M, K] . W[N, K]^T for few rows (M <= 64), bfloat16 operands, float32 sums:
// the decode-time product, bound by streaming W from HBM once.
//
// MFMA v_mfma_f32_16x16x32_bf16 with W as the first operand: a wave owns 16 (or 32) rows of W and
// walks K; lane (r = lane % 16, g = lane / 16) loads 16 bytes W[n0 + r][k + 8 g ..] straight from
// global memory into its operand registers, so W is read exactly once and never staged.  X is
// small and comes from the caches, X[m0 + r][k + 8 g ..] per 16-row tile of M.  The product tile
// is C^T: lane (m = lane % 16, g) holds C[m][n0 + 4 g + i], i < 4.
// The waves of a block split K in interleaved chunks of 128 and add their tiles through LDS in a
// fixed order, so results are reproducible.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define SK_CHUNK 128   // k per wave iteration = 4 MFMA steps of 32

__device__ __forceinline__ bf16x8_t load8(const bf16_t* p, bool ok) {
    bf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (ok) v = *reinterpret_cast<const bf16x8_t*>(p);
    return v;
}

// GATED (with NT = 2): W holds [gate rows | up rows], N is the number of gate rows; tile 0 of a block is
// 16 gate rows, tile 1 the 16 up rows of the same columns, and the block stores silu(gate) * up [M, N]:
// the SwiGLU of a gated feed-forward without a pass of its own.
// (The products of at most 16 rows with weights copied into MFMA tile order are in gemm_decode.hip.)
template <int MT, int NT, int WAVES, typename TC, bool GATED = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                                 TC* __restrict__ C, int M, int N, int K) {
    __shared__ float red[(WAVES - 1) * NT * MT * 64 * 4];
    // the wave index is the same in all lanes: keep it in a scalar register so that loops over it are scalar too
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int n_base = GATED ? blockIdx.x * 16 : blockIdx.x * (16 * NT);
    f32x4_t acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Rows beyond N or M are clamped to the last row: their products land in outputs that are
    // never stored, and the main loop needs no per-lane predicates.  Addresses are a base that is
    // the same in all lanes (it advances with the chunk) plus a 32-bit lane offset that never
    // changes, so the loop recomputes no per-lane address.
    const char* wbase = reinterpret_cast<const char*>(W) + (size_t)n_base * K * 2;
    const char* xbase = reinterpret_cast<const char*>(X);
    unsigned woff[NT], xoff[MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int row = GATED ? nt * N + min(n_base + r, N - 1) : min(n_base + nt * 16 + r, N - 1);
        woff[nt] = (unsigned)(row - n_base) * (unsigned)K * 2u + 16u * g;
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xoff[mt] = (unsigned)min(mt * 16 + r, M - 1) * (unsigned)K * 2u + 16u * g;
    // lanes whose row of X does not exist load nothing (their columns of the result are not stored):
    // with few rows most lanes of the X loads stay idle, which the memory pipeline notices
    bool xok[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xok[mt] = mt * 16 + r < M;
    const bf16_t* wrow[NT];
    const bf16_t* xrow[MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) wrow[nt] = reinterpret_cast<const bf16_t*>(wbase + woff[nt]);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xrow[mt] = reinterpret_cast<const bf16_t*>(xbase + xoff[mt]);

    bf16x8_t a0[NT][4], b0[MT][4], a1[NT][4], b1[MT][4];
#define SK_LOAD(A, B, CHUNK)                                                                         \
    {                                                                                                \
        const char* wb_ = wbase + (size_t)(CHUNK) * (SK_CHUNK * 2);                                  \
        const char* xb_ = xbase + (size_t)(CHUNK) * (SK_CHUNK * 2);                                  \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                              \
            _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                        \
                A[nt][j] = *reinterpret_cast<const bf16x8_t*>(wb_ + woff[nt] + 64 * j);                  \
            _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                        \
                B[mt][j] = load8(reinterpret_cast<const bf16_t*>(xb_ + xoff[mt] + 64 * j), xok[mt]); \
        }                                                                                            \
    }
#define SK_MFMA(A, B, ACC)                                                                           \
    _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                    \
        _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                            \
            _Pragma("unroll") for (int mt = 0; mt < MT; ++mt)                                        \
                ACC[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[nt][j], B[mt][j], ACC[nt][mt], 0, 0, 0);

    // Full chunks, two per round with accumulators of their own (added at the end).  The loop is
    // kept this plain on purpose: a version that issued the next round's loads before this round's
    // products was compiled into code that overwrote live registers.
    f32x4_t acc2[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc2[nt][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const int nfull = K / SK_CHUNK;
    int c = wave;
    for (; c + WAVES < nfull; c += 2 * WAVES) {     // two chunks of this wave per round: 8 loads of W per lane in flight
        SK_LOAD(a0, b0, c)
        SK_LOAD(a1, b1, c + WAVES)
        SK_MFMA(a0, b0, acc)
        SK_MFMA(a1, b1, acc2)
    }
    if (c < nfull) {
        SK_LOAD(a0, b0, c)
        SK_MFMA(a0, b0, acc)
    }
#undef SK_LOAD
#undef SK_MFMA
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] += acc2[nt][mt];
    // the rest of K (fewer than 128 values; K is a multiple of 8), by the wave whose turn it is
    if (nfull * SK_CHUNK < K && wave == nfull % WAVES) {
        const int kc = nfull * SK_CHUNK;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool kok = kc + 32 * j + 8 * g < K;
            bf16x8_t a[NT], b[MT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) a[nt] = load8(wrow[nt] + kc + 32 * j, kok);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) b[mt] = load8(xrow[mt] + kc + 32 * j, kok && xok[mt]);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt], b[mt], acc[nt][mt], 0, 0, 0);
        }
    }

    if (WAVES > 1) {
        if (wave > 0) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        red[((((wave - 1) * NT + nt) * MT + mt) * 4 + i) * 64 + lane] = acc[nt][mt][i];
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[nt][mt][i] += red[((((w - 1) * NT + nt) * MT + mt) * 4 + i) * 64 + lane];
    }
    if (GATED) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r;
            const int n = n_base + 4 * g;
            if (m >= M) continue;
            TC* out = C + (size_t)m * N + n;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float gt = acc[0][mt][i], up = acc[NT - 1][mt][i];
                if (n + i < N) out[i] = from_f32<TC>((gt / (1.0f + expf(-gt))) * up);
            }
        }
        return;
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r;
            const int n = n_base + nt * 16 + 4 * g;
            if (m >= M) continue;
            TC* out = C + (size_t)m * N + n;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (n + i < N) out[i] = from_f32<TC>(acc[nt][mt][i]);
        }
}

template <int MT, int NT, int WAVES, typename TC>
static void launch_skinny(const bf16_t* X, const bf16_t* W, void* C, int M, int N, int K, hipStream_t st) {
    const int blocks = (N + 16 * NT - 1) / (16 * NT);
    gemm_skinny_kernel<MT, NT, WAVES, TC><<<blocks, WAVES * 64, 0, st>>>(X, W, (TC*)C, M, N, K);
}

template <int MT, typename TC>
static void pick_skinny(const bf16_t* X, const bf16_t* W, void* C, int M, int N, int K, hipStream_t st) {
    // Measured on MI355X at the Qwen3-8B shapes (N 4096..151936, K 4096..12288) with 1 and 8 rows:
    // one 16-row tile per block and 8 waves sharing K was the best or within 3 % of it everywhere.
    launch_skinny<MT, 1, 8, TC>(X, W, C, M, N, K, st);
}

// out[M, I] = silu(X . Wgate^T) * (X . Wup^T) with W = [Wgate | Wup] stored [2 I, K]
extern "C" int spy_gemm_skinny_swiglu(const void* X, const void* W, void* C, int c_dtype, int M, int I, int K, hipStream_t st) {
    SPY_REQUIRE(M > 0 && I > 0 && K > 0, "spy_gemm_skinny_swiglu: empty operand");
    SPY_REQUIRE(M <= 16, "spy_gemm_skinny_swiglu: M = %d exceeds 16 rows", M);
    SPY_REQUIRE(K % 8 == 0, "spy_gemm_skinny_swiglu: K = %d is not a multiple of 8", K);
    SPY_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0, "spy_gemm_skinny_swiglu: operands must be 16-byte aligned");
    SPY_REQUIRE((long long)(I + 16) * K * 2 < (1ll << 32), "spy_gemm_skinny_swiglu: the gate and up rows lie too far apart");
    const int blocks = (I + 15) / 16;
    if (c_dtype == SPY_F32)
        gemm_skinny_kernel<1, 2, 8, float, true><<<blocks, 8 * 64, 0, st>>>((const bf16_t*)X, (const bf16_t*)W, (float*)C, M, I, K);
    else
        gemm_skinny_kernel<1, 2, 8, bf16_t, true><<<blocks, 8 * 64, 0, st>>>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)C, M, I, K);
    SPY_CHECK_LAUNCH("spy_gemm_skinny_swiglu");
    return 0;
}

extern "C" int spy_gemm_skinny(const void* X, const void* W, void* C, int c_dtype, int M, int N, int K, hipStream_t st) {
    SPY_REQUIRE(M > 0 && N > 0 && K > 0, "spy_gemm_skinny: empty operand");
    SPY_REQUIRE(M <= 64, "spy_gemm_skinny: M = %d exceeds 64 rows", M);
    SPY_REQUIRE(K % 8 == 0, "spy_gemm_skinny: K = %d is not a multiple of 8 (rows must be 16-byte aligned)", K);
    SPY_REQUIRE(((uintptr_t)X % 16) == 0 && ((uintptr_t)W % 16) == 0, "spy_gemm_skinny: operands must be 16-byte aligned");
    const bf16_t* x = (const bf16_t*)X;
    const bf16_t* w = (const bf16_t*)W;
    const int mt = (M + 15) / 16;
#define SK_CASE(MT_)                                                            \
    case MT_:                                                                   \
        if (c_dtype == SPY_F32) pick_skinny<MT_, float>(x, w, C, M, N, K, st);  \
        else pick_skinny<MT_, bf16_t>(x, w, C, M, N, K, st);                    \
        break;
    switch (mt) {
        SK_CASE(1) SK_CASE(2) SK_CASE(3) SK_CASE(4)
    }
#undef SK_CASE
    SPY_CHECK_LAUNCH("spy_gemm_skinny");
    return 0;
}
