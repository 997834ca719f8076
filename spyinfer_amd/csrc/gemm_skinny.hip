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

template <int MT, int NT, int WAVES, typename TC>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                                 TC* __restrict__ C, int M, int N, int K) {
    __shared__ float red[(WAVES - 1) * NT * MT * 64 * 4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int n_base = blockIdx.x * (16 * NT);
    f32x4_t acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    const bf16_t* wrow[NT];
    bool wok[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int n = n_base + nt * 16 + r;
        wok[nt] = n < N;
        wrow[nt] = W + (size_t)(wok[nt] ? n : 0) * K;
    }
    const bf16_t* xrow[MT];
    bool xok[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        xok[mt] = m < M;
        xrow[mt] = X + (size_t)(xok[mt] ? m : 0) * K;
    }

    for (int kc = wave * SK_CHUNK; kc < K; kc += WAVES * SK_CHUNK) {
        bf16x8_t a[NT][4], b[MT][4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = kc + 32 * j + 8 * g;
            const bool kok = k < K;          // K is a multiple of 8: a lane's 8 elements are all inside or all outside
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) a[nt][j] = load8(wrow[nt] + k, kok && wok[nt]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) b[mt][j] = load8(xrow[mt] + k, kok && xok[mt]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt][j], b[mt][j], acc[nt][mt], 0, 0, 0);
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
    const int tiles = (N + 15) / 16;
    // many rows of W: two tiles per wave halve the traffic of X; few rows: more waves share K
    if (tiles >= 2048 && MT <= 2) launch_skinny<MT, 2, 4, TC>(X, W, C, M, N, K, st);
    else if (tiles >= 1024) launch_skinny<MT, 1, 4, TC>(X, W, C, M, N, K, st);
    else launch_skinny<MT, 1, 8, TC>(X, W, C, M, N, K, st);
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
