// C[M, N] = A[M, K] . W[N, K]^T with float32 products and sums (no reduced-precision matrix
// mode), operands float32 or bfloat16 in any combination.  This is the true 32-bit product of
// the engine and the fallback for shapes the MFMA kernels refuse.  A 64x64 tile of C per block,
// 16x16 threads with 4x4 outputs each, K walked in steps of 16 through LDS.  Each output sums its
// products in ascending k, so a row's result does not depend on the other rows of the batch.
#include "common.h"

#define GT 64
#define GK 16

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                           TC* __restrict__ C, int M, int N, int K) {
    __shared__ float As[GK][GT + 4];
    __shared__ float Ws[GK][GT + 4];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    float acc[4][4] = {};
    // each thread stages 4 elements of A and of W per step: row = tid / 4 (+0), k = (tid % 4) * 4 .. +3
    const int lr = threadIdx.x >> 2, lk = (threadIdx.x & 3) * 4;
    for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k = k0 + lk + e;
            const int am = m0 + lr, wn = n0 + lr;
            As[lk + e][lr] = (am < M && k < K) ? to_f32<TA>(A[(size_t)am * K + k]) : 0.f;
            Ws[lk + e][lr] = (wn < N && k < K) ? to_f32<TW>(W[(size_t)wn * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[k][ty * 4 + i]; b[i] = Ws[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) C[(size_t)m * N + n] = from_f32<TC>(acc[i][j]);
        }
    }
}

extern "C" int spy_gemm(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype, int M, int N, int K,
                        hipStream_t st) {
    SPY_REQUIRE(M > 0 && N > 0 && K > 0, "spy_gemm: empty operand");
    const dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT);
    SPY_REQUIRE(grid.y <= 65535, "spy_gemm: M = %d is too large for this kernel", M);
    SPY_DISPATCH(a_dtype, TA, SPY_DISPATCH(w_dtype, TW, SPY_DISPATCH(c_dtype, TC, (gemm_generic_kernel<TA, TW, TC><<<grid, 256, 0, st>>>(
        (const TA*)A, (const TW*)W, (TC*)C, M, N, K)))));
    SPY_CHECK_LAUNCH("spy_gemm");
    return 0;
}
