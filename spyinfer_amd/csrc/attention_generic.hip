// Plain paged attention, float32 throughout: one block per (query token, query head).  It is the
// attention of the float32 path and the fallback for shapes that the MFMA kernel refuses.
// Keys are walked in chunks of 128 with a running maximum and sum (same result as a two-pass
// softmax up to rounding).  Cache layout: K [pages, n_kv, P, d], V [pages, n_kv, d, P].
#include "common.h"
#include <math.h>

#define AG_THREADS 128
#define AG_MAX_D 512

template <typename TA>
__global__ __launch_bounds__(AG_THREADS) void attention_generic_kernel(
    TA* __restrict__ out, const TA* __restrict__ q, const TA* __restrict__ kc, const TA* __restrict__ vc, int P, int num_pages,
    const int* __restrict__ kv_len, const int* __restrict__ block_table, int max_blocks, const int* __restrict__ token_entry,
    const int* __restrict__ positions, int n_q, int n_kv, int d, float scale, int window) {
    __shared__ float qs[AG_MAX_D];
    __shared__ float ps[AG_THREADS];
    __shared__ int pg[AG_THREADS];
    __shared__ int of[AG_THREADS];
    __shared__ float red[4];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int s = token_entry[t];
    const int p = positions[t];
    const int g = (int)(((long long)h * n_kv) / n_q);
    int hi = p;                                   // last key read (causal)
    if (hi > kv_len[s] - 1) hi = kv_len[s] - 1;
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const TA* qv = q + ((size_t)t * n_q + h) * d;
    for (int j = tid; j < d; j += AG_THREADS) qs[j] = to_f32<TA>(qv[j]);
    float acc[AG_MAX_D / AG_THREADS] = {};
    float m = -INFINITY, l = 0.f;
    const int* bt = block_table + (size_t)s * max_blocks;
    __syncthreads();
    for (int c0 = lo; c0 <= hi; c0 += AG_THREADS) {
        const int c = c0 + tid;
        float sc = -INFINITY;
        int page = -1, off = 0;
        if (c <= hi) {
            page = bt[c / P];
            off = c % P;
            if (page >= 0 && page < num_pages) {
                const TA* kr = kc + (((size_t)page * n_kv + g) * P + off) * d;
                float dot = 0.f;
                for (int j = 0; j < d; ++j) dot = fmaf(qs[j], to_f32<TA>(kr[j]), dot);
                sc = dot * scale;
            } else {
                page = -1;   // a key without a page is not read (never the case for a checked batch)
            }
        }
        const float cm = block_max(sc, red);
        const float m_new = fmaxf(m, cm);
        const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
        const float pr = (sc == -INFINITY) ? 0.f : expf(sc - m_new);
        ps[tid] = pr; pg[tid] = page; of[tid] = off;
        const float csum = block_sum(pr, red);      // has the barriers that publish ps/pg/of
        l = l * alpha + csum;
        m = m_new;
        const int nk = min(AG_THREADS, hi - c0 + 1);
#pragma unroll
        for (int r = 0; r < AG_MAX_D / AG_THREADS; ++r) {
            const int j = tid + r * AG_THREADS;
            if (j < d) {
                float a = acc[r] * alpha;
                for (int i = 0; i < nk; ++i) {
                    if (pg[i] >= 0) a = fmaf(ps[i], to_f32<TA>(vc[(((size_t)pg[i] * n_kv + g) * d + j) * P + of[i]]), a);
                }
                acc[r] = a;
            }
        }
        __syncthreads();
    }
    TA* o = out + ((size_t)t * n_q + h) * d;
#pragma unroll
    for (int r = 0; r < AG_MAX_D / AG_THREADS; ++r) {
        const int j = tid + r * AG_THREADS;
        if (j < d) o[j] = from_f32<TA>(l > 0.f ? acc[r] / l : 0.f);
    }
}

extern "C" int spy_attention_generic(void* out, const void* q, int dtype, const void* kc, const void* vc, int P, int num_pages,
                                     const int* kv_len, const int* block_table, int max_blocks, const int* token_entry,
                                     const int* positions, int S, int T, int n_q, int n_kv, int d, float scale, int window,
                                     hipStream_t st) {
    SPY_REQUIRE(T > 0 && S > 0 && n_q > 0 && n_kv > 0 && d > 0 && P > 0 && num_pages > 0 && max_blocks > 0,
                "spy_attention_generic: empty operand");
    SPY_REQUIRE(d <= AG_MAX_D, "spy_attention_generic: head_dim %d exceeds the supported %d", d, AG_MAX_D);
    SPY_REQUIRE(n_q <= 65535, "spy_attention_generic: too many heads");
    const dim3 grid(T, n_q);
    SPY_DISPATCH(dtype, TA, (attention_generic_kernel<TA><<<grid, AG_THREADS, 0, st>>>(
        (TA*)out, (const TA*)q, (const TA*)kc, (const TA*)vc, P, num_pages, kv_len, block_table, max_blocks, token_entry,
        positions, n_q, n_kv, d, scale, window)));
    SPY_CHECK_LAUNCH("spy_attention_generic");
    return 0;
}
