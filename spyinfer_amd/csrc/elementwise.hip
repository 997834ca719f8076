// Embedding gather, RMS norm with the residual sum folded in, SwiGLU, and the fused
// per-head norm + rotation + cache store.  All arithmetic is float32; a bfloat16 value is
// rounded once, when it is written.
#include "common.h"

// ---------------------------------------------------------------------------------------------
// out[t, :] = table[ids[t], :]  (float32 out: the start of the residual stream)
template <typename TW>
__global__ void embedding_kernel(float* __restrict__ out, const TW* __restrict__ table, const int* __restrict__ ids, int H, int V) {
    const int t = blockIdx.x;
    const int id = ids[t];
    float* o = out + (size_t)t * H;
    if (id < 0 || id >= V) {
        for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = 0.f;
        return;
    }
    const TW* row = table + (size_t)id * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_f32<TW>(row[i]);
}

extern "C" int spy_embedding(float* out, const void* table, int table_dtype, const int* ids, int T, int H, int V, hipStream_t st) {
    SPY_REQUIRE(T > 0 && H > 0 && V > 0, "spy_embedding: empty operand");
    SPY_DISPATCH(table_dtype, TW, embedding_kernel<TW><<<T, 256, 0, st>>>(out, (const TW*)table, ids, H, V));
    SPY_CHECK_LAUNCH("spy_embedding");
    return 0;
}

// The same for at most 64 tokens, prepared for a product that applies the first RMS norm's scale after its sum:
// xw[t] = bf16(h[t] * w_norm) and ss[t] = sum(h[t]^2) (ss[T ..] = 0 up to the next multiple of 16).
// tiled: xw in MFMA operand order, [H/32][MT row tiles][64 lanes][8] with lane 16 g + t % 16 of row tile t / 16 holding
// xw[t][32 s + 8 g ..] (H % 32 == 0); MT = the row tiles that T tokens need.  One block per row of ss (16 MT of them).
template <typename TW>
__global__ __launch_bounds__(256) void embedding_sumsq_kernel(float* __restrict__ out, bf16_t* __restrict__ xw, float* __restrict__ ss,
                                                              const TW* __restrict__ table, const bf16_t* __restrict__ w_norm,
                                                              const int* __restrict__ ids, int T, int H, int V, int tiled) {
    __shared__ float red[8];
    const int t = blockIdx.x;
    if (t >= T) { if (threadIdx.x == 0) ss[t] = 0.f; return; }
    const int id = ids[t];
    float* o = out + (size_t)t * H;
    bf16_t* x = xw + (size_t)t * H;
    const TW* row = table + (size_t)(id < 0 || id >= V ? 0 : id) * H;
    const bool known = id >= 0 && id < V;
    float s = 0.f;
    if (H % 8 == 0 && ((uintptr_t)table % 16) == 0 && ((uintptr_t)w_norm % 16) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)xw % 16) == 0) {
        // 8 values per thread and step: one or two 16-byte loads of the row, one of the weight, two 16-byte stores of
        // the stream and one of the product's input (8 consecutive columns are one piece in operand order too)
        typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
        typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f4_t;
        for (int i = threadIdx.x * 8; i < H; i += blockDim.x * 8) {
            float v[8];
            if (sizeof(TW) == 2) {
                const u32x4_t r4 = *reinterpret_cast<const u32x4_t*>(row + i);
#pragma unroll
                for (int e = 0; e < 4; ++e) { v[2 * e] = __uint_as_float(r4[e] << 16); v[2 * e + 1] = __uint_as_float(r4[e] & 0xffff0000u); }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = to_f32<TW>(row[i + e]);
            }
            const u32x4_t w4 = *reinterpret_cast<const u32x4_t*>(w_norm + i);
            u32x4_t y;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (!known) { v[2 * e] = 0.f; v[2 * e + 1] = 0.f; }
                y[e] = pack_bf16x2(v[2 * e] * __uint_as_float(w4[e] << 16), v[2 * e + 1] * __uint_as_float(w4[e] & 0xffff0000u));
                s += v[2 * e] * v[2 * e] + v[2 * e + 1] * v[2 * e + 1];
            }
            *reinterpret_cast<f4_t*>(o + i) = f4_t{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<f4_t*>(o + i + 4) = f4_t{v[4], v[5], v[6], v[7]};
            bf16_t* dst = tiled ? xw + (((size_t)(i >> 5) * (gridDim.x >> 4) + (t >> 4)) * 64 + ((i & 31) >> 3) * 16 + (t & 15)) * 8 : x + i;
            *reinterpret_cast<u32x4_t*>(dst) = y;
        }
        s = block_sum(s, red);
        if (threadIdx.x == 0) ss[t] = s;
        return;
    }
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float v = known ? to_f32<TW>(row[i]) : 0.f;
        o[i] = v;
        const bf16_t y = f32_to_bf16(v * bf16_to_f32(w_norm[i]));
        if (tiled) xw[(((size_t)(i >> 5) * (gridDim.x >> 4) + (t >> 4)) * 64 + ((i & 31) >> 3) * 16 + (t & 15)) * 8 + (i & 7)] = y;
        else x[i] = y;
        s += v * v;
    }
    s = block_sum(s, red);
    if (threadIdx.x == 0) ss[t] = s;
}

// row_tiles: the 16-row tiles that the products reading the result are built with (at least T / 16; ss and the operand
// order have that many).
extern "C" int spy_embedding_sumsq(float* out, void* xw, float* ss, const void* table, int table_dtype, const void* w_norm,
                                   const int* ids, int T, int H, int V, int tiled, int row_tiles, hipStream_t st) {
    SPY_REQUIRE(T > 0 && T <= 128 && H > 0 && V > 0, "spy_embedding_sumsq: T = %d tokens (1..128 allowed)", T);
    SPY_REQUIRE(row_tiles * 16 >= T && row_tiles <= 8, "spy_embedding_sumsq: %d row tiles for %d tokens", row_tiles, T);
    SPY_REQUIRE(!tiled || H % 32 == 0, "spy_embedding_sumsq: operand order needs a width that is a multiple of 32, not %d", H);
    SPY_DISPATCH(table_dtype, TW, embedding_sumsq_kernel<TW><<<row_tiles * 16, 256, 0, st>>>(out, (bf16_t*)xw, ss, (const TW*)table,
                                                                                 (const bf16_t*)w_norm, ids, T, H, V, tiled));
    SPY_CHECK_LAUNCH("spy_embedding_sumsq");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// x = resid[t] (+ delta[t]);  rows == null: resid[t] = x.  out[r] = (x / sqrt(mean(x^2) + eps)) * w
// One block per row.  The row is read once and kept in registers (4 values per thread and pass,
// up to NORM_PASSES passes); longer rows are read again for the second pass.
#define NORM_PASSES 8
template <typename TA> struct Vec4;
template <> struct Vec4<float> {
    typedef float4 type;
    static __device__ __forceinline__ void load(const float* p, float* v) { const float4 t = *reinterpret_cast<const float4*>(p); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
    static __device__ __forceinline__ void store(float* p, const float* v) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct Vec4<bf16_t> {
    static __device__ __forceinline__ void load(const bf16_t* p, float* v) {
        const uint2 t = *reinterpret_cast<const uint2*>(p);
        v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
        v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
    }
    static __device__ __forceinline__ void store(bf16_t* p, const float* v) {
        uint2 t;
        t.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
        t.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
        *reinterpret_cast<uint2*>(p) = t;
    }
};

template <typename TA, typename TW, bool VEC>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const TA* __restrict__ delta, const TW* __restrict__ w, float eps,
                                   TA* __restrict__ out, const int* __restrict__ rows, int T, int H) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    int t = r;
    if (rows) {
        t = rows[r];
        if (t < 0 || t >= T) {   // never the case for a checked batch; write zeros rather than read outside
            for (int i = threadIdx.x; i < H; i += blockDim.x) out[(size_t)r * H + i] = from_f32<TA>(0.f);
            return;
        }
    }
    float* x = resid + (size_t)t * H;
    const TA* dl = delta ? delta + (size_t)t * H : nullptr;
    TA* o = out + (size_t)r * H;
    const bool write_back = dl && !rows;
    if (VEC) {
        // H % 4 == 0 and 16-byte aligned rows (checked by the launcher); the row fits the register passes
        float v[NORM_PASSES][4];
        float ss = 0.f;
#pragma unroll
        for (int p = 0; p < NORM_PASSES; ++p) {
            const int i = (p * blockDim.x + threadIdx.x) * 4;
            if (i < H) {
                Vec4<float>::load(x + i, v[p]);
                if (dl) {
                    float d4[4];
                    Vec4<TA>::load(dl + i, d4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[p][e] += d4[e];
                }
                if (write_back) Vec4<float>::store(x + i, v[p]);
#pragma unroll
                for (int e = 0; e < 4; ++e) ss += v[p][e] * v[p][e];
            }
        }
        ss = block_sum(ss, red);
        const float scale = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
        for (int p = 0; p < NORM_PASSES; ++p) {
            const int i = (p * blockDim.x + threadIdx.x) * 4;
            if (i < H) {
                float w4[4], y[4];
                Vec4<TW>::load(w + i, w4);
#pragma unroll
                for (int e = 0; e < 4; ++e) y[e] = (scale * v[p][e]) * w4[e];
                Vec4<TA>::store(o + i, y);
            }
        }
        return;
    }
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float v = x[i];
        if (dl) v += to_f32<TA>(dl[i]);
        if (write_back) x[i] = v;
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float v = x[i];
        if (dl && rows) v += to_f32<TA>(dl[i]);
        o[i] = from_f32<TA>((scale * v) * to_f32<TW>(w[i]));
    }
}

extern "C" int spy_add_rmsnorm(float* resid, const void* delta, const void* w, int w_dtype, float eps, void* out, int out_dtype,
                               const int* rows, int n_out, int T, int H, hipStream_t st) {
    SPY_REQUIRE(n_out > 0 && T > 0 && H > 0, "spy_add_rmsnorm: empty operand");
    const int threads = H >= 2048 ? 256 : (H >= 512 ? 128 : 64);
    const bool aligned = H % 4 == 0 && ((uintptr_t)resid % 16) == 0 && ((uintptr_t)delta % 16) == 0 && ((uintptr_t)w % 16) == 0 &&
                         ((uintptr_t)out % 16) == 0;
    const bool vec = aligned && H <= threads * 4 * NORM_PASSES;
    if (vec) {
        SPY_DISPATCH(out_dtype, TA, SPY_DISPATCH(w_dtype, TW, (add_rmsnorm_kernel<TA, TW, true><<<n_out, threads, 0, st>>>(
            resid, (const TA*)delta, (const TW*)w, eps, (TA*)out, rows, T, H))));
    } else {
        SPY_DISPATCH(out_dtype, TA, SPY_DISPATCH(w_dtype, TW, (add_rmsnorm_kernel<TA, TW, false><<<n_out, 512, 0, st>>>(
            resid, (const TA*)delta, (const TW*)w, eps, (TA*)out, rows, T, H))));
    }
    SPY_CHECK_LAUNCH("spy_add_rmsnorm");
    return 0;
}

template <typename TA, typename TW>
__global__ void rmsnorm_kernel(const TA* __restrict__ x, const TW* __restrict__ w, float eps, TA* __restrict__ out, int n) {
    __shared__ float red[16];
    const TA* xr = x + (size_t)blockIdx.x * n;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) { float v = to_f32<TA>(xr[i]); ss += v * v; }
    ss = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)n + eps);
    TA* o = out + (size_t)blockIdx.x * n;
    for (int i = threadIdx.x; i < n; i += blockDim.x) o[i] = from_f32<TA>((scale * to_f32<TA>(xr[i])) * to_f32<TW>(w[i]));
}

extern "C" int spy_rmsnorm(const void* x, int x_dtype, const void* w, int w_dtype, float eps, void* out, int64_t rows, int n,
                           hipStream_t st) {
    SPY_REQUIRE(rows > 0 && rows < (1ll << 31) && n > 0, "spy_rmsnorm: bad sizes");
    const int threads = n >= 1024 ? 512 : (n > 64 ? 256 : 64);
    SPY_DISPATCH(x_dtype, TA, SPY_DISPATCH(w_dtype, TW, (rmsnorm_kernel<TA, TW><<<(unsigned)rows, threads, 0, st>>>(
        (const TA*)x, (const TW*)w, eps, (TA*)out, n))));
    SPY_CHECK_LAUNCH("spy_rmsnorm");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// out[t, i] = silu(in[t, i]) * in[t, I + i]
template <typename TA>
__global__ void swiglu_kernel(const TA* __restrict__ in, TA* __restrict__ out, int T, int I) {
    const size_t n = (size_t)T * I;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (size_t)gridDim.x * blockDim.x) {
        const size_t t = idx / I, i = idx - t * I;
        const float g = to_f32<TA>(in[t * 2 * I + i]);
        const float u = to_f32<TA>(in[t * 2 * I + I + i]);
        out[idx] = from_f32<TA>((g / (1.0f + expf(-g))) * u);
    }
}

// the same, 4 values per thread and step with vector loads (I % 4 == 0, 16-byte aligned rows)
template <typename TA>
__global__ void swiglu_vec_kernel(const TA* __restrict__ in, TA* __restrict__ out, int T, int I4) {
    const size_t n = (size_t)T * I4;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (size_t)gridDim.x * blockDim.x) {
        const size_t t = idx / I4, i = (idx - t * I4) * 4;
        const size_t I = (size_t)I4 * 4;
        float g[4], u[4], y[4];
        Vec4<TA>::load(in + t * 2 * I + i, g);
        Vec4<TA>::load(in + t * 2 * I + I + i, u);
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = (g[e] / (1.0f + expf(-g[e]))) * u[e];
        Vec4<TA>::store(out + t * I + i, y);
    }
}

// bfloat16, 8 values per thread and step: 16-byte loads that do not stay in the caches (the product's output passes
// once), one 16-byte store (the next product reads it)
__global__ void swiglu_bf16x8_kernel(const bf16_t* __restrict__ in, bf16_t* __restrict__ out, int T, int I8) {
    typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
    const size_t n = (size_t)T * I8, I = (size_t)I8 * 8;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (size_t)gridDim.x * blockDim.x) {
        const size_t t = idx / I8, i = (idx - t * I8) * 8;
        const u32x4_t g = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(in + t * 2 * I + i));
        const u32x4_t u = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(in + t * 2 * I + I + i));
        u32x4_t y;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float g0 = __uint_as_float(g[e] << 16), g1 = __uint_as_float(g[e] & 0xffff0000u);
            const float u0 = __uint_as_float(u[e] << 16), u1 = __uint_as_float(u[e] & 0xffff0000u);
            y[e] = pack_bf16x2((g0 / (1.0f + expf(-g0))) * u0, (g1 / (1.0f + expf(-g1))) * u1);
        }
        *reinterpret_cast<u32x4_t*>(out + t * I + i) = y;
    }
}

extern "C" int spy_swiglu(const void* in, void* out, int dtype, int T, int I, hipStream_t st) {
    SPY_REQUIRE(T > 0 && I > 0, "spy_swiglu: empty operand");
    const bool vec = I % 8 == 0 && ((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 16) == 0;
    const size_t n = (size_t)T * I / (vec ? 4 : 1);
    const unsigned blocks = (unsigned)((n + 255) / 256 > 65536 ? 65536 : (n + 255) / 256);
    if (vec && dtype == SPY_BF16) {
        const size_t n8 = (size_t)T * I / 8;
        const unsigned b8 = (unsigned)((n8 + 255) / 256 > 65536 ? 65536 : (n8 + 255) / 256);
        swiglu_bf16x8_kernel<<<b8, 256, 0, st>>>((const bf16_t*)in, (bf16_t*)out, T, I / 8);
    } else if (vec) {
        SPY_DISPATCH(dtype, TA, swiglu_vec_kernel<TA><<<blocks, 256, 0, st>>>((const TA*)in, (TA*)out, T, I / 4));
    } else {
        SPY_DISPATCH(dtype, TA, swiglu_kernel<TA><<<blocks, 256, 0, st>>>((const TA*)in, (TA*)out, T, I));
    }
    SPY_CHECK_LAUNCH("spy_swiglu");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// A matrix [N, K] back from the order the decode products read it ([K/128 chunks][N/16 tiles][4 steps][g = 4][r = 16][8])
// into rows, for the library's products of many rows when only that copy of the matrix is kept.  A block moves
// UNTILE_TILES tiles of 16 rows x 128 columns (4 KiB each, one piece of the source); thread (r, step, g) of a tile
// writes 16 bytes of row r, so that 16 neighbouring lanes write 256 bytes of one row.
#define UNTILE_TILES 4
__global__ __launch_bounds__(256) void untile_weight_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ tiled, int N, int K,
                                                            size_t n_tiles) {
    typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
    const int r = threadIdx.x >> 4, sg = threadIdx.x & 15;
    const size_t col_tiles = (size_t)(N / 16);
    for (size_t t = (size_t)blockIdx.x * UNTILE_TILES; t < n_tiles; t += (size_t)gridDim.x * UNTILE_TILES) {
        u32x4_t v[UNTILE_TILES];
#pragma unroll
        for (int i = 0; i < UNTILE_TILES; ++i)
            if (t + i < n_tiles) v[i] = *reinterpret_cast<const u32x4_t*>(tiled + ((t + i) * 256 + sg * 16 + r) * 8);
#pragma unroll
        for (int i = 0; i < UNTILE_TILES; ++i) {
            if (t + i < n_tiles) {
                const size_t chunk = (t + i) / col_tiles, tile = (t + i) % col_tiles;
                *reinterpret_cast<u32x4_t*>(out + (tile * 16 + r) * (size_t)K + chunk * 128 + sg * 8) = v[i];
            }
        }
    }
}

extern "C" int spy_untile_weight(void* out, const void* tiled, int N, int K, hipStream_t st) {
    SPY_REQUIRE(N > 0 && K > 0 && N % 16 == 0 && K % 128 == 0, "spy_untile_weight: [%d, %d] is not made of tiles of 16 x 128", N, K);
    const size_t n_tiles = (size_t)(N / 16) * (size_t)(K / 128);
    const size_t want = (n_tiles + UNTILE_TILES - 1) / UNTILE_TILES;
    untile_weight_kernel<<<(unsigned)(want > 65536 ? 65536 : want), 256, 0, st>>>((bf16_t*)out, (const bf16_t*)tiled, N, K, n_tiles);
    SPY_CHECK_LAUNCH("spy_untile_weight");
    return 0;
}

// ---------------------------------------------------------------------------------------------
// One wave per (token, head of q|k|v), QK_WAVES heads per block.  q, k: optional RMS norm over the head,
// then half-split rotation of the first `rot` dims: y[j] = x[j] c - x[j+rot/2] s; y[j+rot/2] = x[j] s + x[j+rot/2] c.
// A lane holds both members of its pairs, so the rotation needs no exchange between lanes.
// q -> q_out[t, h, :];  k -> K[page, h, off, :];  v -> V[page, h, :, off]  (values lie transposed in a page).
#define QK_MAX_D 512
#define QK_WAVES 4
template <typename TA, typename TW>
__global__ __launch_bounds__(QK_WAVES * 64) void qknorm_rope_store_kernel(
    const TA* __restrict__ qkv, TA* __restrict__ q_out, int n_q, int n_kv, int d, const TW* __restrict__ qw,
    const TW* __restrict__ kw, float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, int max_pos,
    const int* __restrict__ positions, TA* __restrict__ kc, TA* __restrict__ vc, int P, int num_pages, const int* __restrict__ slots) {
    const int t = blockIdx.x, lane = threadIdx.x & 63;
    const int h = blockIdx.y * QK_WAVES + (threadIdx.x >> 6);
    const int heads = n_q + 2 * n_kv;
    if (h >= heads) return;
    const TA* x = qkv + (size_t)t * heads * d + (size_t)h * d;
    const bool is_q = h < n_q, is_k = !is_q && h < n_q + n_kv;
    int page = -1, off = 0;
    if (!is_q) {
        if (!slots) return;
        const int slot = slots[t];
        if (slot < 0 || slot >= num_pages * P) return;
        page = slot / P;
        off = slot - page * P;
    }
    if (!is_q && !is_k) {   // values: a plain copy into the transposed page
        const int hv = h - n_q - n_kv;
        TA* dst = vc + ((size_t)page * n_kv + hv) * d * P + off;
        for (int j = lane; j < d; j += 64) dst[(size_t)j * P] = x[j];
        return;
    }
    const int half = rot >> 1;
    constexpr int NP = QK_MAX_D / 2 / 64;     // pairs per lane at most
    float a[NP], b[NP], tail[NP * 2];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int j = lane + 64 * i;
        a[i] = b[i] = 0.f;
        if (j < half) { a[i] = to_f32<TA>(x[j]); b[i] = to_f32<TA>(x[j + half]); }
        ss += a[i] * a[i] + b[i] * b[i];
    }
#pragma unroll
    for (int i = 0; i < NP * 2; ++i) {        // dims at and beyond rot are not rotated
        const int j = rot + lane + 64 * i;
        tail[i] = j < d ? to_f32<TA>(x[j]) : 0.f;
        ss += tail[i] * tail[i];
    }
    const TW* w = is_q ? qw : kw;
    float scale = 1.f;
    if (w) {
        ss = wave_sum(ss);
        scale = 1.0f / sqrtf(ss / (float)d + eps);
    }
    int p = positions[t];
    p = p < 0 ? 0 : (p >= max_pos && max_pos > 0 ? max_pos - 1 : p);
    TA* dst = is_q ? q_out + ((size_t)t * n_q + h) * d : kc + (((size_t)page * n_kv + (h - n_q)) * P + off) * d;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int j = lane + 64 * i;
        if (j < half) {
            float ya = a[i], yb = b[i];
            if (w) { ya = (scale * ya) * to_f32<TW>(w[j]); yb = (scale * yb) * to_f32<TW>(w[j + half]); }
            const float c = cos_t[(size_t)p * half + j], s = sin_t[(size_t)p * half + j];
            dst[j] = from_f32<TA>(ya * c - yb * s);
            dst[j + half] = from_f32<TA>(ya * s + yb * c);
        }
    }
#pragma unroll
    for (int i = 0; i < NP * 2; ++i) {
        const int j = rot + lane + 64 * i;
        if (j < d) dst[j] = from_f32<TA>(w ? (scale * tail[i]) * to_f32<TW>(w[j]) : tail[i]);
    }
}

// The same for many tokens of bfloat16 with the whole head rotated (rot == d) and d in {16, 32, 64, 128, 256}:
// d / 16 lanes per (token, q or k head), each with 8 + 8 values that pair up in the rotation, so all loads and
// stores are 16 bytes; and the values of 16 tokens of a kv head go through LDS, so that 8 tokens that follow each
// other in a page are stored as one 16-byte piece of each row of the transposed page (single stores otherwise).
// Blocks [0, qk_blocks) do q and k, the rest one (16 tokens, kv head) tile of v each.
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t qk_u32x4;
template <typename TW, int LPH>
__global__ __launch_bounds__(256) void qknorm_rope_store_vec_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* __restrict__ q_out, int T, int n_q, int n_kv, const TW* __restrict__ qw,
    const TW* __restrict__ kw, float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int max_pos,
    const int* __restrict__ positions, bf16_t* __restrict__ kc, bf16_t* __restrict__ vc, int P, int num_pages,
    const int* __restrict__ slots, int qk_blocks) {
    constexpr int d = LPH * 16, half = LPH * 8;
    __shared__ __align__(16) bf16_t tile[16 * (d + 8)];
    const int heads = n_q + 2 * n_kv, qk_heads = n_q + n_kv;
    if ((int)blockIdx.x < qk_blocks) {
        const long long u = (long long)blockIdx.x * (256 / LPH) + threadIdx.x / LPH;
        const int sub = threadIdx.x % LPH;
        if (u >= (long long)T * qk_heads) return;
        const int t = (int)(u / qk_heads), h = (int)(u % qk_heads);
        const bool is_q = h < n_q;
        int page = 0, off = 0;
        if (!is_q) {
            if (!slots) return;
            const int slot = slots[t];
            if (slot < 0 || slot >= num_pages * P) return;      // (all LPH lanes of a head take the same way)
            page = slot / P;
            off = slot - page * P;
        }
        const bf16_t* x = qkv + (size_t)t * heads * d + (size_t)h * d + 8 * sub;
        const qk_u32x4 ra = *reinterpret_cast<const qk_u32x4*>(x), rb = *reinterpret_cast<const qk_u32x4*>(x + half);
        float a[8], b[8], ss = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a[2 * i] = __uint_as_float(ra[i] << 16); a[2 * i + 1] = __uint_as_float(ra[i] & 0xffff0000u);
            b[2 * i] = __uint_as_float(rb[i] << 16); b[2 * i + 1] = __uint_as_float(rb[i] & 0xffff0000u);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += a[i] * a[i] + b[i] * b[i];
        const TW* w = is_q ? qw : kw;
        if (w) {
#pragma unroll
            for (int o = 1; o < LPH; o <<= 1) ss += __shfl_xor(ss, o, 64);
            const float scale = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                a[i] = (scale * a[i]) * to_f32<TW>(w[8 * sub + i]);
                b[i] = (scale * b[i]) * to_f32<TW>(w[half + 8 * sub + i]);
            }
        }
        int p = positions[t];
        p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);
        const float* cp = cos_t + (size_t)p * half + 8 * sub;
        const float* sp = sin_t + (size_t)p * half + 8 * sub;
        float ya[8], yb[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float c = cp[i], sn = sp[i];
            ya[i] = a[i] * c - b[i] * sn;
            yb[i] = a[i] * sn + b[i] * c;
        }
        bf16_t* dst = (is_q ? q_out + ((size_t)t * n_q + h) * d : kc + (((size_t)page * n_kv + (h - n_q)) * P + off) * d) + 8 * sub;
        const qk_u32x4 oa = {pack_bf16x2(ya[0], ya[1]), pack_bf16x2(ya[2], ya[3]), pack_bf16x2(ya[4], ya[5]), pack_bf16x2(ya[6], ya[7])};
        const qk_u32x4 ob = {pack_bf16x2(yb[0], yb[1]), pack_bf16x2(yb[2], yb[3]), pack_bf16x2(yb[4], yb[5]), pack_bf16x2(yb[6], yb[7])};
        *reinterpret_cast<qk_u32x4*>(dst) = oa;
        *reinterpret_cast<qk_u32x4*>(dst + half) = ob;
        return;
    }
    // ---- values: 16 tokens of one kv head ---------------------------------------------------------------------
    const int vb = blockIdx.x - qk_blocks;
    const int t0 = (vb / n_kv) * 16, hv = vb % n_kv;
    for (int i = threadIdx.x; i < 16 * (d / 8); i += 256) {
        const int tt = i / (d / 8), c8 = i % (d / 8);
        qk_u32x4 v = {0u, 0u, 0u, 0u};
        if (t0 + tt < T) v = *reinterpret_cast<const qk_u32x4*>(qkv + (size_t)(t0 + tt) * heads * d + (size_t)(qk_heads + hv) * d + 8 * c8);
        *reinterpret_cast<qk_u32x4*>(tile + tt * (d + 8) + 8 * c8) = v;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * d; i += 256) {
        const int j = i % d, tg = i / d;                      // dim j of tokens t0 + 8 tg .. + 7
        const int tb = t0 + 8 * tg;
        if (tb >= T) continue;
        const int s0 = slots[tb];
        bool run = tb + 8 <= T && s0 >= 0 && s0 % 8 == 0 && s0 + 8 <= num_pages * P;
        if (run) {
#pragma unroll
            for (int e = 1; e < 8; ++e) run = run && slots[tb + e] == s0 + e;
        }
        if (run) {                                            // P is a multiple of 8: the 8 slots lie in one page
            uint32_t pk[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                pk[e] = (uint32_t)tile[(8 * tg + 2 * e) * (d + 8) + j] | ((uint32_t)tile[(8 * tg + 2 * e + 1) * (d + 8) + j] << 16);
            const int page = s0 / P, off = s0 - page * P;
            *reinterpret_cast<qk_u32x4*>(vc + (((size_t)page * n_kv + hv) * d + j) * P + off) = qk_u32x4{pk[0], pk[1], pk[2], pk[3]};
        } else {
            for (int e = 0; e < 8 && tb + e < T; ++e) {
                const int slot = slots[tb + e];
                if (slot < 0 || slot >= num_pages * P) continue;
                const int page = slot / P, off = slot - page * P;
                vc[(((size_t)page * n_kv + hv) * d + j) * P + off] = tile[(8 * tg + e) * (d + 8) + j];
            }
        }
    }
}

extern "C" int spy_qknorm_rope_store(const void* qkv, int dtype, void* q_out, int T, int n_q, int n_kv, int d, const void* qw,
                                     const void* kw, int w_dtype, float eps, const float* cos_t, const float* sin_t, int rot,
                                     int max_pos, const int* positions, void* kc, void* vc, int P, int num_pages,
                                     const int* slots, hipStream_t st) {
    SPY_REQUIRE(T > 0 && n_q > 0 && n_kv > 0 && d > 0, "spy_qknorm_rope_store: empty operand");
    SPY_REQUIRE(d <= QK_MAX_D, "spy_qknorm_rope_store: head_dim %d exceeds the supported %d", d, QK_MAX_D);
    SPY_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "spy_qknorm_rope_store: rotary_dim %d does not fit head_dim %d", rot, d);
    SPY_REQUIRE(rot == 0 || (cos_t && sin_t && max_pos > 0), "spy_qknorm_rope_store: rotation without tables");
    SPY_REQUIRE(!slots || (kc && vc && P > 0 && num_pages > 0), "spy_qknorm_rope_store: slots without a cache");
    SPY_REQUIRE(n_q + 2 * n_kv <= 65535 * QK_WAVES, "spy_qknorm_rope_store: too many heads");
    const int wd = w_dtype < 0 ? SPY_F32 : w_dtype;
    // many bfloat16 tokens, whole head rotated, a head size that is 16 times a power of two: the kernel with wide accesses
    if (dtype == SPY_BF16 && T >= 64 && rot == d && (d == 16 || d == 32 || d == 64 || d == 128 || d == 256) && slots && P % 8 == 0 &&
        ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)q_out % 16) == 0 && ((uintptr_t)kc % 16) == 0 && ((uintptr_t)vc % 16) == 0 &&
        (!qw) == (!kw)) {
        const int lph = d / 16;
        const long long units = (long long)T * (n_q + n_kv);
        const long long qk_blocks = (units + 256 / lph - 1) / (256 / lph);
        const long long v_blocks = (long long)((T + 15) / 16) * n_kv;
        SPY_REQUIRE(qk_blocks + v_blocks < (1ll << 31), "spy_qknorm_rope_store: too many tokens");
#define QKV_CASE(L)                                                                                                             \
    SPY_DISPATCH(wd, TW, (qknorm_rope_store_vec_kernel<TW, L><<<(unsigned)(qk_blocks + v_blocks), 256, 0, st>>>(               \
        (const bf16_t*)qkv, (bf16_t*)q_out, T, n_q, n_kv, (const TW*)qw, (const TW*)kw, eps, cos_t, sin_t, max_pos, positions,  \
        (bf16_t*)kc, (bf16_t*)vc, P, num_pages, slots, (int)qk_blocks)))
        switch (lph) {
            case 1: QKV_CASE(1); break;
            case 2: QKV_CASE(2); break;
            case 4: QKV_CASE(4); break;
            case 8: QKV_CASE(8); break;
            default: QKV_CASE(16); break;
        }
#undef QKV_CASE
        SPY_CHECK_LAUNCH("spy_qknorm_rope_store");
        return 0;
    }
    const dim3 grid(T, (n_q + 2 * n_kv + QK_WAVES - 1) / QK_WAVES);
    SPY_DISPATCH(dtype, TA, SPY_DISPATCH(wd, TW, (qknorm_rope_store_kernel<TA, TW><<<grid, QK_WAVES * 64, 0, st>>>(
        (const TA*)qkv, (TA*)q_out, n_q, n_kv, d, (const TW*)qw, (const TW*)kw, eps, cos_t, sin_t, rot, max_pos, positions,
        (TA*)kc, (TA*)vc, P, num_pages, slots))));
    SPY_CHECK_LAUNCH("spy_qknorm_rope_store");
    return 0;
}
