// Shared helpers of the gfx950 kernel library: dtype codes, error reporting, bf16 <-> f32,
// wave and block reductions.  Wavefronts are 64 lanes wide.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#define SPY_F32 0
#define SPY_BF16 1
#define SPY_WAVE 64

typedef uint16_t bf16_t;

extern "C" const char* spy_last_error();
int spy_fail(const char* fmt, ...);   // records the message, returns 1

#define SPY_REQUIRE(cond, ...)              \
    do {                                    \
        if (!(cond)) return spy_fail(__VA_ARGS__); \
    } while (0)

#define SPY_CHECK_LAUNCH(name)                                                        \
    do {                                                                              \
        hipError_t e_ = hipGetLastError();                                            \
        if (e_ != hipSuccess) return spy_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); \
    } while (0)

__device__ __forceinline__ float bf16_to_f32(bf16_t x) { return __uint_as_float(((uint32_t)x) << 16); }

// round to nearest, ties to even; NaN stays NaN.  gfx950 converts in hardware (v_cvt_pk_bf16_f32).
__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return __builtin_bit_cast(unsigned short, (__bf16)f); }

// two values in one instruction: a in the low half, b in the high half
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    typedef float f32x2_ __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_ __attribute__((ext_vector_type(2)));
    const f32x2_ v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_));
}

template <typename T> __device__ __forceinline__ float to_f32(T x);
template <> __device__ __forceinline__ float to_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t x) { return bf16_to_f32(x); }

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return f32_to_bf16(x); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Block-wide sum; `red` is shared memory of at least blockDim.x / 64 floats.  Every thread gets the result.
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
    return t;
}

// Dispatch on a dtype code: binds `T` in `body`.
#define SPY_DISPATCH(code, T, ...)                  \
    if ((code) == SPY_F32) { typedef float T; __VA_ARGS__; } \
    else { typedef bf16_t T; __VA_ARGS__; }
