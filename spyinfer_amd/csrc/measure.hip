// A plain read of device memory, for measurements: what a kernel that does nothing but stream gets from this GPU's
// memory.  bench.py quotes its decode step against this rate beside the published one.  (The reference times its own
// kernels the same way, test/performance/test_linear_kernel.cu:58-106.)  Not used by the engine.
#include "common.h"

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

// Every block walks its own contiguous part of the buffer with 16-byte loads that are not kept in the caches, four in
// flight per lane; the sums go out so that nothing can be dropped.
__global__ __launch_bounds__(256) void read_kernel(const u32x4_t* __restrict__ p, size_t n16, uint32_t* __restrict__ sink) {
    const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t lo = (size_t)blockIdx.x * per, hi = lo + per < n16 ? lo + per : n16;
    u32x4_t a = {0, 0, 0, 0};
    size_t i = lo + threadIdx.x;
    for (; i + 3 * 256 < hi; i += 4 * 256) {
        const u32x4_t v0 = __builtin_nontemporal_load(p + i), v1 = __builtin_nontemporal_load(p + i + 256);
        const u32x4_t v2 = __builtin_nontemporal_load(p + i + 512), v3 = __builtin_nontemporal_load(p + i + 768);
        a ^= v0 ^ v1 ^ v2 ^ v3;
    }
    for (; i < hi; i += 256) a ^= __builtin_nontemporal_load(p + i);
    const uint32_t x = a[0] ^ a[1] ^ a[2] ^ a[3];
    if (x == 0x9e3779b9u) sink[blockIdx.x * 256 + threadIdx.x] = x;      // (practically never: the store keeps the loads alive)
}

// Reads `bytes` bytes from `buf` (16-byte aligned, a multiple of 16) once with `blocks` blocks of 256 threads.
// `sink`: blocks * 256 uint32 that the kernel may write.
extern "C" int spy_measure_read(const void* buf, int64_t bytes, int blocks, void* sink, hipStream_t st) {
    SPY_REQUIRE(buf && sink && bytes > 0 && bytes % 16 == 0 && ((uintptr_t)buf % 16) == 0, "spy_measure_read: a 16-byte aligned buffer of a multiple of 16 bytes expected");
    SPY_REQUIRE(blocks > 0 && blocks <= 65536, "spy_measure_read: 1..65536 blocks");
    read_kernel<<<blocks, 256, 0, st>>>((const u32x4_t*)buf, (size_t)(bytes / 16), (uint32_t*)sink);
    SPY_CHECK_LAUNCH("spy_measure_read");
    return 0;
}
