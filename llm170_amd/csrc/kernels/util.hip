// Small service kernels: zero fill (used instead of a memset node so the library stays safe to capture in a HIP
// graph), and a plain 16-byte copy of known size that calibrates the profiler's FETCH_SIZE / WRITE_SIZE counters.
#include "w4a16_common.hpp"

// dst must be 4-byte aligned; n_words 32-bit words are cleared.
extern "C" __global__ __launch_bounds__(256) void w4a16_fill0_u32(uint32_t* __restrict__ dst, size_t n_words) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += stride) dst[i] = 0u;
}

// dst[i] = src[i] for n16 16-byte elements; reads n16*16 bytes and writes n16*16 bytes exactly once.
extern "C" __global__ __launch_bounds__(256) void w4a16_copy_u4(const u4_t* __restrict__ src, u4_t* __restrict__ dst,
                                                                size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
        __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}
