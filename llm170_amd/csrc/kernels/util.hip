// Small service kernel: zero fill, used instead of a memset node so that the library stays safe to capture in a HIP
// graph.
#include "w4a16_common.hpp"

// dst must be 4-byte aligned; n_words 32-bit words are cleared.
extern "C" __global__ __launch_bounds__(256) void w4a16_fill0_u32(uint32_t* __restrict__ dst, size_t n_words) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += stride) dst[i] = 0u;
}
