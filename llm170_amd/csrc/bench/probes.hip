// Measurement probes of the benchmark, not part of the product's asset manifest: bench.py loads this code object by
// itself through w4a16_module_load.  A plain 16-byte copy of known size that calibrates the profiler's FETCH_SIZE /
// WRITE_SIZE counters, and two probes of what the chip sustains: a read-only stream and a matrix-instruction loop.
#include "w4a16_common.hpp"

// dst[i] = src[i] for n16 16-byte elements; reads n16*16 bytes and writes n16*16 bytes exactly once.
extern "C" __global__ __launch_bounds__(256) void w4a16_copy_u4(const u4_t* __restrict__ src, u4_t* __restrict__ dst,
                                                                size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
        __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// Plain streaming read of n16 16-byte elements (nothing else happens): the rate this reaches on a buffer of a
// linear's size is what the memory system gives a kernel that only fetches.  The loads are kept alive by a store that
// no zero-filled buffer triggers.
extern "C" __global__ __launch_bounds__(256) void w4a16_read_u4(const u4_t* __restrict__ src, size_t n16,
                                                                unsigned* __restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    u4_t a = {0u, 0u, 0u, 0u};
    for (; i + 3 * stride < n16; i += 4 * stride) {
        const u4_t v0 = __builtin_nontemporal_load(src + i);
        const u4_t v1 = __builtin_nontemporal_load(src + i + stride);
        const u4_t v2 = __builtin_nontemporal_load(src + i + 2 * stride);
        const u4_t v3 = __builtin_nontemporal_load(src + i + 3 * stride);
        a ^= v0 ^ v1 ^ v2 ^ v3;
    }
    for (; i < n16; i += stride) a ^= __builtin_nontemporal_load(src + i);
    const unsigned r = a.x ^ a.y ^ a.z ^ a.w;
    if (r == 0x9E3779B9u) sink[0] = r;
}

// Back-to-back v_mfma_f32_32x32x16_f16 on four independent accumulators per wave and nothing else: the matrix rate
// the chip sustains at the clock it settles to under that load.  2 * 32*32*16 flops per instruction per wave;
// flops per launch = gridDim.x * 4 waves * iters * 4 * 32768.  Operands are lane-dependent values in [-1, 1).
extern "C" __global__ __launch_bounds__(256) void w4a16_mfma_peak_f16(float* __restrict__ sink, int iters) {
    h8_t a, b;
    unsigned z = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
    for (int j = 0; j < 8; ++j) {
        z = z * 1664525u + 1013904223u;
        a[j] = (_Float16)((float)(int)(z >> 20 & 0xFFF) * (1.0f / 2048.0f) - 1.0f);
        z = z * 1664525u + 1013904223u;
        b[j] = (_Float16)((float)(int)(z >> 20 & 0xFFF) * (1.0f / 2048.0f) - 1.0f);
    }
    f16_t c0 = {}, c1 = {}, c2 = {}, c3 = {};
    for (int it = 0; it < iters; ++it) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(b, a, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, a, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(b, b, c3, 0, 0, 0);
    }
    float s = 0.0f;
    for (int j = 0; j < 16; ++j) s += c0[j] + c1[j] + c2[j] + c3[j];
    if (s == 12345.678f) sink[0] = s;
}
