// Bit-exact device twin of the reference CPU contract dot_row_w4a16_lane_group
// (crates/core/src/quant/lane.rs:2-70): one 64-lane wavefront per output row, lane l walks elements
// l, l+64, l+128, ... with an f32 multiply followed by a separate f32 add (never fused), the 64 partials are widened
// to f64 and folded 32,16,8,4,2,1 exactly as tree64, and the f64 total is rounded once to f32.
// Role of the reference kernel w4a16_gemm_g128 / _g32_bf16 (assets/gptq4.cu:825-951): the gate every fast kernel
// is measured against, and the on-device oracle where the CPU is too slow.  Reads the operand format as given
// (q u32 [n][k/8], s u16 [n][k/group], x f16 [t][k]); out f32 [t][n].
#include "w4a16_common.hpp"

#define LANE_TT 8  // tokens sharing one pass over a row's weights

template <int G, bool SBF>
__device__ __forceinline__ void lane_body(const uint32_t* __restrict__ q, const uint16_t* __restrict__ s,
                                          const uint16_t* __restrict__ x, float* __restrict__ out, int n, int k,
                                          int t) {
    const int lane = threadIdx.x & 63;
    const int o = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int t0 = blockIdx.y * LANE_TT;
    if (o >= n) return;  // whole wave leaves together
    const uint32_t* qrow = q + (size_t)o * (k >> 3);
    const uint16_t* srow = s + (size_t)o * (k / G);
    float acc[LANE_TT];
#pragma unroll
    for (int j = 0; j < LANE_TT; j++) acc[j] = 0.0f;
    for (int i = lane; i < k; i += 64) {
        const int nib = (int)((qrow[i >> 3] >> (4 * (i & 7))) & 0xFu);
        const float sc = w4_scale_to_f32<SBF>(srow[i / G]);
        const float w = __fmul_rn((float)(nib - 8), sc);
#pragma unroll
        for (int j = 0; j < LANE_TT; j++) {
            if (t0 + j < t) {
                const float xv = w4_half_bits_to_f32(x[(size_t)(t0 + j) * k + i]);
                acc[j] = __fadd_rn(acc[j], __fmul_rn(w, xv));
            }
        }
    }
#pragma unroll
    for (int j = 0; j < LANE_TT; j++) {
        if (t0 + j < t) {
            double v = (double)acc[j];
            v = __dadd_rn(v, __shfl_down(v, 32, 64));
            v = __dadd_rn(v, __shfl_down(v, 16, 64));
            v = __dadd_rn(v, __shfl_down(v, 8, 64));
            v = __dadd_rn(v, __shfl_down(v, 4, 64));
            v = __dadd_rn(v, __shfl_down(v, 2, 64));
            v = __dadd_rn(v, __shfl_down(v, 1, 64));
            if (lane == 0) out[(size_t)(t0 + j) * n + o] = (float)v;
        }
    }
}

#define LANE_KERNEL(NAME, G, SBF)                                                                                  \
    extern "C" __global__ __launch_bounds__(256) void NAME(const uint32_t* q, const uint16_t* s, const uint16_t* x, \
                                                           float* out, int n, int k, int t) {                       \
        lane_body<G, SBF>(q, s, x, out, n, k, t);                                                                   \
    }

LANE_KERNEL(w4a16_lane_g128_f16, 128, false)
LANE_KERNEL(w4a16_lane_g128_bf16, 128, true)
LANE_KERNEL(w4a16_lane_g32_f16, 32, false)
LANE_KERNEL(w4a16_lane_g32_bf16, 32, true)
