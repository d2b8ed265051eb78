// Elementwise glue between the linears of a decoder layer, and the on-device synthetic operand generator.
// Role of the reference's norm_resid (assets/norm.cu:4-48: RMS normalisation emitting an f16 copy for the next GEMV)
// and ew (assets/ew.cu:9-32: silu(gate) * up emitting f16), reduced to what a chain of linears needs.
#include "w4a16_common.hpp"

// f32 -> f16 of a value that must first exist as a rounded f32: the empty asm keeps the compiler from folding the
// producing multiply into a mixed-precision instruction that rounds the exact product straight to f16.
__device__ __forceinline__ _Float16 glue_round_f16(float v) {
    asm volatile("" : "+v"(v));
    return (_Float16)v;
}

// out[r][c] = f16(v[r][c] * inv),  inv = f32(1 / sqrt(mean_c(v[r][c]^2) + 1e-6)).
// The sum of squares has a fixed order so that a CPU restatement is bit-identical: thread i adds the (exact) f64
// squares of columns i, i+256, ... in order; the 256 partials are folded pairwise at strides 128, 64, ..., 1.
// One workgroup of 256 threads per row; v rows are ld floats apart (a column slice of a wider matrix is allowed).
extern "C" __global__ __launch_bounds__(256) void w4a16_rms_rescale_f16(const float* __restrict__ v, int ld, int ncols,
                                                                       uint16_t* __restrict__ out) {
    __shared__ double red[256];
    const int tid = threadIdx.x;
    const float* row = v + (size_t)blockIdx.x * ld;
    double ss = 0.0;
    for (int c = tid; c < ncols; c += 256) {
        const double d = (double)row[c];
        ss = ss + d * d;
    }
    red[tid] = ss;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) {
        if (tid < st) red[tid] = red[tid] + red[tid + st];
        __syncthreads();
    }
    const float inv = (float)(1.0 / sqrt(red[0] / (double)ncols + 1e-6));
    _Float16* o = reinterpret_cast<_Float16*>(out) + (size_t)blockIdx.x * ncols;
    for (int c = tid; c < ncols; c += 256) o[c] = glue_round_f16(row[c] * inv);
}

// out[r][c] = f16((g / (1 + exp(-g))) * u),  g = gu[r][c], u = gu[r][n_ff + c], all in f32 (assets/ew.cu:19-30).
extern "C" __global__ __launch_bounds__(256) void w4a16_silu_mul_f16(const float* __restrict__ gu, int n_ff, int t,
                                                                    uint16_t* __restrict__ out) {
    const size_t total = (size_t)t * n_ff;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / n_ff, c = i % n_ff;
        const float g = gu[r * 2 * n_ff + c], u = gu[r * 2 * n_ff + n_ff + c];
        const float e = expf(-g);
        reinterpret_cast<_Float16*>(out)[i] = glue_round_f16((g / (1.0f + e)) * u);
    }
}

// ---- synthetic operands on the device: the SplitMix64 streams of the reference's parity gate
// (crates/server/src/probes/w4a16/gates.rs:182-196); output i of stream `seed` is mix(seed + (i+1)*GAMMA).
__device__ __forceinline__ unsigned long long w4_splitmix(unsigned long long seed, unsigned long long i) {
    unsigned long long z = seed + (i + 1ull) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

// q[i] = low 32 bits of output i: eight independent uniform nibbles per word.
extern "C" __global__ __launch_bounds__(256) void w4a16_synth_q(uint32_t* __restrict__ q, unsigned long long words,
                                                               unsigned long long seed) {
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < words;
         i += (unsigned long long)gridDim.x * blockDim.x)
        q[i] = (uint32_t)w4_splitmix(seed, i);
}

// s[i] = f16(lo + span * u), u = (output i >> 40) / 2^24, multiply and add rounded separately in f32.
extern "C" __global__ __launch_bounds__(256) void w4a16_synth_s(uint16_t* __restrict__ s, unsigned long long count,
                                                               unsigned long long seed, float lo, float span) {
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < count;
         i += (unsigned long long)gridDim.x * blockDim.x) {
        const float u = (float)(w4_splitmix(seed, i) >> 40) / 16777216.0f;
        const float m = span * u;
        reinterpret_cast<_Float16*>(s)[i] = glue_round_f16(lo + m);
    }
}
