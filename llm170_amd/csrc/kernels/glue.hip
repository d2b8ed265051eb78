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
// The sum of squares has a fixed order so that a CPU restatement is bit-identical: partial i (i < 1024) adds the
// (exact) f64 squares of columns i, i+1024, ... in order; the 1024 partials are folded pairwise at strides 512, 256,
// ..., 1.  One workgroup of 1024 threads per row; every thread has its few loads in flight at once.  v rows are ld
// floats apart (a column slice of a wider matrix is allowed).
#define RMS_LANES 1024
#define RMS_UNROLL 8
extern "C" __global__ __launch_bounds__(RMS_LANES) void w4a16_rms_rescale_f16(const float* __restrict__ v, int ld,
                                                                             int ncols, uint16_t* __restrict__ out) {
    __shared__ double red[RMS_LANES];
    const int tid = threadIdx.x;
    const float* row = v + (size_t)blockIdx.x * ld;
    double ss = 0.0;
    float first[RMS_UNROLL];  // the row's first RMS_LANES * RMS_UNROLL columns stay in registers for the second pass
    for (int c0 = tid; c0 < ncols; c0 += RMS_LANES * RMS_UNROLL) {
        float x[RMS_UNROLL];
#pragma unroll
        for (int j = 0; j < RMS_UNROLL; j++) {
            const int c = c0 + j * RMS_LANES;
            x[j] = c < ncols ? row[c] : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < RMS_UNROLL; j++) {
            const double d = (double)x[j];
            ss = ss + d * d;  // a zero past the row end adds +0.0 and changes nothing
            if (c0 == tid) first[j] = x[j];
        }
    }
    red[tid] = ss;
    __syncthreads();
    for (int st = RMS_LANES / 2; st >= 64; st >>= 1) {
        if (tid < st) red[tid] = red[tid] + red[tid + st];
        __syncthreads();
    }
    // the last 64 partials are folded inside wave 0 with the same pairing (strides 32, 16, ..., 1)
    double r = red[tid & 63];
#pragma unroll
    for (int st = 32; st > 0; st >>= 1) r = r + __shfl_down(r, st);
    r = __shfl(r, 0);
    const float inv = (float)(1.0 / sqrt(r / (double)ncols + 1e-6));
    _Float16* o = reinterpret_cast<_Float16*>(out) + (size_t)blockIdx.x * ncols;
#pragma unroll
    for (int j = 0; j < RMS_UNROLL; j++) {
        const int c = tid + j * RMS_LANES;
        if (c < ncols) o[c] = glue_round_f16(first[j] * inv);
    }
    for (int c = tid + RMS_LANES * RMS_UNROLL; c < ncols; c += RMS_LANES) o[c] = glue_round_f16(row[c] * inv);
}

// RMS normalisation with residual add, the producer of the f16 A operand of a layer's first linear
// (assets/norm.cu:4-48 norm_resid and :97-148 norm_resid_g, one kernel here).  Per token row r, with v = x + ab:
//   x <- v;  xn = v * inv * nw[w_off + c],  inv = 1 / sqrtf(sum(v^2) / hidden + 1e-6f);
//   xn32 (optional) = xn rounded to f16 and widened back;  xn16 (optional) = the f16 bits.
// The f32 arithmetic is the reference's, in its order, so results agree bit for bit with a CPU restatement: thread tid
// of 1024 adds its columns tid, tid + 1024, ... with one fused multiply-add each (that kernel file is built with
// nvcc's default -fmad=true, scripts/build_cuda_kernels.sh:67), the 1024 partials are folded pairwise at strides 512,
// 256, ..., 1, the division and square root are correctly rounded, and v * inv * nw is two roundings.  hidden <= 8192.
extern "C" __global__ __launch_bounds__(1024) void w4a16_norm_resid(float* __restrict__ x, const float* __restrict__ nw,
                                                                    const float* __restrict__ ab, float* __restrict__ xn,
                                                                    float* __restrict__ xn32, uint16_t* __restrict__ xn16,
                                                                    int w_off, int hidden) {
    __shared__ float red[1024];
    const int tid = threadIdx.x;
    const size_t base = (size_t)blockIdx.x * hidden;
    float v[8];
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int c = j * 1024 + tid;
        v[j] = 0.0f;
        if (c < hidden) {
            v[j] = x[base + c] + ab[base + c];
            ss = __builtin_fmaf(v[j], v[j], ss);
        }
    }
    red[tid] = ss;
    __syncthreads();
    for (int st = 512; st >= 64; st >>= 1) {
        if (tid < st) red[tid] = red[tid] + red[tid + st];
        __syncthreads();
    }
    float r = red[tid & 63];  // strides 32..1 inside every wave, same pairing; lane 0 ends with the row's sum
#pragma unroll
    for (int st = 32; st > 0; st >>= 1) r = r + __shfl_down(r, st);
    r = __shfl(r, 0);
    const float inv = 1.0f / sqrtf(r / (float)hidden + 1e-6f);
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int c = j * 1024 + tid;
        if (c >= hidden) continue;
        float y = v[j] * inv;
        asm volatile("" : "+v"(y));  // two roundings, never one fused product
        y = y * nw[w_off + c];
        xn[base + c] = y;
        if (xn32 || xn16) {
            const _Float16 h = glue_round_f16(y);
            if (xn32) xn32[base + c] = (float)h;
            if (xn16) xn16[base + c] = __builtin_bit_cast(uint16_t, h);
        }
        x[base + c] = v[j];
    }
}

// out[r][c] = f16((g / (1 + exp(-g))) * u),  g = gu[r][c], u = gu[r][n_ff + c], all in f32 (assets/ew.cu:19-30).
// Four columns per thread when n_ff % 4 == 0.
extern "C" __global__ __launch_bounds__(256) void w4a16_silu_mul_f16(const float* __restrict__ gu, int n_ff, int t,
                                                                    uint16_t* __restrict__ out, int act_kind) {
    if ((n_ff & 3) == 0) {
        const size_t total = (size_t)t * n_ff / 4;
        for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
            const size_t r = (i * 4) / n_ff, c = (i * 4) % n_ff;
            const f4_t g = *reinterpret_cast<const f4_t*>(gu + r * 2 * n_ff + c);
            const f4_t u = *reinterpret_cast<const f4_t*>(gu + r * 2 * n_ff + n_ff + c);
            h4_t o;
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = glue_round_f16(w4_act_mul(g[j], u[j], act_kind));
            *reinterpret_cast<h4_t*>(reinterpret_cast<_Float16*>(out) + i * 4) = o;
        }
        return;
    }
    const size_t total = (size_t)t * n_ff;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / n_ff, c = i % n_ff;
        const float g = gu[r * 2 * n_ff + c], u = gu[r * 2 * n_ff + n_ff + c];
        reinterpret_cast<_Float16*>(out)[i] = glue_round_f16(w4_act_mul(g, u, act_kind));
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
