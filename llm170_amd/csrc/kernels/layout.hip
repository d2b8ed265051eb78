// Upload-time re-layout of W4A16 operands into the tiled form the streaming and MFMA kernels read, its inverse,
// and dequantised dumps.  Counterpart of the reference's host-side repack before upload
// (crates/core/src/marlin.rs:2-67 via w4a16_dec/upload.rs:99-179); the layout itself is this library's own and is
// described in w4a16_common.hpp.
#include "w4a16_common.hpp"

// One thread per tiled dword.  n_pad = 16 * row_blocks >= n; rows >= n are filled with nibble 8 (weight 0).
extern "C" __global__ __launch_bounds__(256) void w4a16_tile_q(const uint32_t* __restrict__ q,
                                                               uint32_t* __restrict__ qt, int n, int k,
                                                               int row_blocks) {
    const int kt_n = k / W4_TILE_K;
    const size_t total = (size_t)row_blocks * kt_n * 256;
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int w = id & 3, l = (id >> 2) & 63;
    const size_t tile = id >> 8;
    const int kt = tile % kt_n, nb = tile / kt_n;
    const int r = l & 15, g = l >> 4;
    const int row = nb * 16 + r;
    uint32_t d = 0x88888888u;
    if (row < n) {
        const uint32_t src = q[(size_t)row * (k >> 3) + ((kt * W4_TILE_K + w * 32 + g * 8) >> 3)];
        d = 0;
#pragma unroll
        for (int p = 0; p < 8; p++) d |= ((src >> (4 * w4_perm(p))) & 0xFu) << (4 * p);
    }
    qt[id] = d;
}

// One thread per tiled scale: st[(nb*kg_n + kg)*16 + r] = s[(nb*16 + r)*kg_n + kg] (0 for padded rows).
extern "C" __global__ __launch_bounds__(256) void w4a16_tile_s(const uint16_t* __restrict__ s,
                                                               uint16_t* __restrict__ st, int n, int kg_n,
                                                               int row_blocks) {
    const size_t total = (size_t)row_blocks * kg_n * 16;
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int r = id & 15;
    const size_t rest = id >> 4;
    const int kg = rest % kg_n, nb = rest / kg_n;
    const int row = nb * 16 + r;
    st[id] = row < n ? s[(size_t)row * kg_n + kg] : (uint16_t)0;
}

// Inverse of w4a16_tile_q: one thread per operand-format word q[row][kw].
extern "C" __global__ __launch_bounds__(256) void w4a16_untile_q(const uint32_t* __restrict__ qt,
                                                                 uint32_t* __restrict__ q, int n, int k) {
    const int kw_n = k >> 3, kt_n = k / W4_TILE_K;
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (size_t)n * kw_n) return;
    const int kw = id % kw_n, row = id / kw_n;
    const int k0 = kw * 8, kt = k0 / W4_TILE_K, within = k0 % W4_TILE_K;
    const int w = within / 32, g = (within % 32) / 8;
    const int nb = row / 16, r = row % 16;
    const uint32_t d = qt[(((size_t)nb * kt_n + kt) * 64 + g * 16 + r) * 4 + w];
    uint32_t o = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) o |= ((d >> (4 * w4_pos(j))) & 0xFu) << (4 * j);
    q[id] = o;
}

extern "C" __global__ __launch_bounds__(256) void w4a16_untile_s(const uint16_t* __restrict__ st,
                                                                 uint16_t* __restrict__ s, int n, int kg_n) {
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (size_t)n * kg_n) return;
    const int kg = id % kg_n, row = id / kg_n;
    s[id] = st[((size_t)(row / 16) * kg_n + kg) * 16 + (row % 16)];
}

// Dequantised weights from the tiled copy, through the same w4_deq8 the fast kernels use:
// out[row][k] = (float)(nibble - 8) * scale, one thread per tiled dword (8 outputs).
template <bool SBF>
__device__ __forceinline__ void dump_tiled_body(const uint32_t* __restrict__ qt, const uint16_t* __restrict__ st,
                                                float* __restrict__ out, int n, int k, int group, int row_blocks) {
    const int kt_n = k / W4_TILE_K, kg_n = k / group;
    const size_t total = (size_t)row_blocks * kt_n * 256;
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int w = id & 3, l = (id >> 2) & 63;
    const size_t tile = id >> 8;
    const int kt = tile % kt_n, nb = tile / kt_n;
    const int r = l & 15, g = l >> 4;
    const int row = nb * 16 + r;
    if (row >= n) return;
    const int k0 = kt * W4_TILE_K + w * 32 + g * 8;
    const float sc = w4_scale_to_f32<SBF>(st[((size_t)nb * kg_n + k0 / group) * 16 + r]);
    const h8_t v = w4_deq8(qt[id]);
#pragma unroll
    for (int j = 0; j < 8; j++) out[(size_t)row * k + k0 + j] = __fmul_rn((float)v[j], sc);
}

extern "C" __global__ __launch_bounds__(256) void w4a16_dump_tiled_f16(const uint32_t* qt, const uint16_t* st,
                                                                       float* out, int n, int k, int group,
                                                                       int row_blocks) {
    dump_tiled_body<false>(qt, st, out, n, k, group, row_blocks);
}
extern "C" __global__ __launch_bounds__(256) void w4a16_dump_tiled_bf16(const uint32_t* qt, const uint16_t* st,
                                                                        float* out, int n, int k, int group,
                                                                        int row_blocks) {
    dump_tiled_body<true>(qt, st, out, n, k, group, row_blocks);
}

// Dequantised weights from the operand format as given: one thread per word (8 outputs).
template <bool SBF>
__device__ __forceinline__ void dump_raw_body(const uint32_t* __restrict__ q, const uint16_t* __restrict__ s,
                                              float* __restrict__ out, int n, int k, int group) {
    const int kw_n = k >> 3;
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (size_t)n * kw_n) return;
    const int kw = id % kw_n, row = id / kw_n;
    const float sc = w4_scale_to_f32<SBF>(s[(size_t)row * (k / group) + (kw * 8) / group]);
    const uint32_t d = q[id];
#pragma unroll
    for (int j = 0; j < 8; j++) out[(size_t)row * k + kw * 8 + j] = __fmul_rn((float)((int)((d >> (4 * j)) & 0xFu) - 8), sc);
}

extern "C" __global__ __launch_bounds__(256) void w4a16_dump_raw_f16(const uint32_t* q, const uint16_t* s,
                                                                     float* out, int n, int k, int group) {
    dump_raw_body<false>(q, s, out, n, k, group);
}
extern "C" __global__ __launch_bounds__(256) void w4a16_dump_raw_bf16(const uint32_t* q, const uint16_t* s,
                                                                      float* out, int n, int k, int group) {
    dump_raw_body<true>(q, s, out, n, k, group);
}

// Largest row norm of the dequantised weights, max over rows of sqrt(sum_k ((nib - 8) * scale)^2): with an input of
// unit root mean square over k columns no output element exceeds it times sqrt(k) (Cauchy-Schwarz), which sizes the
// power-of-two factor of an f16 hand-over.  One wave per row block of the tiled copy; lanes of a row add their shares,
// the 16 rows take the maximum, and the waves join through an integer maximum on the bits of the non-negative f32
// (unsigned order = float order; a maximum does not depend on the order of its operands).  *out starts at zero.
template <bool SBF>
__device__ __forceinline__ void row_norm_body(const u4_t* __restrict__ qt, const uint16_t* __restrict__ st,
                                              unsigned* __restrict__ out, int row_blocks, int kt_n, int group) {
    const int wave = (int)(((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6), lane = threadIdx.x & 63;
    if (wave >= row_blocks) return;
    const int r = lane & 15, gpt = W4_TILE_K / group, kg_n = kt_n * gpt;
    float ss = 0.f;
    for (int kt = 0; kt < kt_n; kt++) {
        const u4_t d = qt[((size_t)wave * kt_n + kt) * 64 + lane];
#pragma unroll
        for (int w = 0; w < 4; w++) {
            int isum = 0;
#pragma unroll
            for (int p = 0; p < 8; p++) {
                const int v = (int)((d[w] >> (4 * p)) & 0xFu) - 8;
                isum += v * v;
            }
            const float sc = w4_scale_to_f32<SBF>(st[((size_t)wave * kg_n + kt * gpt + (w * 32) / group) * 16 + r]);
            ss += (float)isum * (sc * sc);
        }
    }
    ss += __shfl_xor(ss, 16);
    ss += __shfl_xor(ss, 32);
    float nrm = sqrtf(ss);
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) nrm = fmaxf(nrm, __shfl_xor(nrm, off));
    if (lane == 0) atomicMax(out, __builtin_bit_cast(unsigned, nrm));
}
extern "C" __global__ __launch_bounds__(256) void w4a16_row_norm_max_f16(const u4_t* qt, const uint16_t* st, unsigned* out,
                                                                         int row_blocks, int kt_n, int group) {
    row_norm_body<false>(qt, st, out, row_blocks, kt_n, group);
}
extern "C" __global__ __launch_bounds__(256) void w4a16_row_norm_max_bf16(const u4_t* qt, const uint16_t* st, unsigned* out,
                                                                          int row_blocks, int kt_n, int group) {
    row_norm_body<true>(qt, st, out, row_blocks, kt_n, group);
}
