// Decode regime (t = 1..16 activation rows): HBM-streaming skinny GEMM  y[t][n] = x[t][k] * W^T.
// Role of the reference's gemv_t / split-K decode kernels (assets/gptq4.cu:522-553, assets/decode.cu:46-267),
// designed for CDNA4 instead:
//   * weights are read once, as 1 KiB tiles (64 lanes x global_load_dwordx4, non-temporal) of the tiled layout in
//     w4a16_common.hpp — every wave-level load is one fully used contiguous KiB;
//   * the int4 -> f16 unpack is 9 VALU ops per 8 weights and stays in registers; the multiply-accumulate runs on
//     the matrix core: dword w of the 64 lanes is the A operand of v_mfma_f32_16x16x32_f16 (16 rows x 32 k), the
//     B operand is x (32 k x 16 token columns, columns >= t are zero), so t = 1 and t = 16 cost the same;
//   * weights enter the MFMA as exact integers; the per-group scale multiplies the f32 group sum, so no weight is
//     ever rounded to f16 (error vs the f32 lane contract is summation order only);
//   * split-K lives inside the workgroup: the W waves of a block take consecutive k-tile slices of the same RB row
//     blocks and wave 0 folds the partial tiles through LDS in fixed order (deterministic, no atomics, no second
//     launch).  The host picks RB and W so that a wave streams about 8 KiB.
#include "w4a16_common.hpp"

template <int G, bool SBF, int RB>
__device__ __forceinline__ void decode_body(const u4_t* __restrict__ qt, const uint16_t* __restrict__ st,
                                            const uint16_t* __restrict__ x, void* __restrict__ y, int row_blocks,
                                            int k, int n, int t, int out_f16) {
    extern __shared__ f4_t red[];  // [W][RB][64]
    constexpr int GPT = W4_TILE_K / G;  // scale groups per k tile
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, W = blockDim.x >> 6;
    const int kt_n = k / W4_TILE_K;
    const int kg_n = kt_n * GPT;
    const int nb0 = blockIdx.x * RB;
    const int kt0 = (kt_n * wave) / W, kt1 = (kt_n * (wave + 1)) / W;
    const int m = lane & 15, g = lane >> 4;
    const bool xact = m < t;
    const uint16_t* xp = x + (size_t)(xact ? m : 0) * k + g * 8;

    f4_t acc[RB];
    const u4_t* qp[RB];
    const uint16_t* sp[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        acc[rb] = (f4_t){0.f, 0.f, 0.f, 0.f};
        const int nb = min(nb0 + rb, row_blocks - 1);  // a tail block re-reads the last row block, never stores it
        qp[rb] = qt + (size_t)nb * kt_n * 64 + lane;
        sp[rb] = st + (size_t)nb * kg_n * 16 + 4 * g;
    }

#pragma unroll 2
    for (int kt = kt0; kt < kt1; ++kt) {
        u4_t qv[RB];
        u2_t sv[RB][GPT];
        h8_t xb[4];
#pragma unroll
        for (int rb = 0; rb < RB; rb++) qv[rb] = __builtin_nontemporal_load(qp[rb] + (size_t)kt * 64);
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int gi = 0; gi < GPT; gi++)
                sv[rb][gi] = *reinterpret_cast<const u2_t*>(sp[rb] + ((size_t)kt * GPT + gi) * 16);
#pragma unroll
        for (int w = 0; w < 4; w++) {
            xb[w] = (h8_t){0, 0, 0, 0, 0, 0, 0, 0};
            if (xact) xb[w] = *reinterpret_cast<const h8_t*>(xp + kt * W4_TILE_K + w * 32);
        }
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            if (G == 128) {
                f4_t part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int w = 0; w < 4; w++)
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(qv[rb][w]), xb[w], part, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; i++)
                    acc[rb][i] += w4_scale_fast<SBF>((sv[rb][0][i >> 1] >> (16 * (i & 1))) & 0xFFFFu) * part[i];
            } else {
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    f4_t part = {0.f, 0.f, 0.f, 0.f};
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(qv[rb][w]), xb[w], part, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        acc[rb][i] +=
                            w4_scale_fast<SBF>((sv[rb][w % GPT][i >> 1] >> (16 * (i & 1))) & 0xFFFFu) * part[i];
                }
            }
        }
    }

    if (W > 1) {
        if (wave != 0) {
#pragma unroll
            for (int rb = 0; rb < RB; rb++) red[(wave * RB + rb) * 64 + lane] = acc[rb];
        }
        __syncthreads();
        if (wave != 0) return;
        for (int w = 1; w < W; w++) {
#pragma unroll
            for (int rb = 0; rb < RB; rb++) acc[rb] += red[(w * RB + rb) * 64 + lane];
        }
    }
    if (!xact) return;
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        if (nb0 + rb >= row_blocks) break;
        const int row = (nb0 + rb) * 16 + 4 * g;
        if (out_f16) {
            _Float16* yo = reinterpret_cast<_Float16*>(y) + (size_t)m * n + row;
            if (row + 3 < n) {
                h4_t v = {(_Float16)acc[rb][0], (_Float16)acc[rb][1], (_Float16)acc[rb][2], (_Float16)acc[rb][3]};
                *reinterpret_cast<h4_t*>(yo) = v;
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (row + i < n) yo[i] = (_Float16)acc[rb][i];
            }
        } else {
            float* yo = reinterpret_cast<float*>(y) + (size_t)m * n + row;
            if (row + 3 < n) {
                *reinterpret_cast<f4_t*>(yo) = acc[rb];
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (row + i < n) yo[i] = acc[rb][i];
            }
        }
    }
}

#define DECODE_KERNEL(NAME, G, SBF, RB)                                                                     \
    extern "C" __global__ __launch_bounds__(1024) void NAME(const u4_t* qt, const uint16_t* st,             \
                                                            const uint16_t* x, void* y, int row_blocks, int k, \
                                                            int n, int t, int out_f16) {                    \
        decode_body<G, SBF, RB>(qt, st, x, y, row_blocks, k, n, t, out_f16);                                \
    }

DECODE_KERNEL(w4a16_decode_g128_f16_rb1, 128, false, 1)
DECODE_KERNEL(w4a16_decode_g128_f16_rb2, 128, false, 2)
DECODE_KERNEL(w4a16_decode_g128_f16_rb4, 128, false, 4)
DECODE_KERNEL(w4a16_decode_g32_f16_rb1, 32, false, 1)
DECODE_KERNEL(w4a16_decode_g32_f16_rb2, 32, false, 2)
DECODE_KERNEL(w4a16_decode_g32_f16_rb4, 32, false, 4)
DECODE_KERNEL(w4a16_decode_g128_bf16_rb1, 128, true, 1)
DECODE_KERNEL(w4a16_decode_g128_bf16_rb2, 128, true, 2)
DECODE_KERNEL(w4a16_decode_g128_bf16_rb4, 128, true, 4)
DECODE_KERNEL(w4a16_decode_g32_bf16_rb1, 32, true, 1)
DECODE_KERNEL(w4a16_decode_g32_bf16_rb2, 32, true, 2)
DECODE_KERNEL(w4a16_decode_g32_bf16_rb4, 32, true, 4)
