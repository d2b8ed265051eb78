// Decode regime (t = 1..16 activation rows): HBM-streaming skinny GEMM  y[t][n] = x[t][k] * W^T.
// Role of the reference's gemv_t / split-K decode kernels (assets/gptq4.cu:522-553, assets/decode.cu:46-267),
// designed for CDNA4 instead:
//   * weights are read once, as 1 KiB tiles (64 lanes x buffer_load_dwordx4) of the tiled layout in
//     w4a16_common.hpp — every wave-level load is one fully used contiguous KiB;
//   * the int4 -> f16 unpack is 9 VALU ops per 8 weights and stays in registers; the multiply-accumulate runs on
//     the matrix core: dword w of the 64 lanes is the A operand of v_mfma_f32_16x16x32_f16 (16 rows x 32 k), the
//     B operand is x (32 k x 16 token columns), so t = 1 and t = 16 cost the same arithmetic;
//   * x: every vector-memory instruction costs the CU's address unit about as much as a full 1 KiB load however few
//     lanes are live, so one B-operand load per MFMA would cost more than the weight stream.  For t <= 4 a single
//     buffer load per k tile brings all four 32-k chunks (lane m fetches chunk m/4 of token m%4; lanes for tokens
//     >= t are out of range: zeros, no traffic) and v_mov_b32_dpp row_shl moves chunk c to the token's column;
//     t <= 8 takes two loads, t <= 16 four (no shuffles).  No LDS and no barrier on the streaming path;
//   * weights enter the MFMA as exact integers; the per-group scale multiplies the f32 group sum, so no weight is
//     ever rounded to f16 (error vs the f32 lane contract is summation order only);
//   * each wave keeps DEPTH k-tiles of loads in flight (register ring, software pipelined);
//   * split-K lives inside the workgroup: the W waves of a block take consecutive k-tile slices of the same RB row
//     blocks and wave 0 folds the partial tiles through LDS in fixed order (deterministic, no atomics, no second
//     launch).  The host picks RB and W.
#include "w4a16_common.hpp"

// One pipeline stage = the loads of one k tile: RB weight tiles, their scales, and XL loads of x.
template <int G, int RB, int XL>
struct DecodeStage {
    u4_t q[RB];
    u2_t s[RB][W4_TILE_K / G];
    u4_t x[XL];
};

// Data of lane (i + SH) of the same 16-lane row (zero past the row end): v_mov_b32_dpp row_shl.
template <int SH>
__device__ __forceinline__ u4_t w4_row_shl(u4_t v) {
    u4_t r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = __builtin_amdgcn_update_dpp(0u, v[i], 0x100 + SH, 0xF, 0xF, true);
    return r;
}

// XL = vector loads of x per k tile: 1 serves t <= 4, 2 serves t <= 8, 4 serves t <= 16.
template <int G, bool SBF, int RB, int DEPTH, int XL>
__device__ __forceinline__ void decode_body(const u4_t* __restrict__ qt, const uint16_t* __restrict__ st,
                                            const uint16_t* __restrict__ x, void* __restrict__ y, int row_blocks,
                                            int k, int n, int t, int out_f16) {
    extern __shared__ f4_t red[];  // [W][RB][64] partial tiles of the in-block split-K
    constexpr int GPT = W4_TILE_K / G;  // scale groups per k tile
    constexpr int C = 4 / XL;           // 32-k chunks (MFMAs) served by one x load
    constexpr int TPL = 16 / C;         // token columns served by one x load
    const int lane = threadIdx.x & 63, W = blockDim.x >> 6;
    // the wave index is uniform across the wave: keep it (and everything derived from it) in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kt_n = k / W4_TILE_K;
    const int kg_n = kt_n * GPT;
    const int nb0 = blockIdx.x * RB;
    const int kt0 = (kt_n * wave) / W, kt1 = (kt_n * (wave + 1)) / W;
    const int m = lane & 15, g = lane >> 4;

    // Every load is a raw buffer load: an out-of-range offset returns zeros and costs no memory traffic, which
    // predicates tiles past kt1 and token columns >= t without a branch.
    const __amdgpu_buffer_rsrc_t qr = w4_make_rsrc(qt, (unsigned)row_blocks * (unsigned)kt_n * 1024u);
    const __amdgpu_buffer_rsrc_t sr = w4_make_rsrc(st, (unsigned)row_blocks * (unsigned)kg_n * 32u);
    const __amdgpu_buffer_rsrc_t xr = w4_make_rsrc(x, (unsigned)t * (unsigned)k * 2u);
    // x load l of a tile: lane (m, g) fetches, for token m % TPL, the 8 halves of chunk l*C + m / TPL at k offset g*8
    const int xtok = m % TPL, xchunk = m / TPL;
    const unsigned xoff = xtok < t ? ((unsigned)xtok * (unsigned)k + (unsigned)(xchunk * 32 + g * 8)) * 2u : W4_OOB;
    f4_t acc[RB];
    unsigned qoff[RB], soff[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        acc[rb] = (f4_t){0.f, 0.f, 0.f, 0.f};
        const unsigned nb = (unsigned)min(nb0 + rb, row_blocks - 1);  // a tail block re-reads the last row block
        qoff[rb] = nb * (unsigned)kt_n * 1024u + (unsigned)lane * 16u;
        soff[rb] = nb * (unsigned)kg_n * 32u + (unsigned)g * 8u;
    }

    DecodeStage<G, RB, XL> stage[DEPTH];
    auto load = [&](DecodeStage<G, RB, XL>& s_, int kt) {
        const bool live = kt < kt1;
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
            s_.q[rb] = __builtin_amdgcn_raw_buffer_load_b128(qr, live ? qoff[rb] + (unsigned)kt * 1024u : W4_OOB, 0,
                                                             2 /* nt: read-once stream */);
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int gi = 0; gi < GPT; gi++)
                s_.s[rb][gi] = __builtin_amdgcn_raw_buffer_load_b64(
                    sr, live ? soff[rb] + (unsigned)(kt * GPT + gi) * 32u : W4_OOB, 0, 0);
#pragma unroll
        for (int l = 0; l < XL; l++)
            s_.x[l] = __builtin_amdgcn_raw_buffer_load_b128(
                xr, live ? xoff + (unsigned)(kt * W4_TILE_K + l * C * 32) * 2u : W4_OOB, 0, 0);
    };
    auto compute = [&](const DecodeStage<G, RB, XL>& s_) {
        // B operand of MFMA w = chunk w of x for token column m: held by lane (m + (w % C) * TPL) of load w / C
        u4_t xb[4];
#pragma unroll
        for (int l = 0; l < XL; l++) {
            xb[l * C] = s_.x[l];
            if (C >= 2) xb[l * C + 1] = w4_row_shl<TPL>(s_.x[l]);
            if (C == 4) {
                xb[2] = w4_row_shl<2 * TPL>(s_.x[l]);
                xb[3] = w4_row_shl<3 * TPL>(s_.x[l]);
            }
        }
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            if (G == 128) {
                f4_t part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int w = 0; w < 4; w++)
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][w]),
                                                                  __builtin_bit_cast(h8_t, xb[w]), part, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; i++)
                    acc[rb][i] += w4_scale_fast<SBF>((s_.s[rb][0][i >> 1] >> (16 * (i & 1))) & 0xFFFFu) * part[i];
            } else {
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    f4_t part = {0.f, 0.f, 0.f, 0.f};
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][w]),
                                                                  __builtin_bit_cast(h8_t, xb[w]), part, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        acc[rb][i] +=
                            w4_scale_fast<SBF>((s_.s[rb][w % GPT][i >> 1] >> (16 * (i & 1))) & 0xFFFFu) * part[i];
                }
            }
        }
    };

    // One counted loop does the pipeline fill (round -1, compute skipped) and the steady state, so on every path
    // into a stage's compute the outstanding loads are in ring order and the wait can leave the younger stages' loads
    // in flight (s_waitcnt vmcnt(N > 0)).  Tiles past kt1 load zeros and are never computed; the last partial round
    // is finished by the unrolled tail.  The scheduling barriers keep each stage's loads together.
    const int tiles = kt1 - kt0;
    const int rounds = tiles / DEPTH;
    for (int r = -1; r < rounds; r++) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            if (r >= 0) compute(stage[d]);
            __builtin_amdgcn_sched_barrier(0);
            load(stage[d], kt0 + (r + 1) * DEPTH + d);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int d = 0; d < DEPTH - 1; d++)
        if (rounds * DEPTH + d < tiles) compute(stage[d]);

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
    if (m >= t) return;
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

// ring depth: as many stages as ~96 VGPRs of load buffers allow
#define DECODE_DEPTH(G, RB, XL) \
    ((96 / (4 * RB + 2 * RB * (W4_TILE_K / G) + 4 * XL)) < 2 ? 2 : (96 / (4 * RB + 2 * RB * (W4_TILE_K / G) + 4 * XL)) > 8 ? 8 : (96 / (4 * RB + 2 * RB * (W4_TILE_K / G) + 4 * XL)))

#define DECODE_KERNEL_X(NAME, G, SBF, RB, XL)                                                                        \
    extern "C" __global__ __launch_bounds__(512) void NAME##_x##XL(const u4_t* qt, const uint16_t* st,               \
                                                                   const uint16_t* x, void* y, int row_blocks,       \
                                                                   int k, int n, int t, int out_f16) {               \
        decode_body<G, SBF, RB, DECODE_DEPTH(G, RB, XL), XL>(qt, st, x, y, row_blocks, k, n, t, out_f16);            \
    }
#define DECODE_KERNEL(NAME, G, SBF, RB) \
    DECODE_KERNEL_X(NAME, G, SBF, RB, 1) DECODE_KERNEL_X(NAME, G, SBF, RB, 2) DECODE_KERNEL_X(NAME, G, SBF, RB, 4)

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
