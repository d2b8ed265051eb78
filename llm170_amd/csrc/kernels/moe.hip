// MoE expert FFN on W4A16 experts: routing, slot alignment, grouped/ragged expert GEMMs, top-k reduction.
// Role of the reference's route -> align -> grouped gate+up -> SiLU*up -> grouped down (x top-k weight) -> sum
// sequence (w4a16_dec/kernels/marlin_moe.rs:290-422 over assets/moe.cu:686-759, 860-908, 1599-1674 and the vendored
// grouped Marlin kernels), designed for CDNA4:
//   * a "slot" is one (token, chosen expert) pair, slot j = token * top_k + choice.  The align kernel sorts slots by
//     expert (stable) and pads every expert's run to a multiple of the segment size; a segment = up to BLK slots of
//     one expert.  Workgroups are numbered (segment, output-row group); segments past the padded total exit at once.
//   * expert weights live in one arena in the tiled layout of w4a16_common.hpp, experts at a fixed stride; the
//     gate and up projections are one fused matrix (rows 0..n_ff gate, n_ff..2 n_ff up; upload.rs:1116-1235).
//   * both regimes multiply on v_mfma_f32_16x16x32_f16 with weights as exact integers (A operand = one dword of the
//     64 lanes of a tile) and apply the group scale to the f32 group sum, like the dense decode kernel.
//       - moe_dec (segments of <= 4 or <= 16 slots, decode steps): HBM streaming, in-block split-K over the waves,
//         x gathered straight from global memory (one load + DPP row shifts for <= 4 slots);
//       - moe_mm (segments of 16..64 slots, prefill chunks): the waves of a block take different output rows of the
//         same segment and share the gathered x rows through LDS (double buffered, one k tile per stage), so x is
//         fetched once per block instead of once per wave.
//   * decode steps of at most four tokens skip the alignment: the gate|up GEMM runs one segment per slot (segment table
//     = identity, expert table = idx itself) and moe_down_sum does the down projection of a token's experts, the
//     routing-weight multiply, the f16 rounding and the slot-order sum in one launch — two launches per FFN;
//   * GLU epilogue: a wave owns gate row block u and up row block u + n_ff/16, rounds both sums to f16 (the reference
//     materialises them as f16, moe.cu:1649-1660) and writes silu(g)*u as f16 — the intermediate never reaches
//     memory.  LIN epilogue: optional multiply by the slot's routing weight, f16 or f32 rows scattered by slot id.
//   * for group size 32 the four scale groups of a k tile come with ONE load per row block: lane c of each quad
//     fetches group c % 4 and v_mov_b32_dpp quad_perm broadcasts group w when MFMA w needs it.
#include <type_traits>

#include "w4a16_common.hpp"

#define MOE_LDX 136  // halves per staged x row: 128 + 8 padding (272-byte stride: 16-lane b128 reads hit all banks once)

template <int W>
__device__ __forceinline__ unsigned w4_quad_bcast(unsigned v) {
    return __builtin_amdgcn_update_dpp(0u, v, W * 0x55, 0xF, 0xF, true);
}

template <int SH>
__device__ __forceinline__ u4_t moe_row_shl(u4_t v) {
    u4_t r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = __builtin_amdgcn_update_dpp(0u, v[i], 0x100 + SH, 0xF, 0xF, true);
    return r;
}

// The four scales (rows 4q..4q+3 of the row block) of scale group W of the current k tile, as f32.
// s = the lane's b64 scale load: for G = 128 the tile's only group, for G = 32 group (lane % 4).
template <int G, bool SBF, int W>
__device__ __forceinline__ f4_t moe_scale4(u2_t s) {
    unsigned d0 = s[0], d1 = s[1];
    if (G == 32) {
        d0 = w4_quad_bcast<W>(d0);
        d1 = w4_quad_bcast<W>(d1);
    }
    f4_t r;
    r[0] = w4_scale_fast<SBF>(d0 & 0xFFFFu);
    r[1] = w4_scale_fast<SBF>(d0 >> 16);
    r[2] = w4_scale_fast<SBF>(d1 & 0xFFFFu);
    r[3] = w4_scale_fast<SBF>(d1 >> 16);
    return r;
}

__device__ __forceinline__ float moe_round_f16(float v) { return (float)(_Float16)v; }

// Epilogue of one 16 x 16 result tile pair for one token column.  a0/a1: the lane's four rows of row blocks 0/1 of
// the unit.  GLU: a0 = gate, a1 = up -> act[slot][u*16 + 4q + i] = f16(silu(f16(g)) * f16(u)).
// LIN: rows of row blocks rbA / rbB, scaled by wgt, as f16 or f32.
template <bool GLU>
__device__ __forceinline__ void moe_store(f4_t a0, f4_t a1, int slot, int q, int u, int rbA, int rbB, bool haveB,
                                          void* __restrict__ y, int y_f16, float wgt, int n, int act_kind) {
    if (GLU) {
        const int n_ff = n >> 1;
        h4_t o;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // expert FFN: gate and up are f16 tensors in the reference and are rounded first; a dense gated linear
            // (bit 1 of act_kind) applies the activation to the f32 sums, like the separate element-wise kernel
            float g = (act_kind & 2) ? a0[i] : moe_round_f16(a0[i]), up = (act_kind & 2) ? a1[i] : moe_round_f16(a1[i]);
            float v = w4_act_mul(g, up, act_kind & 1);
            asm volatile("" : "+v"(v));  // the product is rounded to f32 before the f16 conversion
            o[i] = (_Float16)v;
        }
        *reinterpret_cast<h4_t*>(reinterpret_cast<_Float16*>(y) + (size_t)slot * n_ff + u * 16 + 4 * q) = o;
    } else {
#pragma unroll
        for (int rb = 0; rb < 2; rb++) {
            if (rb == 1 && !haveB) break;
            const f4_t a = (rb == 0 ? a0 : a1) * wgt;
            const int row = (rb == 0 ? rbA : rbB) * 16 + 4 * q;
            if (y_f16) {
                _Float16* yo = reinterpret_cast<_Float16*>(y) + (size_t)slot * n + row;
                if (row + 3 < n) {
                    h4_t v = {(_Float16)a[0], (_Float16)a[1], (_Float16)a[2], (_Float16)a[3]};
                    *reinterpret_cast<h4_t*>(yo) = v;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (row + i < n) yo[i] = (_Float16)a[i];
                }
            } else {
                float* yo = reinterpret_cast<float*>(y) + (size_t)slot * n + row;
                if (row + 3 < n) {
                    *reinterpret_cast<f4_t*>(yo) = a;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (row + i < n) yo[i] = a[i];
                }
            }
        }
    }
}

// Arguments shared by the two grouped kernels.
//   qa/sa: arena bases, expert e at qa + e*q_stride / sa + e*s_stride (bytes); each expert is row_blocks x k/128
//          tiles and [row_blocks][k/G][16] scales.  x: f16 [x_rows][k]; slot j reads row j / x_div.
//   y: GLU -> f16 [ns][n/2]; LIN -> f16 or f32 [ns][n].  topw: null or f32 [ns] (LIN only).
//   sorted_ids[seg*blk + i]: slot id or the sentinel ns; expert_ids[seg]; num_post[0] = padded slot total.
//   A segment whose expert id is outside 0..n_exp-1 is skipped (its slots stay unwritten).
//   ws / tickets: workspace and zeroed counters of a launch split over k across workgroups (gridDim.y slices; the
//   LDS-staged kernel only): [slice][block][wave][2*TT] partial tiles, one counter per (block, wave).
//   act_kind (GLU only): bit 0: 0 = silu(gate) * up (w4a16_moe_act_silu_f16), 1 = the tanh form of gelu on the gate
//   (w4a16_moe_act_gelu_f16, assets/moe.cu:1635-1647); bit 1: gate and up enter the activation as f32 sums (a dense
//   gated linear) instead of being rounded to f16 first (the expert FFN).
//   wpb: waves per block (the block size, as an argument: read from the dispatch packet it costs one more dependent
//   scalar-cache miss before the first weight load).
#define MOE_PARAMS                                                                                                  \
    const char *__restrict__ qa, const char *__restrict__ sa, unsigned long long q_stride,                          \
        unsigned long long s_stride, const uint16_t *__restrict__ x, int x_rows, int x_div, void *__restrict__ y,   \
        int y_f16, const float *__restrict__ topw, const int *__restrict__ sorted_ids,                              \
        const int *__restrict__ expert_ids, const int *__restrict__ num_post, int blk, int ns, int row_blocks, int k, \
        int n, int n_exp, f4_t *ws, int *tickets, int wpb, int act_kind
#define MOE_ARGS \
    qa, sa, q_stride, s_stride, x, x_rows, x_div, y, y_f16, topw, sorted_ids, expert_ids, num_post, blk, ns, row_blocks, k, n, n_exp, ws, tickets, wpb, act_kind

// ---------------------------------------------------------------------------------------------------- moe_dec
template <int RB, int XL>
struct MoeDecStage {
    u4_t q[RB];
    u2_t s[RB];
    u4_t x[XL];
};

// One block = (segment, unit of two row blocks); its W waves split k.  XL = 1: blk <= 4; XL = 4: blk <= 16.
template <int G, bool SBF, bool GLU, int XL, int DEPTH>
__device__ __forceinline__ void moe_dec_body(MOE_PARAMS) {
    extern __shared__ f4_t red[];  // [W][2][64]
    constexpr int GPT = W4_TILE_K / G;
    constexpr int C = 4 / XL, TPL = 16 / C;
    const int lane = threadIdx.x & 63, W = wpb;
    // every kernel argument is fetched here, in one batch: left to the compiler they arrive in three dependent
    // scalar-cache misses spread over the prologue, each ahead of the first weight load
    asm volatile("" ::"s"(qa), "s"(sa), "s"(q_stride), "s"(s_stride), "s"(x), "s"(x_rows), "s"(x_div), "s"(y), "s"(topw),
                 "s"(sorted_ids), "s"(blk), "s"(ns), "s"(row_blocks), "s"(k), "s"(n),
                 "s"(n_exp), "s"(wpb));
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int units = GLU ? row_blocks >> 1 : (row_blocks + 1) >> 1;
    const int seg = blockIdx.x / units, u = blockIdx.x % units;
    const int m = lane & 15, g = lane >> 4;
    const int xtok = m % TPL, xchunk = m / TPL;
    // The three table reads (padded total, the segment's expert, the lane's slot id) are issued together, ahead of
    // the tests that use them: one memory round trip before the first weight load instead of three.  The tables hold
    // an entry for every segment the grid was sized for.
    int np = num_post[0], e = expert_ids[seg], xslot = sorted_ids[seg * blk + min(xtok, blk - 1)];
    asm volatile("" : "+s"(np), "+s"(e), "+v"(xslot));
    if (seg * blk >= np) return;
    if ((unsigned)e >= (unsigned)n_exp) return;  // uniform for the block
    if (xtok >= blk) xslot = ns;
    const int kt_n = k / W4_TILE_K, kg_n = kt_n * GPT;
    const int kt0 = (kt_n * wave) / W, kt1 = (kt_n * (wave + 1)) / W;
    const int rbA = GLU ? u : 2 * u, rbB = GLU ? u + units : min(2 * u + 1, row_blocks - 1);
    const bool haveB = GLU || 2 * u + 1 < row_blocks;

    const __amdgpu_buffer_rsrc_t qr =
        w4_make_rsrc(qa + (unsigned long long)e * q_stride, (unsigned)row_blocks * (unsigned)kt_n * 1024u);
    const __amdgpu_buffer_rsrc_t sr =
        w4_make_rsrc(sa + (unsigned long long)e * s_stride, (unsigned)row_blocks * (unsigned)kg_n * 32u);
    const __amdgpu_buffer_rsrc_t xr = w4_make_rsrc(x, (unsigned)x_rows * (unsigned)k * 2u);

    const unsigned xoff =
        xslot < ns ? ((unsigned)(xslot / x_div) * (unsigned)k + (unsigned)(xchunk * 32 + g * 8)) * 2u : W4_OOB;
    const unsigned qoff[2] = {(unsigned)rbA * (unsigned)kt_n * 1024u + (unsigned)lane * 16u,
                              (unsigned)rbB * (unsigned)kt_n * 1024u + (unsigned)lane * 16u};
    // scale load: G = 128 -> the tile's group; G = 32 -> group (lane % 4) of the tile's four
    const unsigned sg = G == 32 ? (unsigned)(lane & 3) * 32u : 0u;
    const unsigned soff[2] = {(unsigned)rbA * (unsigned)kg_n * 32u + sg + (unsigned)g * 8u,
                              (unsigned)rbB * (unsigned)kg_n * 32u + sg + (unsigned)g * 8u};
    f4_t acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};

    MoeDecStage<2, XL> stage[DEPTH];
    auto load = [&](MoeDecStage<2, XL>& s_, int kt) {
        const bool live = kt < kt1;
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
            s_.q[rb] = __builtin_amdgcn_raw_buffer_load_b128(qr, live ? qoff[rb] + (unsigned)kt * 1024u : W4_OOB, 0, 2);
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
            s_.s[rb] = __builtin_amdgcn_raw_buffer_load_b64(sr, live ? soff[rb] + (unsigned)kt * (GPT * 32u) : W4_OOB, 0, 0);
#pragma unroll
        for (int l = 0; l < XL; l++)
            s_.x[l] = __builtin_amdgcn_raw_buffer_load_b128(
                xr, live ? xoff + (unsigned)(kt * W4_TILE_K + l * C * 32) * 2u : W4_OOB, 0, 0);
    };
    auto compute = [&](const MoeDecStage<2, XL>& s_) {
        u4_t xb[4];
#pragma unroll
        for (int l = 0; l < XL; l++) {
            xb[l * C] = s_.x[l];
            if (C == 4) {
                xb[1] = moe_row_shl<TPL>(s_.x[l]);
                xb[2] = moe_row_shl<2 * TPL>(s_.x[l]);
                xb[3] = moe_row_shl<3 * TPL>(s_.x[l]);
            }
        }
#pragma unroll
        for (int rb = 0; rb < 2; rb++) {
            const f4_t zero = {0.f, 0.f, 0.f, 0.f};
            if (G == 128) {
                f4_t part = zero;
#pragma unroll
                for (int w = 0; w < 4; w++)
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][w]),
                                                                  __builtin_bit_cast(h8_t, xb[w]), part, 0, 0, 0);
                acc[rb] = w4_fma4(moe_scale4<G, SBF, 0>(s_.s[rb]), part, acc[rb]);
            } else {
                f4_t p0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][0]), __builtin_bit_cast(h8_t, xb[0]), zero, 0, 0, 0);
                f4_t p1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][1]), __builtin_bit_cast(h8_t, xb[1]), zero, 0, 0, 0);
                f4_t p2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][2]), __builtin_bit_cast(h8_t, xb[2]), zero, 0, 0, 0);
                f4_t p3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][3]), __builtin_bit_cast(h8_t, xb[3]), zero, 0, 0, 0);
                acc[rb] = w4_fma4(moe_scale4<G, SBF, 0>(s_.s[rb]), p0, acc[rb]);
                acc[rb] = w4_fma4(moe_scale4<G, SBF, 1>(s_.s[rb]), p1, acc[rb]);
                acc[rb] = w4_fma4(moe_scale4<G, SBF, 2>(s_.s[rb]), p2, acc[rb]);
                acc[rb] = w4_fma4(moe_scale4<G, SBF, 3>(s_.s[rb]), p3, acc[rb]);
            }
        }
    };

    // counted loop: round -1 fills the ring with compute skipped, so the loads outstanding at every stage's wait are
    // in ring order (see the dense decode kernel)
    const int tiles = kt1 - kt0;
    const int rounds = tiles / DEPTH;
    for (int r = -1; r < rounds; r++) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            __builtin_amdgcn_s_setprio(1);  // compute ahead of the waves that are queueing loads (1-2 % at T <= 4)
            if (r >= 0) compute(stage[d]);
            __builtin_amdgcn_s_setprio(0);
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
            red[(wave * 2 + 0) * 64 + lane] = acc[0];
            red[(wave * 2 + 1) * 64 + lane] = acc[1];
        }
        __syncthreads();
        if (wave != 0) return;
        for (int w = 1; w < W; w++) {
            acc[0] += red[(w * 2 + 0) * 64 + lane];
            acc[1] += red[(w * 2 + 1) * 64 + lane];
        }
    }
    const int slot = m < blk ? sorted_ids[seg * blk + m] : ns;
    if (slot >= ns) return;
    const float wgt = (!GLU && topw) ? topw[slot] : 1.0f;
    moe_store<GLU>(acc[0], acc[1], slot, g, u, rbA, rbB, haveB, y, y_f16, wgt, n, act_kind);
}

// ---------------------------------------------------------------------------------------------------- moe_down_sum
// Decode steps (a handful of tokens): the down projection of all of a token's experts and the slot-order sum in one
// launch.  One block = (token, unit of two row blocks); wave w < top_k owns slot token*top_k + w: it streams that
// expert's rows over the whole k range with the slot's activation row as x, multiplies by the routing weight and
// rounds to f16 exactly as the staged path materialises c2; wave 0 then adds the waves' values in slot order in f32
// (the same order as the separate sum kernel) and writes y f32 [t][n].  No alignment pass is needed: the expert of
// a slot is read straight from idx.
// RB: row blocks of a workgroup's unit — 2, or 1 for a handful of tokens, when units of two leave most CUs without work.
template <int G, bool SBF, int DEPTH, int RB>
__device__ __forceinline__ void moe_down_sum_body(const char* __restrict__ qa, const char* __restrict__ sa,
                                                  unsigned long long q_stride, unsigned long long s_stride,
                                                  const uint16_t* __restrict__ act, const int* __restrict__ idx,
                                                  const float* __restrict__ topw, float* __restrict__ y, int top_k,
                                                  int ns, int row_blocks, int k, int n, int n_exp) {
    extern __shared__ f4_t red[];  // [top_k][RB][64]
    constexpr int GPT = W4_TILE_K / G;
    const int lane = threadIdx.x & 63;
    // every kernel argument is fetched here, in one batch (see moe_dec_body)
    asm volatile("" ::"s"(qa), "s"(sa), "s"(q_stride), "s"(s_stride), "s"(act), "s"(idx), "s"(topw), "s"(y), "s"(top_k),
                 "s"(ns), "s"(row_blocks), "s"(k), "s"(n), "s"(n_exp));
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int units = (row_blocks + RB - 1) / RB;
    const int token = blockIdx.x / units, u = blockIdx.x % units;
    const int slot = token * top_k + wave;
    const int e_raw = __builtin_amdgcn_readfirstlane(idx[slot]);
    const bool valid = (unsigned)e_raw < (unsigned)n_exp;  // an out-of-range expert id contributes zero
    const int e = valid ? e_raw : 0;
    const int kt_n = k / W4_TILE_K, kg_n = kt_n * GPT;
    const int m = lane & 15, g = lane >> 4;
    const int rbA = RB * u, rbB = min(RB * u + 1, row_blocks - 1);
    const bool haveB = RB == 2 && 2 * u + 1 < row_blocks;

    const __amdgpu_buffer_rsrc_t qr = w4_make_rsrc(qa + (unsigned long long)e * q_stride,
                                                   valid ? (unsigned)row_blocks * (unsigned)kt_n * 1024u : 0u);
    const __amdgpu_buffer_rsrc_t sr = w4_make_rsrc(sa + (unsigned long long)e * s_stride,
                                                   valid ? (unsigned)row_blocks * (unsigned)kg_n * 32u : 0u);
    const __amdgpu_buffer_rsrc_t xr = w4_make_rsrc(act, (unsigned)ns * (unsigned)k * 2u);
    // one x load per k tile: lane m = 4c fetches chunk c of the slot's row; DPP row shifts bring chunk c to column 0
    const unsigned xoff = (m & 3) == 0 ? ((unsigned)slot * (unsigned)k + (unsigned)((m >> 2) * 32 + g * 8)) * 2u : W4_OOB;
    const unsigned qoff[2] = {(unsigned)rbA * (unsigned)kt_n * 1024u + (unsigned)lane * 16u,
                              (unsigned)rbB * (unsigned)kt_n * 1024u + (unsigned)lane * 16u};
    const unsigned sg = G == 32 ? (unsigned)(lane & 3) * 32u : 0u;
    const unsigned soff[2] = {(unsigned)rbA * (unsigned)kg_n * 32u + sg + (unsigned)g * 8u,
                              (unsigned)rbB * (unsigned)kg_n * 32u + sg + (unsigned)g * 8u};
    f4_t acc[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) acc[rb] = (f4_t){0.f, 0.f, 0.f, 0.f};

    MoeDecStage<RB, 1> stage[DEPTH];
    auto load = [&](MoeDecStage<RB, 1>& s_, int kt) {
        const bool live = kt < kt_n;
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
            s_.q[rb] = __builtin_amdgcn_raw_buffer_load_b128(qr, live ? qoff[rb] + (unsigned)kt * 1024u : W4_OOB, 0, 2);
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
            s_.s[rb] = __builtin_amdgcn_raw_buffer_load_b64(sr, live ? soff[rb] + (unsigned)kt * (GPT * 32u) : W4_OOB, 0, 0);
        s_.x[0] = __builtin_amdgcn_raw_buffer_load_b128(xr, live ? xoff + (unsigned)(kt * W4_TILE_K) * 2u : W4_OOB, 0, 0);
    };
    auto compute = [&](const MoeDecStage<RB, 1>& s_) {
        u4_t xb[4];
        xb[0] = s_.x[0];
        xb[1] = moe_row_shl<4>(s_.x[0]);
        xb[2] = moe_row_shl<8>(s_.x[0]);
        xb[3] = moe_row_shl<12>(s_.x[0]);
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            const f4_t zero = {0.f, 0.f, 0.f, 0.f};
            if (G == 128) {
                f4_t part = zero;
#pragma unroll
                for (int w = 0; w < 4; w++)
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][w]),
                                                                  __builtin_bit_cast(h8_t, xb[w]), part, 0, 0, 0);
                acc[rb] = w4_fma4(moe_scale4<G, SBF, 0>(s_.s[rb]), part, acc[rb]);
            } else {
                f4_t p0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][0]), __builtin_bit_cast(h8_t, xb[0]), zero, 0, 0, 0);
                f4_t p1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][1]), __builtin_bit_cast(h8_t, xb[1]), zero, 0, 0, 0);
                f4_t p2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][2]), __builtin_bit_cast(h8_t, xb[2]), zero, 0, 0, 0);
                f4_t p3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][3]), __builtin_bit_cast(h8_t, xb[3]), zero, 0, 0, 0);
                acc[rb] = w4_fma4(moe_scale4<G, SBF, 0>(s_.s[rb]), p0, acc[rb]);
                acc[rb] = w4_fma4(moe_scale4<G, SBF, 1>(s_.s[rb]), p1, acc[rb]);
                acc[rb] = w4_fma4(moe_scale4<G, SBF, 2>(s_.s[rb]), p2, acc[rb]);
                acc[rb] = w4_fma4(moe_scale4<G, SBF, 3>(s_.s[rb]), p3, acc[rb]);
            }
        }
    };
    const int rounds = kt_n / DEPTH;
    for (int r = -1; r < rounds; r++) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            __builtin_amdgcn_s_setprio(1);  // compute ahead of the waves that are queueing loads (1-2 % at T <= 4)
            if (r >= 0) compute(stage[d]);
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            load(stage[d], (r + 1) * DEPTH + d);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int d = 0; d < DEPTH - 1; d++)
        if (rounds * DEPTH + d < kt_n) compute(stage[d]);

    // c2 of this slot: routing weight, one rounding to f16 (the value the staged path stores), back to f32
    const float wgt = topw[slot];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // the product is rounded to f32 first, as where c2 is materialised (the compiler would otherwise fold the
            // multiply into the conversion, v_fma_mixlo_f16: one rounding of the exact product instead of two)
            float p = acc[rb][i] * wgt;
            asm volatile("" : "+v"(p));
            acc[rb][i] = moe_round_f16(p);
        }
        red[(wave * RB + rb) * 64 + lane] = acc[rb];
    }
    __syncthreads();
    if (wave != 0 || m != 0) return;
    f4_t sum[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) sum[rb] = (f4_t){0.f, 0.f, 0.f, 0.f};
    for (int w = 0; w < top_k; w++) {
#pragma unroll
        for (int rb = 0; rb < RB; rb++) sum[rb] += red[(w * RB + rb) * 64 + lane];
    }
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        if (rb == 1 && !haveB) break;
        const int row = (rb == 0 ? rbA : rbB) * 16 + 4 * g;
        float* yo = y + (size_t)token * n + row;
        if (row + 3 < n) {
            *reinterpret_cast<f4_t*>(yo) = sum[rb];
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (row + i < n) yo[i] = sum[rb][i];
        }
    }
}

#define MOE_DOWN_SUM_KERNEL(NAME, G, SBF, RB)                                                                     \
    extern "C" __global__ __launch_bounds__(512) void NAME(                                                       \
        const char* qa, const char* sa, unsigned long long q_stride, unsigned long long s_stride,                 \
        const uint16_t* act, const int* idx, const float* topw, float* y, int top_k, int ns, int row_blocks, int k, \
        int n, int n_exp) {                                                                                       \
        moe_down_sum_body<G, SBF, 3, RB>(qa, sa, q_stride, s_stride, act, idx, topw, y, top_k, ns, row_blocks, k, \
                                         n, n_exp);                                                               \
    }
MOE_DOWN_SUM_KERNEL(w4a16_moe_g32_f16_down_sum, 32, false, 2)
MOE_DOWN_SUM_KERNEL(w4a16_moe_g32_bf16_down_sum, 32, true, 2)
MOE_DOWN_SUM_KERNEL(w4a16_moe_g128_f16_down_sum, 128, false, 2)
MOE_DOWN_SUM_KERNEL(w4a16_moe_g128_bf16_down_sum, 128, true, 2)
MOE_DOWN_SUM_KERNEL(w4a16_moe_g32_f16_down_sum1, 32, false, 1)
MOE_DOWN_SUM_KERNEL(w4a16_moe_g32_bf16_down_sum1, 32, true, 1)
MOE_DOWN_SUM_KERNEL(w4a16_moe_g128_f16_down_sum1, 128, false, 1)
MOE_DOWN_SUM_KERNEL(w4a16_moe_g128_bf16_down_sum1, 128, true, 1)

// ---------------------------------------------------------------------------------------------------- moe_mm
template <int RB>
struct MoeMmStage {
    u4_t q[RB];
    u2_t s[RB];
};

#define MOE_MAX_KSPLIT 8  // k slices across workgroups; the host clamps to this

// One block = (segment of blk = 16*TT slots, group of W units); wave w owns unit group*W + w over the whole k range.
// KS: the launch may be split over k across workgroups (dense linears run as one expert; the expert FFN never splits, and
// its kernels are built without the epilogue that costs them registers).
// TT: the 16-slot blocks of the segment this workgroup multiplies (those that hold a slot); TTMAX: the blocks of a full
// segment, which size a wave's share of the split-k workspace.
template <int G, bool SBF, bool GLU, int TT, int TTMAX, int DEPTH, bool KS>
__device__ __forceinline__ void moe_mm_body(MOE_PARAMS) {
    extern __shared__ _Float16 xs[];  // [2][16*TT][MOE_LDX]
    constexpr int GPT = W4_TILE_K / G;
    constexpr int ROWS = 16 * TT;
    const int tid = threadIdx.x, lane = tid & 63, W = wpb;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int units = GLU ? row_blocks >> 1 : (row_blocks + 1) >> 1;
    const int groups = (units + W - 1) / W;
    const int seg = blockIdx.x / groups, grp = blockIdx.x % groups;
    // the table reads (padded total, the segment's expert, this thread's slot ids) are issued together, ahead of the
    // tests that use them (see moe_dec_body)
    const int rows_pp = 4 * W;
    int np = num_post[0], e = expert_ids[seg];
    int slot_of[TT];
#pragma unroll
    for (int p = 0; p < TT; p++) slot_of[p] = sorted_ids[seg * blk + min(p * rows_pp + (tid >> 4), ROWS - 1)];
    asm volatile("" : "+s"(np), "+s"(e));
#pragma unroll
    for (int p = 0; p < TT; p++) asm volatile("" : "+v"(slot_of[p]));
    if (seg * blk >= np) return;  // uniform for the block, before any barrier
    const int u_raw = grp * W + wave;
    const bool active = u_raw < units;  // a surplus wave repeats the last unit and stores nothing
    const int u = min(u_raw, units - 1);
    if ((unsigned)e >= (unsigned)n_exp) return;  // uniform for the block, before any barrier
    const int kt_n = k / W4_TILE_K, kg_n = kt_n * GPT;
    const int nks = KS ? (int)gridDim.y : 1, ky = KS ? (int)blockIdx.y : 0;  // k slices across workgroups
    const int kt_lo = (kt_n * ky) / nks, kt_hi = (kt_n * (ky + 1)) / nks;
    const int c = lane & 15, q = lane >> 4;
    const int rbA = GLU ? u : 2 * u, rbB = GLU ? u + units : min(2 * u + 1, row_blocks - 1);
    const bool haveB = GLU || 2 * u + 1 < row_blocks;

    const __amdgpu_buffer_rsrc_t qr =
        w4_make_rsrc(qa + (unsigned long long)e * q_stride, (unsigned)row_blocks * (unsigned)kt_n * 1024u);
    const __amdgpu_buffer_rsrc_t sr =
        w4_make_rsrc(sa + (unsigned long long)e * s_stride, (unsigned)row_blocks * (unsigned)kg_n * 32u);
    const __amdgpu_buffer_rsrc_t xr = w4_make_rsrc(x, (unsigned)x_rows * (unsigned)k * 2u);

    // x staging: one k tile of the segment's rows = ROWS x 256 B; 16 threads cover a row, 4*W rows per pass
    unsigned xg_off[TT];
    int xl_off[TT];
#pragma unroll
    for (int p = 0; p < TT; p++) {
        const int row = p * rows_pp + (tid >> 4);
        const int slot = row < ROWS ? slot_of[p] : ns;
        xg_off[p] = slot < ns ? ((unsigned)(slot / x_div) * (unsigned)k + (unsigned)(tid & 15) * 8u) * 2u : W4_OOB;
        xl_off[p] = row < ROWS ? row * MOE_LDX + (tid & 15) * 8 : -1;
    }
    // x tiles travel global -> registers -> LDS two k tiles ahead of their use: the gathered rows come from L2 with a
    // latency longer than one k tile of compute.  One register set: an iteration stores the tile loaded in the previous
    // one and then loads the next into the same registers.
    u4_t xreg[TT];
    auto load_x = [&](u4_t (&r)[TT], int kt) {
#pragma unroll
        for (int p = 0; p < TT; p++)
            r[p] = __builtin_amdgcn_raw_buffer_load_b128(
                xr, (kt < kt_hi && xg_off[p] != W4_OOB) ? xg_off[p] + (unsigned)kt * (W4_TILE_K * 2u) : W4_OOB, 0, 0);
    };
    auto store_x = [&](const u4_t (&r)[TT], int buf) {
        _Float16* base = xs + buf * (ROWS * MOE_LDX);
#pragma unroll
        for (int p = 0; p < TT; p++)
            if (xl_off[p] >= 0) *reinterpret_cast<u4_t*>(base + xl_off[p]) = r[p];
    };

    const unsigned qoff[2] = {(unsigned)rbA * (unsigned)kt_n * 1024u + (unsigned)lane * 16u,
                              (unsigned)rbB * (unsigned)kt_n * 1024u + (unsigned)lane * 16u};
    const unsigned sg = G == 32 ? (unsigned)(lane & 3) * 32u : 0u;
    const unsigned soff[2] = {(unsigned)rbA * (unsigned)kg_n * 32u + sg + (unsigned)q * 8u,
                              (unsigned)rbB * (unsigned)kg_n * 32u + sg + (unsigned)q * 8u};
    MoeMmStage<2> stage[DEPTH];
    auto load_w = [&](MoeMmStage<2>& s_, int kt) {
        const bool live = kt < kt_hi;
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
            s_.q[rb] = __builtin_amdgcn_raw_buffer_load_b128(qr, live ? qoff[rb] + (unsigned)kt * 1024u : W4_OOB, 0, 2);
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
            s_.s[rb] = __builtin_amdgcn_raw_buffer_load_b64(sr, live ? soff[rb] + (unsigned)kt * (GPT * 32u) : W4_OOB, 0, 0);
    };

    f4_t acc[2][TT];
#pragma unroll
    for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int tt = 0; tt < TT; tt++) acc[rb][tt] = (f4_t){0.f, 0.f, 0.f, 0.f};

    auto compute = [&](const MoeMmStage<2>& s_, int buf) {
        const _Float16* xb = xs + buf * (ROWS * MOE_LDX) + c * MOE_LDX + q * 8;
        const f4_t zero = {0.f, 0.f, 0.f, 0.f};
        f4_t part[2][TT];
        auto step = [&](auto wc) {
            constexpr int w = decltype(wc)::value;
            h8_t b[TT];
#pragma unroll
            for (int tt = 0; tt < TT; tt++) b[tt] = *reinterpret_cast<const h8_t*>(xb + tt * 16 * MOE_LDX + w * 32);
#pragma unroll
            for (int rb = 0; rb < 2; rb++) {
                // G = 32 (segments of 64 slots only; smaller ones run compute32 below): every 32-k group's products are
                // scaled on their own, and left alone the compiler issues all 8 * TT MFMAs of a k tile into separate
                // result registers before the first scaled sum.  The empty asm statements pin the order group by group:
                // this group's unpack starts after the previous group's sums, so one group's results are live at a time.
                unsigned qw = s_.q[rb][w];
                if (G == 32) asm volatile("" : "+v"(qw));
                const h8_t a = w4_deq8(qw);
                if (G == 32) {
                    const f4_t sc = moe_scale4<G, SBF, w>(s_.s[rb]);
#pragma unroll
                    for (int tt = 0; tt < TT; tt++)
                        acc[rb][tt] = w4_fma4(sc, __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b[tt], zero, 0, 0, 0), acc[rb][tt]);
#pragma unroll
                    for (int tt = 0; tt < TT; tt++) asm volatile("" : "+v"(acc[rb][tt]));
                } else {
#pragma unroll
                    for (int tt = 0; tt < TT; tt++)
                        part[rb][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b[tt], w == 0 ? zero : part[rb][tt], 0, 0, 0);
                }
            }
        };
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
        step(std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 3>{});
        if (G == 128) {
#pragma unroll
            for (int rb = 0; rb < 2; rb++) {
                const f4_t sc = moe_scale4<G, SBF, 0>(s_.s[rb]);
#pragma unroll
                for (int tt = 0; tt < TT; tt++) acc[rb][tt] = w4_fma4(sc, part[rb][tt], acc[rb][tt]);
            }
        }
    };

    // Group size 32, up to three 16-slot blocks, software-pipelined by hand: a k tile is eight groups (32 k x one row
    // block), each TT MFMAs into fresh results, the scale conversion and 4 * TT scaled sums.  Issue order per group: its
    // MFMAs; then the NEXT group's unpack (and, when the 32-k chunk changes, the next B operands from LDS) while the
    // matrix pipe works; then this group's scaled sums; then the next group's MFMAs, whose operands are ready.  A wave
    // does not wait for its own MFMAs (the order "unpack, MFMAs, sums" group by group left 5-8 idle cycles after every
    // MFMA for the other waves to fill).  Scheduling barriers hold the phases in this order; one group's results are
    // live at a time.  128 experts, top-8: T = 64 77.6 -> 76.1 us, T = 512 117.9 -> 115.6 us; with four blocks the
    // extra registers cost a wave per SIMD (T = 1024 +2 %), so 64-slot segments keep the plain order.
    auto compute32 = [&](const MoeMmStage<2>& s_, int buf) {
        const _Float16* xb = xs + buf * (ROWS * MOE_LDX) + c * MOE_LDX + q * 8;
        const f4_t zero = {0.f, 0.f, 0.f, 0.f};
        h8_t b[TT];
#pragma unroll
        for (int tt = 0; tt < TT; tt++) b[tt] = *reinterpret_cast<const h8_t*>(xb + tt * 16 * MOE_LDX);
        h8_t a = w4_deq8(s_.q[0][0]);
        auto group = [&](auto gc) {
            constexpr int g = decltype(gc)::value, w = g >> 1, rb = g & 1;
            f4_t p[TT];
#pragma unroll
            for (int tt = 0; tt < TT; tt++) p[tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b[tt], zero, 0, 0, 0);
            if constexpr (TT == 1) asm volatile("" : "+v"(p[0]));
            if constexpr (TT == 2) asm volatile("" : "+v"(p[0]), "+v"(p[1]));
            if constexpr (TT == 3) asm volatile("" : "+v"(p[0]), "+v"(p[1]), "+v"(p[2]));
            if constexpr (TT == 4) asm volatile("" : "+v"(p[0]), "+v"(p[1]), "+v"(p[2]), "+v"(p[3]));
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (g < 7) {
                constexpr int w2 = (g + 1) >> 1, rb2 = (g + 1) & 1;
                if constexpr (w2 != w) {
#pragma unroll
                    for (int tt = 0; tt < TT; tt++) b[tt] = *reinterpret_cast<const h8_t*>(xb + tt * 16 * MOE_LDX + w2 * 32);
                }
                a = w4_deq8(s_.q[rb2][w2]);
                asm volatile("" : "+v"(a));
            }
            __builtin_amdgcn_sched_barrier(0);
            const f4_t sc = moe_scale4<G, SBF, w>(s_.s[rb]);
#pragma unroll
            for (int tt = 0; tt < TT; tt++) acc[rb][tt] = w4_fma4(sc, p[tt], acc[rb][tt]);
#pragma unroll
            for (int tt = 0; tt < TT; tt++) asm volatile("" : "+v"(acc[rb][tt]));
            __builtin_amdgcn_sched_barrier(0);
        };
        group(std::integral_constant<int, 0>{});
        group(std::integral_constant<int, 1>{});
        group(std::integral_constant<int, 2>{});
        group(std::integral_constant<int, 3>{});
        group(std::integral_constant<int, 4>{});
        group(std::integral_constant<int, 5>{});
        group(std::integral_constant<int, 6>{});
        group(std::integral_constant<int, 7>{});
    };

    // prologue: the slice's first x tile into LDS buffer 0, the second in registers (both loads issued before the first
    // is stored: the first tile's registers are free again before the accumulators are live), DEPTH weight stages in
    // flight
    {
        u4_t first[TT];
        load_x(first, kt_lo);
        load_x(xreg, kt_lo + 1);
#pragma unroll
        for (int d = 0; d < DEPTH; d++) load_w(stage[d], kt_lo + d);
        store_x(first, 0);
    }
    __syncthreads();
    int xb = 0;  // LDS buffer of the tile being multiplied
    for (int kt0 = kt_lo; kt0 < kt_hi; kt0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            const int kt = kt0 + d;
            // a wave that holds a landed tile issues ahead of the waves that are queueing loads (about 1 % at every T)
            __builtin_amdgcn_s_setprio(1);
            if (kt < kt_hi) {
                if constexpr (G == 32 && TT <= 3) compute32(stage[d], xb);
                else compute(stage[d], xb);
            }
            __builtin_amdgcn_s_setprio(0);
            load_w(stage[d], kt + DEPTH);
            store_x(xreg, xb ^ 1);  // tile kt+1, loaded an iteration ago, into the buffer tile kt-1 was read from
            load_x(xreg, kt + 2);   // out of range past the last tile: zeros, no traffic
            __syncthreads();
            xb ^= 1;
        }
    }

    if (!active) return;
    if (KS && nks > 1) {
        // every wave on its own: park the partial tiles (device-scope stores), draw the (block, wave) ticket, and the
        // wave that draws the last one adds the slices in slice order and stores.  The hand-over is the one of the
        // dense decode kernel (decode.hip): write-through stores completed before the agent-scope ticket atomic,
        // cache-bypassing loads behind an agent-scope acquire fence in the wave that drew the last ticket; the slice
        // offset travels in the vector offset (scalar offset 0) so that the compiler inserts the wait state a write to
        // the data registers of a 16-byte store needs, and the tiles stay live until the stores have completed.
        constexpr unsigned PER_WAVE = 2u * TTMAX * 1024u;
        const unsigned per_slice = gridDim.x * (unsigned)W * PER_WAVE;
        const __amdgpu_buffer_rsrc_t wr = w4_make_rsrc(ws, per_slice * (unsigned)nks);
        const unsigned mine = (blockIdx.x * (unsigned)W + (unsigned)wave) * PER_WAVE + (unsigned)lane * 16u;
        const unsigned park = mine + (unsigned)ky * per_slice;
        constexpr int DEV = 16;  // cache policy: device scope
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
            for (int tt = 0; tt < TT; tt++)
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4_t, acc[rb][tt]), wr,
                                                       park + (unsigned)(rb * TT + tt) * 1024u, 0, DEV);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
            for (int tt = 0; tt < TT; tt++) asm volatile("" ::"v"(acc[rb][tt]));
        int ticket = 0;
        int* const tk = tickets + blockIdx.x * W + wave;
        if (lane == 0) ticket = __hip_atomic_fetch_add(tk, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ticket = __builtin_amdgcn_readfirstlane(ticket);
        if (ticket != nks - 1) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
            for (int tt = 0; tt < TT; tt++) {
                f4_t part[MOE_MAX_KSPLIT];  // all slices in flight at once; slices past nks: zero-length descriptor, zeros
#pragma unroll
                for (int s_ = 0; s_ < MOE_MAX_KSPLIT; s_++)
                    part[s_] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                                            s_ < nks ? wr : w4_make_rsrc(ws, 0u),
                                                            mine + (unsigned)(rb * TT + tt) * 1024u, s_ * per_slice, DEV));
                f4_t sum = part[0];
#pragma unroll
                for (int s_ = 1; s_ < MOE_MAX_KSPLIT; s_++) sum += part[s_];
                acc[rb][tt] = sum;
            }
        if (lane == 0) __hip_atomic_store(tk, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        const int slot = sorted_ids[seg * blk + tt * 16 + c];
        if (slot >= ns) continue;
        const float wgt = (!GLU && topw) ? topw[slot] : 1.0f;
        moe_store<GLU>(acc[0][tt], acc[1][tt], slot, q, u, rbA, rbB, haveB, y, y_f16, wgt, n, act_kind);
    }
}

// A segment's slots are a prefix of it (the alignment pads an expert's run at its end), so the first slot of each
// 16-slot block tells whether the block holds any: the workgroup runs the body built for the blocks that do, and the
// MFMAs, scaled sums and x rows of all-padding blocks are never issued (128 experts, top-8, T = 512: runs of 32 +- 6
// slots in 48-slot segments, every other expert fills two blocks of three).
template <int G, bool SBF, bool GLU, int TT, int DEPTH, bool KS>
__device__ __forceinline__ void moe_mm_entry(MOE_PARAMS) {
    if constexpr (TT == 1) {
        moe_mm_body<G, SBF, GLU, 1, 1, DEPTH, KS>(MOE_ARGS);
    } else {
        const int units = GLU ? row_blocks >> 1 : (row_blocks + 1) >> 1;
        const int seg = blockIdx.x / ((units + wpb - 1) / wpb);
        int live = 1;
#pragma unroll
        for (int p = 1; p < TT; p++) live += sorted_ids[seg * blk + 16 * p] < ns ? 1 : 0;
        if (live == 1) moe_mm_body<G, SBF, GLU, 1, TT, DEPTH, KS>(MOE_ARGS);
        else if (TT == 2 || live == 2) moe_mm_body<G, SBF, GLU, 2, TT, DEPTH, KS>(MOE_ARGS);
        else if (TT == 3 || live == 3) moe_mm_body<G, SBF, GLU, TT >= 3 ? 3 : 2, TT, DEPTH, KS>(MOE_ARGS);
        else moe_mm_body<G, SBF, GLU, TT, TT, DEPTH, KS>(MOE_ARGS);
    }
}

#define MOE_DEC_KERNEL(NAME, G, SBF, GLU, XL, DEPTH)                                  \
    extern "C" __global__ __launch_bounds__(512) void NAME(MOE_PARAMS) {              \
        moe_dec_body<G, SBF, GLU, XL, DEPTH>(MOE_ARGS);                               \
    }
#define MOE_MM_KERNEL(NAME, G, SBF, GLU, TT, DEPTH, KS)                               \
    extern "C" __global__ __launch_bounds__(512) void NAME(MOE_PARAMS) {              \
        moe_mm_entry<G, SBF, GLU, TT, DEPTH, KS>(MOE_ARGS);                           \
    }
// Ring depths, from sweeps on the 128-expert shape: the one-slot segments of the direct mode run best with two k tiles
// in flight per wave (T = 4..12: 9-11 % faster than four: fewer registers, more waves resident at once); so do the
// segments of up to 16 slots (5 % faster than three).  The LDS-staged kernels keep two (group 32) or four (group 128);
// the LDS buffer of a k tile alternates on its own, whatever the ring depth.
#define MOE_FAMILY(PFX, G, SBF, DMM)                             \
    MOE_DEC_KERNEL(PFX##_dec_glu_x1, G, SBF, true, 1, 2)     \
    MOE_DEC_KERNEL(PFX##_dec_glu_x4, G, SBF, true, 4, 2)     \
    MOE_DEC_KERNEL(PFX##_dec_lin_x1, G, SBF, false, 1, 2)    \
    MOE_DEC_KERNEL(PFX##_dec_lin_x4, G, SBF, false, 4, 2)    \
    MOE_MM_KERNEL(PFX##_mm_glu_t1, G, SBF, true, 1, DMM, false)    \
    MOE_MM_KERNEL(PFX##_mm_glu_t2, G, SBF, true, 2, DMM, false)    \
    MOE_MM_KERNEL(PFX##_mm_glu_t3, G, SBF, true, 3, DMM, false)    \
    MOE_MM_KERNEL(PFX##_mm_glu_t4, G, SBF, true, 4, DMM, false)    \
    MOE_MM_KERNEL(PFX##_mm_lin_t1, G, SBF, false, 1, DMM, false)   \
    MOE_MM_KERNEL(PFX##_mm_lin_t2, G, SBF, false, 2, DMM, false)   \
    MOE_MM_KERNEL(PFX##_mm_lin_t3, G, SBF, false, 3, DMM, false)   \
    MOE_MM_KERNEL(PFX##_mm_lin_t4, G, SBF, false, 4, DMM, false)   \
    MOE_MM_KERNEL(PFX##_mm_lin_t1_ks, G, SBF, false, 1, DMM, true) \
    MOE_MM_KERNEL(PFX##_mm_lin_t2_ks, G, SBF, false, 2, DMM, true) \
    MOE_MM_KERNEL(PFX##_mm_lin_t3_ks, G, SBF, false, 3, DMM, true) \
    MOE_MM_KERNEL(PFX##_mm_lin_t4_ks, G, SBF, false, 4, DMM, true)

#ifndef MOE_G32_DEPTH
#define MOE_G32_DEPTH 2
#endif
MOE_FAMILY(w4a16_moe_g32_f16, 32, false, MOE_G32_DEPTH)
MOE_FAMILY(w4a16_moe_g32_bf16, 32, true, MOE_G32_DEPTH)
MOE_FAMILY(w4a16_moe_g128_f16, 128, false, 4)
MOE_FAMILY(w4a16_moe_g128_bf16, 128, true, 4)

// ---------------------------------------------------------------------------------------------------- routing
// Routing rule of the reference (w4a16_dec/mod.rs:168-185, device counterpart assets/moe.cu:686-759): softmax over all
// experts, the k largest probabilities with ties to the lower index, weights renormalised by the selected sum.
// One wave per token, n <= 1024 (16 experts per lane).  Selection runs on ONE unique, totally ordered 64-bit key per
// expert — the probability's bit pattern (monotone for non-negative floats) above the complement of the expert index —
// so "larger probability, then lower index" is a plain unsigned maximum: a round takes the lane's largest key, a
// butterfly of unsigned maxima over the wave, and retires the winner by comparing keys (0 = absent or taken; no real
// key is 0 because index complements are non-zero).
__device__ __forceinline__ unsigned long long topk_wave_max(unsigned long long v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned lo = __shfl_xor((unsigned)v, off), hi = __shfl_xor((unsigned)(v >> 32), off);
        const unsigned long long o = ((unsigned long long)hi << 32) | lo;
        v = o > v ? o : v;
    }
    return v;
}

extern "C" __global__ __launch_bounds__(256) void w4a16_moe_topk_t(const float* __restrict__ lg, int* __restrict__ idx,
                                                                   float* __restrict__ wt, int t, int n, int k) {
    constexpr int PER_LANE = 16;
    const int lane = threadIdx.x & 63;
    const int token = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (token >= t) return;
    const float* logits = lg + (size_t)token * n;
    float e[PER_LANE];
    float top = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER_LANE; j++) {
        const int i = lane + 64 * j;
        e[j] = i < n ? logits[i] : -INFINITY;
        top = fmaxf(top, e[j]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) top = fmaxf(top, __shfl_xor(top, off));
    float total = 0.f;
#pragma unroll
    for (int j = 0; j < PER_LANE; j++) {
        e[j] = lane + 64 * j < n ? expf(e[j] - top) : 0.f;
        total += e[j];  // lane-local sum in index order, then the butterfly: the order the host statement follows too
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) total += __shfl_xor(total, off);
    unsigned long long key[PER_LANE];
#pragma unroll
    for (int j = 0; j < PER_LANE; j++) {
        const unsigned i = (unsigned)(lane + 64 * j);
        const float p = e[j] / total;
        key[j] = i < (unsigned)n ? ((unsigned long long)__builtin_bit_cast(unsigned, p) << 32) | (unsigned long long)(~i) : 0ull;
    }
    float chosen_sum = 0.f, kept = 0.f;  // lane r keeps the r-th chosen probability (k <= 64)
    for (int r = 0; r < k; r++) {
        unsigned long long best = 0ull;
#pragma unroll
        for (int j = 0; j < PER_LANE; j++) best = key[j] > best ? key[j] : best;
        best = topk_wave_max(best);
#pragma unroll
        for (int j = 0; j < PER_LANE; j++) key[j] = key[j] == best ? 0ull : key[j];
        const float p = __builtin_bit_cast(float, (unsigned)(best >> 32));
        if (lane == 0) idx[(size_t)token * k + r] = (int)(~(unsigned)best);
        kept = lane == r ? p : kept;
        chosen_sum += p;
    }
    if (lane < k) wt[(size_t)token * k + lane] = kept / chosen_sum;
}

// Stable counting sort of slots by expert with every expert's run padded to a multiple of `block`
// (assets/moe.cu:860-908 + 1599-1633 in one launch).  One workgroup of 1024 threads, n_exp <= 1024.
//   sorted_ids: slot ids in expert order, padding = sentinel ns; expert_ids[b]: expert of segment b;
//   num_post[0] = padded total, num_post[1] = number of distinct experts hit.
// Wave w owns the contiguous slot range [w*chunk, (w+1)*chunk): per-wave counts, an exclusive prefix over the
// waves per expert, a two-level scan over the experts' padded counts, then every wave places its slots in order.
// An out-of-range expert id is dropped (its slot is never placed).
#define MOE_ALIGN_WAVES 16
#define MOE_ALIGN_THREADS (64 * MOE_ALIGN_WAVES)
#define MOE_ALIGN_KEEP 4  // 64-slot steps of a wave whose expert ids stay in registers between the two passes
extern "C" __global__ __launch_bounds__(MOE_ALIGN_THREADS) void w4a16_moe_align(const int* __restrict__ idx, int ns,
                                                                               int n_exp, int block,
                                                                               int* __restrict__ sorted_ids,
                                                                               int* __restrict__ expert_ids,
                                                                               int* __restrict__ num_post) {
    extern __shared__ unsigned align_lds[];  // cnt[WAVES][n_exp] (per wave count, then exclusive prefix over the waves),
                                             // tot[n_exp], poff[n_exp]
    unsigned* const cnt = align_lds;
    unsigned* const tot = cnt + MOE_ALIGN_WAVES * n_exp;
    unsigned* const poff = tot + n_exp;
    __shared__ unsigned wsum[MOE_ALIGN_WAVES], whit[MOE_ALIGN_WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < MOE_ALIGN_WAVES * n_exp; i += MOE_ALIGN_THREADS) cnt[i] = 0;
    const int chunk = ((ns + MOE_ALIGN_WAVES * 64 - 1) / (MOE_ALIGN_WAVES * 64)) * 64;  // slots per wave, multiple of 64
    const int j0 = wave * chunk, steps = chunk / 64;
    int keep[MOE_ALIGN_KEEP];
#pragma unroll
    for (int s = 0; s < MOE_ALIGN_KEEP; s++) {
        const int j = j0 + s * 64 + lane;
        int e = (s < steps && j < ns) ? idx[j] : -1;
        keep[s] = (unsigned)e < (unsigned)n_exp ? e : -1;
    }
    auto expert_of = [&](int s) -> int {
        int e = -1;
#pragma unroll
        for (int i = 0; i < MOE_ALIGN_KEEP; i++)
            if (i == s) e = keep[i];
        if (s >= MOE_ALIGN_KEEP) {
            const int j = j0 + s * 64 + lane;
            e = j < ns ? idx[j] : -1;
            if ((unsigned)e >= (unsigned)n_exp) e = -1;
        }
        return e;
    };
    __syncthreads();
    for (int s = 0; s < steps; s++) {
        const int e = expert_of(s);
        if (e >= 0) atomicAdd(&cnt[wave * n_exp + e], 1u);
    }
    __syncthreads();
    // thread i owns expert i: total over the waves, then a scan of the padded totals over all threads
    unsigned padded = 0, hits = 0;
    {
        const int e = tid;
        unsigned run = 0;
        if (e < n_exp) {
            for (int w = 0; w < MOE_ALIGN_WAVES; w++) {
                const unsigned c = cnt[w * n_exp + e];
                cnt[w * n_exp + e] = run;
                run += c;
            }
            tot[e] = run;
        }
        padded = ((run + block - 1) / block) * block;
        hits = run != 0;
    }
    unsigned incl = padded, hincl = hits;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned v = __shfl_up(incl, off), hv = __shfl_up(hincl, off);
        if (lane >= off) {
            incl += v;
            hincl += hv;
        }
    }
    if (lane == 63) {
        wsum[wave] = incl;
        whit[wave] = hincl;
    }
    __syncthreads();
    unsigned base = 0, all = 0, allhit = 0;
#pragma unroll
    for (int w = 0; w < MOE_ALIGN_WAVES; w++) {
        if (w < wave) base += wsum[w];
        all += wsum[w];
        allhit += whit[w];
    }
    const unsigned pos0 = base + incl - padded;
    if (tid < n_exp) poff[tid] = pos0;
    // every position gets the padding sentinel first, coalesced; the slots are placed over it after the barrier (a
    // workgroup barrier waits for the stores issued before it, so the order of the two writes to a position is fixed)
    for (unsigned p = tid; p < all; p += MOE_ALIGN_THREADS) sorted_ids[p] = ns;
    if (tid < n_exp)
        for (unsigned b = 0; b < padded / block; b++) expert_ids[pos0 / block + b] = tid;
    if (tid == 0) {
        num_post[0] = (int)all;
        num_post[1] = (int)allhit;
    }
    __syncthreads();
    // placement in slot order: every wave walks its range 64 slots at a time; rank among equal experts in the step.
    // The wave's row of cnt is private to it and LDS operations of one wave execute in order, so the loop needs no
    // workgroup barrier; the wave-scope fences keep the compiler from reordering the LDS accesses.
    int nbits = 1;  // bits that tell experts 0..n_exp-1 apart; the bit above them tells a dropped slot (-1) from all
    while ((1 << nbits) < n_exp) nbits++;
    for (int s = 0; s < steps; s++) {
        const int e = expert_of(s);
        // lanes of the step with this lane's expert: one ballot per bit of the expert id, each lane keeps the side
        // of the ballot its own bit is on (a dropped slot, e = -1, matches only other dropped slots and is not placed)
        unsigned long long peers = ~0ull;
        for (int bit = 0; bit <= nbits; bit++) {
            const bool on = (e >> bit) & 1;
            const unsigned long long bal = __ballot(on);
            peers &= on ? bal : ~bal;
        }
        const unsigned same = (unsigned)__popcll(peers);
        const unsigned rank = __builtin_amdgcn_mbcnt_hi((unsigned)(peers >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)peers, 0u));
        unsigned before = 0;
        if (e >= 0) before = cnt[wave * n_exp + e];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (e >= 0) {
            sorted_ids[poff[e] + before + rank] = j0 + s * 64 + lane;
            if (rank + 1 == same) cnt[wave * n_exp + e] = before + same;
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}

// out[t][c] = sum over the token's k slots of f16 c2[slot][c], added in slot order in f32 (assets/moe.cu:1662-1674).
// Eight columns per thread when h % 8 == 0 (16-byte loads), one otherwise.
extern "C" __global__ __launch_bounds__(256) void w4a16_moe_topk_sum_f16(const uint16_t* __restrict__ c2,
                                                                         float* __restrict__ out, int t, int h, int top_k) {
    if ((h & 7) == 0) {
        const size_t total = (size_t)t * h / 8;
        for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
            const size_t r = (i * 8) / h, c = (i * 8) % h;
            float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            for (int kk = 0; kk < top_k; kk++) {
                const h8_t v = *reinterpret_cast<const h8_t*>(c2 + (r * top_k + kk) * h + c);
#pragma unroll
                for (int j = 0; j < 8; j++) acc[j] += (float)v[j];
            }
            f4_t* o = reinterpret_cast<f4_t*>(out + i * 8);
            o[0] = (f4_t){acc[0], acc[1], acc[2], acc[3]};
            o[1] = (f4_t){acc[4], acc[5], acc[6], acc[7]};
        }
        return;
    }
    const size_t total = (size_t)t * h;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / h, c = i % h;
        float acc = 0.f;
        for (int kk = 0; kk < top_k; kk++)
            acc += (float)__builtin_bit_cast(_Float16, c2[(r * top_k + kk) * h + c]);
        out[i] = acc;
    }
}
