// Prefill regime (t > 16 activation rows): tiled GEMM  y[t][n] = x[t][k] * W^T  on v_mfma_f32_32x32x16_f16.
// Role of the reference's prefill path gemm_launch -> marlin_gemm_try / w4a16_gemm_g128_mma
// (w4a16_dec/kernels/gemm.rs:4-51, kernels/marlin.rs:94-213, assets/gptq4.cu:984-1147), designed for CDNA4:
//   * workgroup = 4 waves along n, block tile 128 (m) x 256 (n), wave tile 128 x 64 = 4 x 2 MFMA tiles of 32 x 32 with
//     f32 accumulators in arch VGPRs (128 registers); two workgroups per CU, so one block's barriers and LDS writes
//     overlap the other's MFMAs;
//   * x (the A operand) is staged through LDS in k slabs of 64, double buffered, by LDS DMA (buffer_load ... lds:
//     no staging registers, no ds_write); rows are unpadded and their 16-byte chunks swizzled by row so the
//     ds_read_b128 fragment reads are bank-conflict free; rows >= t come from out-of-range loads (zeros);
//   * the weights (B operand) never touch LDS: the tiled layout of w4a16_common.hpp already is the MFMA B layout —
//     lane (n = l % 32, khalf = l / 32) reads 16 B of tile lane g = 2h + khalf, r = n % 16 of its row block, dword w of
//     which is the k16 block (w, h) of the k tile — so each wave fetches its 64 x 128 weights with four coalesced
//     dwordx4 loads per k tile (one k tile ahead) and unpacks them in registers (9 VALU ops per MFMA operand);
//   * weights enter the MFMA as exact integers.  The per-group scale is carried as a running unit: the accumulator
//     holds sum / s_g; at each group boundary it is multiplied by s_prev / s_cur and the new group's integer products
//     are added by the MFMA itself; the epilogue multiplies by the last scale.  No weight is rounded to f16 and no
//     second accumulator set is needed.  (Linears with a zero or non-finite scale are not routed here.)
//   * workgroups are numbered so that the blocks resident on one XCD form a super-tile (8 x 8 block tiles on large
//     grids: each x slab and each weight panel is fetched into that L2 once per eight uses; smaller on small grids so
//     that all eight XCDs get work).
#include "w4a16_common.hpp"

// s_prev / s_cur of a group boundary: the hardware reciprocal (1 ulp) and one Newton step on the quotient (the residual
// s_prev - q * s_cur is exact in a fused multiply-add), which leaves the quotient within about half an ulp.  The
// accumulators are re-expressed with this factor once per scale group, so its error enters every output once per
// group: with the bare reciprocal the kernel's distance from the exact dot product was several times that of the f32
// lane order at k = 17408 (136 groups); with the corrected quotient it is of the same size.  Three instructions per scale
// instead of the ten of an IEEE division (+2 % at group 128, +4.5 % at group 32 at M = 4096 for the division).
__device__ __forceinline__ float pf_ratio(float s_prev, float s_cur) {
    const float r = __builtin_amdgcn_rcpf(s_cur);
    const float q = s_prev * r;
    return __builtin_fmaf(__builtin_fmaf(-q, s_cur, s_prev), r, q);
}

#define PF_BN 256
#define PF_KS 64          // k per LDS stage
#define PF_LDA 64         // halves per staged x row (unpadded; chunks swizzled)
#define PF_THREADS 256

// MI = 32-row MFMA tiles along m per wave: 4 (block tile 128 x 256, 128 accumulator registers, two workgroups per CU) or
// 2 (64 x 256, 64 registers, three workgroups per CU) for a few dozen to a couple of hundred rows, where 128-row tiles
// would spend half their MFMAs on padding and leave too few workgroups.
//
// Grouped form for the expert FFN (MODE 1, 2): the role of the reference's grouped Marlin GEMM at prefill sizes
// (assets/moe.cu:686-759 via kernels/marlin_moe.rs:290-422).  The rows of a block tile are one 64-slot segment of the
// alignment pass (sorted_ids, padded with the sentinel ns; expert_ids per segment; num_post = padded slot total), the
// weights are those of the segment's expert in its arena, x rows are gathered by slot id (slot j reads row j / x_div)
// straight into the LDS stage by the same DMA, and the epilogue scatters by slot id:
//   MODE 1 (gate|up, n = 2 n_ff): a wave's two 32-column sub-tiles are gate columns c.. and up columns n_ff + c.., so
//     the lane that holds a gate sum holds the matching up sum; both are rounded to f16 (the reference materialises
//     them as f16) and act[slot][c] = f16(act(gate) * up) is written, f16 [ns][n_ff];
//   MODE 2 (down, n = hidden): y[slot][c] = sum * topw[slot] as f16 or f32 [ns][n].
//
// Dense gated form (MODE 3): a fused gate|up linear (rows 0..n/2 gate, n/2..n up) with the element-wise kernel that
// follows it in the reference's prefill chain (lin_forward + ew, w4a16_dec/prefill.rs:148-207, assets/ew.cu:9-57)
// folded into the epilogue: column pairing as in MODE 1, tile numbering and split-K as in MODE 0, and
// y[m][c] = f16(act(g) * u) on the f32 sums g, u (f16 [t][n/2]) — the bits of the MODE 0 launch with f32 output
// followed by w4a16_act_mul_f16, without the [t][n] f32 round trip (285 of the 419 MB a 4096-row launch moves on the
// 27B gate|up shape).  A split launch writes f32 partials of all n columns and w4a16_prefill_splitk_sum applies the
// activation after adding them.
template <int MODE>
struct PfGroup {
    const int* sorted_ids;
    const int* expert_ids;
    const int* num_post;
    const float* topw;
    unsigned long long q_stride, s_stride;  // bytes per expert
    int ns, x_rows, x_div, n_exp, act_kind;
};

// Epilogue options of the dense kernels (MODE 0 and 3), the prefill-regime form of what the decode kernel does for a
// normalisation deferred across linears (the element-wise parts of the reference's norm_resid, assets/norm.cu:4-48,
// moved into the linears either side of it).  Every part is optional (a null pointer / 0 / 1.0 switches it off):
//   consumer side: stats_in [n_stats_in][ld_stats] are partial sums of squares of the INPUT rows left by the launch
//     that produced x; the output row m is multiplied by 1/sqrt(sum_e stats_in[e][m] * inv_cols_in + 1e-6) * in_scale
//     (in_scale = 2^e undoes the power-of-two factor x was handed over with); ldx = halves between x rows (0 = k);
//   producer side: resid f32 [t][n] takes the output (v = resid + y, written back); stats_out[(tile_n*4 + wave)][m]
//     receives this wave's partial sum of v^2 over its columns below stat_cols (one entry per wave and block tile
//     column, no atomics); nw f32 [n] multiplies what y receives; out_scale = 2^-e is applied last.
struct PfEpi {
    const float* stats_in;
    float* stats_out;
    float* resid;
    const float* nw;
    int n_stats_in, ld_stats, stat_cols, ldx;
    float inv_cols_in, in_scale, out_scale;
};

template <int G, bool SBF, int MI, int MODE = 0>
__device__ __forceinline__ void prefill_body(const u4_t* __restrict__ qt, const uint16_t* __restrict__ st,
                                             const uint16_t* __restrict__ x, void* __restrict__ y, int row_blocks,
                                             int k, int n, int t, int out_f16, int sup_m, int sup_n,
                                             const PfGroup<MODE> gp = PfGroup<MODE>(), const PfEpi epi = PfEpi()) {
    extern __shared__ _Float16 lds[];  // 2 stages x [PF_BM][PF_LDA]; then PF_BM ints: slot ids (grouped) / row factors (dense)
    constexpr int GPT = W4_TILE_K / G;
    constexpr int PF_BM = 32 * MI, PF_STAGE_BYTES = PF_BM * PF_LDA * 2;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave;  // 4 waves along n
    const int kt_n = k / W4_TILE_K, kg_n = kt_n * GPT;

    // XCD-aware tile numbering.  Block b runs on XCD b % 8 and is the (b / 8)-th block of that XCD; consecutive
    // blocks of an XCD walk one super-tile of sup_m x sup_n block tiles (m fastest), so the blocks resident on an XCD
    // at a time share x slabs and weight panels through its L2.  Super-tiles are dealt round-robin to the XCDs.  The
    // host picks the super-tile shape: 8 x 8 on large grids, smaller on small ones so that every XCD gets work.
    int m0, n0;
    constexpr bool DENSE = MODE == 0 || MODE == 3, PAIRED = MODE == 1 || MODE == 3;  // PAIRED: gate and up columns per wave
    if (DENSE) {
        const int tiles_m = (t + PF_BM - 1) / PF_BM,
                  tiles_n = MODE == 3 ? ((n >> 1) + PF_BN / 2 - 1) / (PF_BN / 2) : (n + PF_BN - 1) / PF_BN;
        const int sm_n = (tiles_m + sup_m - 1) / sup_m, sn_n = (tiles_n + sup_n - 1) / sup_n;
        const int per = sup_m * sup_n;
        const int j = blockIdx.x >> 3;
        const int super = (blockIdx.x & 7) + 8 * (j / per), within = j % per;
        if (super >= sm_n * sn_n) return;  // uniform for the whole block
        const int tm = (super % sm_n) * sup_m + within % sup_m, tn = (super / sm_n) * sup_n + within / sup_m;
        if (tm >= tiles_m || tn >= tiles_n) return;
        m0 = tm * PF_BM;
        n0 = tn * (MODE == 3 ? PF_BN / 2 : PF_BN);
    } else {
        // grouped: blockIdx.x = column tile (fastest, so the tiles of a segment run together and share its x rows
        // through the L2), blockIdx.y = segment.  Gate|up tiles span 128 gate and the 128 matching up columns.
        const int seg = blockIdx.y;
        m0 = seg * PF_BM;  // position in sorted_ids
        if (m0 >= gp.num_post[0]) return;
        const int e = gp.expert_ids[seg];
        if ((unsigned)e >= (unsigned)gp.n_exp) return;
        qt = reinterpret_cast<const u4_t*>(reinterpret_cast<const char*>(qt) + (size_t)e * gp.q_stride);
        st = reinterpret_cast<const uint16_t*>(reinterpret_cast<const char*>(st) + (size_t)e * gp.s_stride);
        n0 = blockIdx.x * (MODE == 1 ? PF_BN / 2 : PF_BN);
    }

    const unsigned ldx = DENSE && epi.ldx ? (unsigned)epi.ldx : (unsigned)k;  // halves between x rows
    const __amdgpu_buffer_rsrc_t xr = w4_make_rsrc(x, DENSE ? ((unsigned)(t - 1) * ldx + (unsigned)k) * 2u : (unsigned)gp.x_rows * (unsigned)k * 2u);
    const __amdgpu_buffer_rsrc_t qr = w4_make_rsrc(qt, (unsigned)row_blocks * (unsigned)kt_n * 1024u);
    const __amdgpu_buffer_rsrc_t sr = w4_make_rsrc(st, (unsigned)row_blocks * (unsigned)kg_n * 32u);

    // ---- x staging by LDS DMA (buffer_load ... lds: global -> LDS without passing through registers).  A stage is
    // PF_BM rows x 64 k = PF_BM * 8 chunks of 16 B, 4 per thread; one instruction of a wave fills 1 KiB of LDS, lane i
    // at byte 16*i, so rows are 128 B apart without padding.  To keep the fragment reads conflict free the chunks of a
    // row are stored swizzled: chunk position p of row r holds k chunk p ^ (r & 7) — the lane that fills position p
    // simply fetches that k chunk.  Rows >= t fetch out of range: zeros.
    typedef __attribute__((address_space(3))) char lds_char_t;
    lds_char_t* const lds_base = (lds_char_t*)lds;
    unsigned xa_off[MI];  // PF_BM * 8 chunks over 256 threads
#pragma unroll
    for (int i = 0; i < MI; i++) {
        const int c = tid + i * PF_THREADS, row = c >> 3, kc = (c & 7) ^ (row & 7);
        if (DENSE) {
            xa_off[i] = (m0 + row < t) ? ((unsigned)(m0 + row) * ldx + (unsigned)kc * 8u) * 2u : W4_OOB;
        } else {
            const int id = gp.sorted_ids[m0 + row];  // padding rows carry the sentinel ns: zeros, never stored
            xa_off[i] = id < gp.ns ? ((unsigned)(id / gp.x_div) * (unsigned)k + (unsigned)kc * 8u) * 2u : W4_OOB;
        }
    }
    int* const seg_ids = reinterpret_cast<int*>(lds_base + 2 * PF_STAGE_BYTES);
    if (!DENSE && tid < PF_BM) seg_ids[tid] = gp.sorted_ids[m0 + tid];  // visible after the first barrier
    // Dense, input statistics given: the 1/rms factor of this block's PF_BM input rows, once, into the same LDS words
    // (thread r < PF_BM owns row m0 + r: entries added in index order with eight loads in flight — the same bits on
    // every run; consecutive threads read consecutive floats of an entry).  Read back in the epilogue.
    float* const row_fac = reinterpret_cast<float*>(lds_base + 2 * PF_STAGE_BYTES);
    if (DENSE && epi.stats_in != nullptr && tid < PF_BM) {
        const int row = m0 + tid;
        float sum = 0.f;
        if (row < t) {
            const float* sp = epi.stats_in + row;
            int e = 0;
            for (; e + 8 <= epi.n_stats_in; e += 8) {
                float v[8];
#pragma unroll
                for (int j = 0; j < 8; j++) v[j] = sp[(size_t)(e + j) * epi.ld_stats];
#pragma unroll
                for (int j = 0; j < 8; j++) sum += v[j];
            }
            for (; e < epi.n_stats_in; e++) sum += sp[(size_t)e * epi.ld_stats];
        }
        row_fac[tid] = (float)(1.0 / sqrt((double)sum * (double)epi.inv_cols_in + 1e-6)) * epi.in_scale;
    }
    auto load_a = [&](int s, int buf) {
#pragma unroll
        for (int i = 0; i < MI; i++)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                xr, (__attribute__((address_space(3))) void*)(lds_base + buf * PF_STAGE_BYTES + (i * PF_THREADS + wave * 64) * 16),
                16, xa_off[i], s * (PF_KS * 2), 0, 0);
    };

    // ---- weights: lane (nl = l % 32, khalf = l / 32); per n sub-tile ni and half h one dwordx4 per k tile
    const int nl = lane & 31, khalf = lane >> 5;
    unsigned q_off[2][2], s_off[2];
#pragma unroll
    for (int ni = 0; ni < 2; ni++) {
        const int nrow = PAIRED ? ni * (n >> 1) + n0 + wn * 32 + nl : n0 + wn * 64 + ni * 32 + nl;
        const unsigned rb = (unsigned)min(nrow >> 4, row_blocks - 1);  // rows past n re-read the last block, never stored
        const unsigned r = (unsigned)(nrow & 15);
#pragma unroll
        for (int h = 0; h < 2; h++) q_off[ni][h] = (rb * (unsigned)kt_n * 64u + (unsigned)(2 * h + khalf) * 16u + r) * 16u;
        s_off[ni] = (rb * (unsigned)kg_n * 16u + r) * 2u;
    }
    u4_t bq[2][2], bqn[2][2];
    unsigned sc[2][GPT], scn[2][GPT];
    auto load_b = [&](u4_t (&dst)[2][2], unsigned (&sdst)[2][GPT], int kt) {
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
#pragma unroll
            for (int h = 0; h < 2; h++)
                dst[ni][h] = __builtin_amdgcn_raw_buffer_load_b128(qr, q_off[ni][h], kt * 1024, 0);  // k tile in the scalar offset
#pragma unroll
            for (int gi = 0; gi < GPT; gi++)
                sdst[ni][gi] = __builtin_amdgcn_raw_buffer_load_b16(sr, s_off[ni], (kt * GPT + gi) * 32, 0);
        }
    };

    f16_t acc[MI][2];
#pragma unroll
    for (int mi = 0; mi < MI; mi++)
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[mi][ni][e] = 0.f;
    float unit[2] = {1.f, 1.f};  // scale the accumulator of sub-tile ni is currently expressed in

    const int a_row = nl;  // + mi * 32
    // split-K over gridDim.y (narrow outputs at moderate t, where the tile grid alone cannot fill the chip): this
    // block covers k tiles [kt_lo, kt_hi) and writes an f32 partial; a second launch adds the partials in order
    const int kt_lo = DENSE ? (kt_n * (int)blockIdx.y) / (int)gridDim.y : 0,
              kt_hi = DENSE ? (kt_n * ((int)blockIdx.y + 1)) / (int)gridDim.y : kt_n;
    const int stages = 2 * kt_hi;
    constexpr bool PF_WAVE_PRIO = G == 128;  // wave priority over a stage's MFMAs (see the k loop)

    load_a(2 * kt_lo, 0);
    load_b(bq, sc, kt_lo);
    __syncthreads();  // the compiler waits for the LDS DMA (vmcnt) ahead of the barrier

    for (int kt = kt_lo; kt < kt_hi; kt++) {
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const int s = kt * 2 + half;
            // stage s+1 goes into the buffer that stage s-1 was read from: every wave is past the barrier that ended it
            if (s + 1 < stages) load_a(s + 1, (s + 1) & 1);
            if (half == 0 && kt + 1 < kt_hi) load_b(bqn, scn, kt + 1);
            const _Float16* abuf = lds + (s & 1) * (PF_BM * PF_LDA) + a_row * PF_LDA;
#pragma unroll
            for (int kbl = 0; kbl < 4; kbl++) {
                const int kb = half * 4 + kbl, w = kb >> 1, h = kb & 1;
                // Group boundary: re-express the accumulators in the next group's scale.
                //   group 128: the multiply is done at the END of a k tile, tile by tile right after each tile's last
                //   MFMA of the group, with the scale of the next k tile (already loaded), so the VALU work of tile j
                //   runs in the shadow of the MFMAs of tiles j+1.. instead of stalling the next stage's first MFMAs;
                //   group 32: at the first k16 of each 32-k group, before the tile's first MFMA.
                // Wave priority: raised while a stage's MFMAs issue, dropped for the accumulator rescale at the end of a
                // k tile, so that a wave in that VALU-only stretch yields the issue port to the waves that feed the
                // matrix pipe.  64- and 96-row tiles (three waves per SIMD): M = 512 186 -> 180 us, M = 1024 328 -> 317 us
                // on 5120 x 34816; 17408 x 5120 at M = 4096 630 -> 620 us.  128-row tile (two waves per SIMD), built with
                // the max-ILP scheduler: 5120 x 34816 at M = 4096 -0.5...-1.5 % on five boxes (with the default
                // scheduler the same lost 0.4-0.9 % on the faster boxes).  Group 32 rescales inside the stage and has no
                // such stretch.
                if (PF_WAVE_PRIO && kbl == 0) __builtin_amdgcn_s_setprio(1);
                const bool boundary32 = G == 32 && h == 0;
                float ratio[2] = {1.f, 1.f};
                if (boundary32) {
#pragma unroll
                    for (int ni = 0; ni < 2; ni++) {
                        const float s_cur = w4_scale_fast<SBF>(sc[ni][w]);
                        ratio[ni] = pf_ratio(unit[ni], s_cur);
                        unit[ni] = s_cur;
                    }
                }
                if (G == 128 && kb == 0 && kt == kt_lo) {  // the very first group: unit = its scale, accumulators are zero
#pragma unroll
                    for (int ni = 0; ni < 2; ni++) unit[ni] = w4_scale_fast<SBF>(sc[ni][0]);
                }
                h8_t a[MI];
#pragma unroll
                for (int mi = 0; mi < MI; mi++)
                    a[mi] = *reinterpret_cast<const h8_t*>(abuf + mi * 32 * PF_LDA + (((kbl * 2 + khalf) ^ (nl & 7)) * 8));
                const bool last128 = G == 128 && kb == 7;  // branch free: the last k tile multiplies by 1
                float next_ratio[2] = {1.f, 1.f};
                if (last128) {
                    const bool more = kt + 1 < kt_hi;
#pragma unroll
                    for (int ni = 0; ni < 2; ni++) {
                        const float s_next = more ? w4_scale_fast<SBF>(scn[ni][0]) : unit[ni];
                        next_ratio[ni] = pf_ratio(unit[ni], s_next);
                        unit[ni] = s_next;
                    }
                }
#pragma unroll
                for (int ni = 0; ni < 2; ni++) {
                    const h8_t b = w4_deq8(bq[ni][h][w]);
#pragma unroll
                    for (int mi = 0; mi < MI; mi++) {
                        if (boundary32) acc[mi][ni] *= ratio[ni];
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mi], b, acc[mi][ni], 0, 0, 0);
                    }
                }
                if (last128) {
                    if (PF_WAVE_PRIO) __builtin_amdgcn_s_setprio(0);
#pragma unroll
                    for (int ni = 0; ni < 2; ni++)
#pragma unroll
                        for (int mi = 0; mi < MI; mi++) acc[mi][ni] *= next_ratio[ni];
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
#pragma unroll
            for (int h = 0; h < 2; h++) bq[ni][h] = bqn[ni][h];
#pragma unroll
            for (int gi = 0; gi < GPT; gi++) sc[ni][gi] = scn[ni][gi];
        }
    }

    // ---- epilogue: y[m][n] = acc * unit; D register e of lane (nl, khalf) is row 8*(e/4) + 4*khalf + e%4, column nl
    if (MODE == 1) {
        const int n_ff = n >> 1, col = n0 + wn * 32 + nl;
        if (col >= n_ff) return;
#pragma unroll
        for (int mi = 0; mi < MI; mi++) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int slot = seg_ids[mi * 32 + 8 * (e >> 2) + 4 * khalf + (e & 3)];
                if (slot < gp.ns) {
                    const float gt = (float)(_Float16)(acc[mi][0][e] * unit[0]), up = (float)(_Float16)(acc[mi][1][e] * unit[1]);
                    reinterpret_cast<_Float16*>(y)[(size_t)slot * n_ff + col] = (_Float16)w4_act_mul(gt, up, gp.act_kind);
                }
            }
        }
        return;
    }
    if (MODE == 2) {
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            const int col = n0 + wn * 64 + ni * 32 + nl;
            if (col >= n) continue;
#pragma unroll
            for (int mi = 0; mi < MI; mi++) {
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int slot = seg_ids[mi * 32 + 8 * (e >> 2) + 4 * khalf + (e & 3)];
                    if (slot < gp.ns) {
                        float v = acc[mi][ni][e] * unit[ni];
                        if (gp.topw != nullptr) v *= gp.topw[slot];
                        if (out_f16)
                            reinterpret_cast<_Float16*>(y)[(size_t)slot * n + col] = (_Float16)v;
                        else
                            reinterpret_cast<float*>(y)[(size_t)slot * n + col] = v;
                    }
                }
            }
        }
        return;
    }
    // x arrived as its true value times 1/in_scale and (with input statistics) un-normalised: one factor per row
    const bool use_fac = DENSE && (epi.stats_in != nullptr || (epi.in_scale != 1.0f && epi.in_scale != 0.0f));
    if (MODE == 3 && gridDim.y == 1) {
        const int n_ff = n >> 1, col = n0 + wn * 32 + nl;
        if (col >= n_ff) return;
#pragma unroll
        for (int mi = 0; mi < MI; mi++) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int row = m0 + mi * 32 + 8 * (e >> 2) + 4 * khalf + (e & 3);
                if (row < t) {
                    float gt = acc[mi][0][e] * unit[0], up = acc[mi][1][e] * unit[1];
                    asm volatile("" : "+v"(gt), "+v"(up));  // the sums are rounded to f32 as the separate launch stores them
                    if (use_fac) {
                        const float f = epi.stats_in != nullptr ? row_fac[row - m0] : epi.in_scale;
                        gt *= f;
                        up *= f;
                    }
                    float v = w4_act_mul(gt, up, gp.act_kind);
                    asm volatile("" : "+v"(v));  // and the product before the f16 conversion, as in the separate kernel
                    if (epi.out_scale != 1.0f && epi.out_scale != 0.0f) {
                        v *= epi.out_scale;
                        asm volatile("" : "+v"(v));
                    }
                    reinterpret_cast<_Float16*>(y)[(size_t)row * n_ff + col] = (_Float16)v;
                }
            }
        }
        return;
    }
    if (gridDim.y > 1) {  // partial (f32) of a split launch: w4a16_prefill_splitk_sum finishes (activation, epilogue options)
        y = reinterpret_cast<float*>(y) + (size_t)blockIdx.y * (size_t)t * (size_t)n;
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            const int col = MODE == 3 ? ni * (n >> 1) + n0 + wn * 32 + nl : n0 + wn * 64 + ni * 32 + nl;
            if (MODE == 3 ? n0 + wn * 32 + nl >= (n >> 1) : col >= n) continue;
#pragma unroll
            for (int mi = 0; mi < MI; mi++) {
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int row = m0 + mi * 32 + 8 * (e >> 2) + 4 * khalf + (e & 3);
                    if (row < t) reinterpret_cast<float*>(y)[(size_t)row * n + col] = acc[mi][ni][e] * unit[ni];
                }
            }
        }
        return;
    }
    // MODE 0, whole k range: y = acc * unit, then the optional parts in the order of the decode kernel's epilogue — row
    // factor, residual stream, statistics of what continues, norm weight, power-of-two hand-over factor
    const bool plain = !use_fac && epi.resid == nullptr && epi.stats_out == nullptr && epi.nw == nullptr && (epi.out_scale == 1.0f || epi.out_scale == 0.0f);
#pragma unroll
    for (int mi = 0; mi < MI; mi++) {
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int row = m0 + mi * 32 + 8 * (e >> 2) + 4 * khalf + (e & 3);
            float p = 0.f;  // this lane's share of the row's sum of squares
            if (row < t) {
                const float f = !use_fac ? 1.0f : epi.stats_in != nullptr ? row_fac[row - m0] : epi.in_scale;
#pragma unroll
                for (int ni = 0; ni < 2; ni++) {
                    const int col = n0 + wn * 64 + ni * 32 + nl;
                    if (col >= n) continue;
                    float v = acc[mi][ni][e] * unit[ni];
                    if (!plain) {
                        asm volatile("" : "+v"(v));
                        if (use_fac) v *= f;
                        if (epi.resid != nullptr) {
                            float* const rp = epi.resid + (size_t)row * n + col;
                            v += *rp;
                            *rp = v;
                        }
                        if (col < epi.stat_cols) p = __builtin_fmaf(v, v, p);
                        if (epi.nw != nullptr) v *= epi.nw[col];
                        if (epi.out_scale != 1.0f && epi.out_scale != 0.0f) {
                            v *= epi.out_scale;
                            asm volatile("" : "+v"(v));  // rounded to f32 on its own, not fused into the f16 conversion
                        }
                    }
                    if (out_f16)
                        reinterpret_cast<_Float16*>(y)[(size_t)row * n + col] = (_Float16)v;
                    else
                        reinterpret_cast<float*>(y)[(size_t)row * n + col] = v;
                }
            }
            if (epi.stats_out != nullptr) {  // uniform: the 32 lanes of a row (same khalf) add up in a fixed order
#pragma unroll
                for (int off = 16; off > 0; off >>= 1) p += __shfl_xor(p, off);
                if (nl == 0 && row < t && n0 + wn * 64 < epi.stat_cols)
                    epi.stats_out[(size_t)((n0 + wn * 64) >> 6) * epi.ld_stats + row] = p;
            }
        }
    }
}

#define PREFILL_KERNEL(NAME, G, SBF, MI, WPE)                                                                      \
    extern "C" __global__ __launch_bounds__(PF_THREADS) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void NAME(      \
        const u4_t* qt, const uint16_t* st, const uint16_t* x, void* y, int row_blocks, int k, int n, int t,          \
        int out_f16, int sup_m, int sup_n, int act_kind, PfEpi epi) {                                                  \
        (void)act_kind;                                                                                                \
        prefill_body<G, SBF, MI>(qt, st, x, y, row_blocks, k, n, t, out_f16, sup_m, sup_n, PfGroup<0>(), epi);         \
    }

// Dense gated kernels: same arguments (the plain kernels ignore act_kind, W4A16_ACT_*); y is f16 [t][n/2], or the f32
// partials [slices][t][n] of a split launch.
#define PREFILL_GLU_KERNEL(NAME, G, SBF, MI, WPE)                                                                  \
    extern "C" __global__ __launch_bounds__(PF_THREADS) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void NAME(      \
        const u4_t* qt, const uint16_t* st, const uint16_t* x, void* y, int row_blocks, int k, int n, int t,          \
        int out_f16, int sup_m, int sup_n, int act_kind, PfEpi epi) {                                                  \
        PfGroup<3> gp;                                                                                                 \
        gp.act_kind = act_kind;                                                                                        \
        prefill_body<G, SBF, MI, 3>(qt, st, x, y, row_blocks, k, n, t, out_f16, sup_m, sup_n, gp, epi);                \
    }

// Grouped kernels for the expert FFN: same arguments as the streaming grouped kernels of moe.hip (blk must be 64, the
// rows of a block tile; ws, tickets and wpb are unused).
#define PREFILL_MOE_KERNEL(NAME, G, SBF, MODE)                                                                          \
    extern "C" __global__ __launch_bounds__(PF_THREADS) __attribute__((amdgpu_waves_per_eu(3, 3))) void NAME(            \
        const char* qa, const char* sa, unsigned long long q_stride, unsigned long long s_stride, const uint16_t* x,      \
        int x_rows, int x_div, void* y, int y_f16, const float* topw, const int* sorted_ids, const int* expert_ids,      \
        const int* num_post, int blk, int ns, int row_blocks, int k, int n, int n_exp, f4_t* ws, int* tickets, int wpb,  \
        int act_kind) {                                                                                                  \
        PfGroup<MODE> gp;                                                                                                \
        gp.sorted_ids = sorted_ids;                                                                                      \
        gp.expert_ids = expert_ids;                                                                                      \
        gp.num_post = num_post;                                                                                          \
        gp.topw = topw;                                                                                                  \
        gp.q_stride = q_stride;                                                                                          \
        gp.s_stride = s_stride;                                                                                          \
        gp.ns = ns;                                                                                                      \
        gp.x_rows = x_rows;                                                                                              \
        gp.x_div = x_div;                                                                                                \
        gp.n_exp = n_exp;                                                                                                \
        gp.act_kind = act_kind;                                                                                          \
        (void)blk, (void)ws, (void)tickets, (void)wpb;                                                                   \
        prefill_body<G, SBF, 2, MODE>(reinterpret_cast<const u4_t*>(qa), reinterpret_cast<const uint16_t*>(sa), x, y,    \
                                      row_blocks, k, n, 0, y_f16, 1, 1, gp);                                             \
    }

// This file builds two code objects.  Compiled on its own it holds everything but the dense group-128 kernels;
// prefill_g128.hip includes it with PF_DENSE_G128 defined and holds those twelve, built with the backend's max-ILP
// instruction scheduler (5120 x 34816 at M = 4096: 1.204 -> 1.193 ms, the other layer shapes -0.2...-0.6 %; the
// group-32 builds spill registers under that scheduler and keep the default).
#ifdef PF_DENSE_G128
PREFILL_KERNEL(w4a16_prefill_g128_f16, 128, false, 4, 2)
PREFILL_KERNEL(w4a16_prefill_g128_bf16, 128, true, 4, 2)
PREFILL_KERNEL(w4a16_prefill_g128_f16_m64, 128, false, 2, 3)
PREFILL_KERNEL(w4a16_prefill_g128_bf16_m64, 128, true, 2, 3)
PREFILL_KERNEL(w4a16_prefill_g128_f16_m96, 128, false, 3, 3)
PREFILL_KERNEL(w4a16_prefill_g128_bf16_m96, 128, true, 3, 3)
PREFILL_GLU_KERNEL(w4a16_prefill_g128_f16_glu, 128, false, 4, 2)
PREFILL_GLU_KERNEL(w4a16_prefill_g128_bf16_glu, 128, true, 4, 2)
PREFILL_GLU_KERNEL(w4a16_prefill_g128_f16_m64_glu, 128, false, 2, 3)
PREFILL_GLU_KERNEL(w4a16_prefill_g128_bf16_m64_glu, 128, true, 2, 3)
PREFILL_GLU_KERNEL(w4a16_prefill_g128_f16_m96_glu, 128, false, 3, 3)
PREFILL_GLU_KERNEL(w4a16_prefill_g128_bf16_m96_glu, 128, true, 3, 3)
#else
// y[i] = sum over the nks partials of a split-K launch, added in split order in f32; f32 or f16 out.
// glu != 0: the partials are those of a fused gate|up linear, [slices][t][n]; y is f16 [t][n/2] = act(g) * u on the
// summed gate and up columns (act_kind as in w4_act_mul), the same arithmetic as the unsplit gated epilogue.
extern "C" __global__ __launch_bounds__(256) void w4a16_prefill_splitk_sum(const float* __restrict__ part, void* __restrict__ y,
                                                                           int nks, size_t count, int out_f16, int glu,
                                                                           int n, int act_kind) {
    if (glu) {
        const size_t n_ff = (size_t)(n >> 1), q_ff = n_ff / 4, total = (count / (size_t)n) * q_ff;  // n_ff % 4 == 0 (host)
        for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
            const size_t row = i / q_ff, c4 = i - row * q_ff;
            const float* pg = part + row * (size_t)n + c4 * 4;
            f4_t g = *reinterpret_cast<const f4_t*>(pg), u = *reinterpret_cast<const f4_t*>(pg + n_ff);
            for (int ks = 1; ks < nks; ks++) {
                g += *reinterpret_cast<const f4_t*>(pg + (size_t)ks * count);
                u += *reinterpret_cast<const f4_t*>(pg + (size_t)ks * count + n_ff);
            }
            h4_t o;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float v = w4_act_mul(g[j], u[j], act_kind);
                asm volatile("" : "+v"(v));
                o[j] = (_Float16)v;
            }
            reinterpret_cast<h4_t*>(y)[row * q_ff + c4] = o;
        }
        return;
    }
    const size_t n4 = count / 4;  // count = t*n with n % 4 == 0 is guaranteed by the host
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) {
        f4_t a = reinterpret_cast<const f4_t*>(part)[i];
        for (int ks = 1; ks < nks; ks++) a += reinterpret_cast<const f4_t*>(part + (size_t)ks * count)[i];
        if (out_f16) {
            h4_t v = {(_Float16)a[0], (_Float16)a[1], (_Float16)a[2], (_Float16)a[3]};
            reinterpret_cast<h4_t*>(y)[i] = v;
        } else {
            reinterpret_cast<f4_t*>(y)[i] = a;
        }
    }
}

// Finish of a split launch that carries epilogue options (MODE 0 only; n % 1024 == 0): one workgroup per (row,
// 1024-column chunk) adds the slices in order and applies the options of PfEpi in the order of the unsplit epilogue.
// Statistics: one entry per chunk, stats_out[chunk][row] (the four waves' sums folded in wave order).
extern "C" __global__ __launch_bounds__(256) void w4a16_prefill_splitk_finish(const float* __restrict__ part, void* __restrict__ y,
                                                                              int nks, int t, int n, int out_f16, PfEpi epi) {
    __shared__ float red[4];
    __shared__ float fac_s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int chunks = n >> 10, row = blockIdx.x / chunks, chunk = blockIdx.x - row * chunks;
    if (row >= t) return;
    const bool use_fac = epi.stats_in != nullptr || (epi.in_scale != 1.0f && epi.in_scale != 0.0f);
    if (epi.stats_in != nullptr && wave == 0) {
        float sum = 0.f;
        for (int e = lane; e < epi.n_stats_in; e += 64) sum += epi.stats_in[(size_t)e * epi.ld_stats + row];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
        if (lane == 0) fac_s = (float)(1.0 / sqrt((double)sum * (double)epi.inv_cols_in + 1e-6)) * epi.in_scale;
    }
    if (epi.stats_in != nullptr) __syncthreads();
    const float f = !use_fac ? 1.0f : epi.stats_in != nullptr ? fac_s : epi.in_scale;
    const int col = (chunk << 10) + tid * 4;
    const size_t count = (size_t)t * (size_t)n, at = (size_t)row * n + col;
    f4_t a = *reinterpret_cast<const f4_t*>(part + at);
    for (int ks = 1; ks < nks; ks++) a += *reinterpret_cast<const f4_t*>(part + (size_t)ks * count + at);
    float p = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float v = a[j];
        if (use_fac) v *= f;
        if (epi.resid != nullptr) {
            v += epi.resid[at + j];
            epi.resid[at + j] = v;
        }
        if (col + j < epi.stat_cols) p = __builtin_fmaf(v, v, p);
        if (epi.nw != nullptr) v *= epi.nw[col + j];
        if (epi.out_scale != 1.0f && epi.out_scale != 0.0f) {
            v *= epi.out_scale;
            asm volatile("" : "+v"(v));
        }
        a[j] = v;
    }
    if (out_f16) {
        h4_t o = {(_Float16)a[0], (_Float16)a[1], (_Float16)a[2], (_Float16)a[3]};
        *reinterpret_cast<h4_t*>(reinterpret_cast<_Float16*>(y) + at) = o;
    } else {
        *reinterpret_cast<f4_t*>(reinterpret_cast<float*>(y) + at) = a;
    }
    if (epi.stats_out != nullptr) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) p += __shfl_xor(p, off);
        if (lane == 0) red[wave] = p;
        __syncthreads();
        if (tid == 0 && (chunk << 10) < epi.stat_cols) epi.stats_out[(size_t)chunk * epi.ld_stats + row] = ((red[0] + red[1]) + red[2]) + red[3];
    }
}

PREFILL_KERNEL(w4a16_prefill_g32_f16, 32, false, 4, 2)
PREFILL_KERNEL(w4a16_prefill_g32_bf16, 32, true, 4, 2)
PREFILL_KERNEL(w4a16_prefill_g32_f16_m64, 32, false, 2, 3)
PREFILL_KERNEL(w4a16_prefill_g32_bf16_m64, 32, true, 2, 3)
PREFILL_KERNEL(w4a16_prefill_g32_f16_m96, 32, false, 3, 3)
PREFILL_KERNEL(w4a16_prefill_g32_bf16_m96, 32, true, 3, 3)
PREFILL_GLU_KERNEL(w4a16_prefill_g32_f16_glu, 32, false, 4, 2)
PREFILL_GLU_KERNEL(w4a16_prefill_g32_bf16_glu, 32, true, 4, 2)
PREFILL_GLU_KERNEL(w4a16_prefill_g32_f16_m64_glu, 32, false, 2, 3)
PREFILL_GLU_KERNEL(w4a16_prefill_g32_bf16_m64_glu, 32, true, 2, 3)
PREFILL_GLU_KERNEL(w4a16_prefill_g32_f16_m96_glu, 32, false, 3, 3)
PREFILL_GLU_KERNEL(w4a16_prefill_g32_bf16_m96_glu, 32, true, 3, 3)
PREFILL_MOE_KERNEL(w4a16_moe_g128_f16_pf_glu, 128, false, 1)
PREFILL_MOE_KERNEL(w4a16_moe_g128_f16_pf_lin, 128, false, 2)
PREFILL_MOE_KERNEL(w4a16_moe_g128_bf16_pf_glu, 128, true, 1)
PREFILL_MOE_KERNEL(w4a16_moe_g128_bf16_pf_lin, 128, true, 2)
PREFILL_MOE_KERNEL(w4a16_moe_g32_f16_pf_glu, 32, false, 1)
PREFILL_MOE_KERNEL(w4a16_moe_g32_f16_pf_lin, 32, false, 2)
PREFILL_MOE_KERNEL(w4a16_moe_g32_bf16_pf_glu, 32, true, 1)
PREFILL_MOE_KERNEL(w4a16_moe_g32_bf16_pf_lin, 32, true, 2)
#endif
