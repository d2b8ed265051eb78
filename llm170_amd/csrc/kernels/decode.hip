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
//   * scales: a per-row-block scale load per k tile is a vector-memory instruction that moves 32 distinct bytes; with
//     the x load they cost more address-unit time than the weight stream itself (measured: without them the same
//     load structure runs 13 % faster).  So the scales of a wave's WHOLE k slice (its row blocks x its tiles x groups
//     x 16 rows, contiguous per row block in the tiled scale array) are staged once, ahead of the first weight load,
//     into a wave-private LDS area by LDS DMA (buffer_load ... lds: no registers, no ds_write) and each MFMA group reads
//     its four scales back with ds_read_b64.  (One 8-byte load per ring round into a double-buffered slot was 0.2-0.8 us
//     per launch slower on the 27B shapes: the small loads sit on every round's critical path.)
//   * split-K lives inside the workgroup: the W waves of a block take consecutive k-tile slices of the same RB row
//     blocks and wave 0 folds the partial tiles through LDS in fixed order (deterministic, no atomics, no second
//     launch).  The host picks RB and W;
//   * an output too narrow to give every CU its share of row blocks is also split over k across workgroups
//     (gridDim.y slices): each block parks its partial tile in a workspace and takes a ticket; the block that draws the
//     last ticket of its row blocks adds the slices in slice order (whoever is last: deterministic) and runs the
//     epilogue.  Still one launch, no atomics on data.
#include "w4a16_common.hpp"

#define W4_DECODE_MAX_KSPLIT 8  // k slices across workgroups; the host clamps to this
#ifndef W4_TICKET_ORDER
#define W4_TICKET_ORDER __ATOMIC_RELAXED  // see the hand-over in decode_body
#endif

// One pipeline stage = the loads of one k tile: RB weight tiles, their scales, and XL loads of x.
template <int RB, int XL>
struct DecodeStage {
    u4_t q[RB];
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
// GLU (RB = 2 only): the linear is a fused gate|up projection (rows 0..n/2 gate, n/2..n up); the wave owns gate row
// block u and up row block u + n/32 and writes f16(silu(gate) * up) [t][n/2] instead of the two sums — the
// elementwise kernel between the projections (assets/ew.cu:9-32) folded into the producer, same f32 arithmetic.
// Outputs of a launch over fused linears (plain kernels only).  Part 0 writes y; part j >= 1 starts at output row
// first[j - 1] (a multiple of 16) and writes out[j - 1], each part as its own [t][rows of the part] tensor.  A launch
// with one output passes first[] = INT_MAX: every row then selects y and the row length n.
struct DecodeMulti {
    unsigned long long out[3];
    int first[3];
    int reserved;
};

#define DECODE_ONE_OUTPUT (DecodeMulti{{0ull, 0ull, 0ull}, {0x7fffffff, 0x7fffffff, 0x7fffffff}, 0})

template <int G, bool SBF, int RB, int DEPTH, int XL, bool GLU = false, bool MULTI = false>
__device__ __forceinline__ void decode_body(const u4_t* __restrict__ qt, const uint16_t* __restrict__ st,
                                            const uint16_t* __restrict__ x, void* __restrict__ y, int row_blocks,
                                            int k, int n, int t, int out_f16, f4_t* ws, int* tickets, int W, int nks,
                                            int kt_per_slice, int kt_per_wave, int ldx,
                                            const float* __restrict__ stats_in, int n_stats_in, float inv_cols_in,
                                            float* __restrict__ stats_out, int stat_rows, float* __restrict__ resid,
                                            const float* __restrict__ nw, int act_kind, float in_scale, float out_scale,
                                            DecodeMulti mo) {
    extern __shared__ f4_t red[];  // [W][RB][64] partial tiles of the in-block split-K, then the waves' staged scales
    constexpr int GPT = W4_TILE_K / G;  // scale groups per k tile
    constexpr int C = 4 / XL;           // 32-k chunks (MFMAs) served by one x load
    constexpr int TPL = 16 / C;         // token columns served by one x load
    // The launch geometry (W waves per block, nks k slices over blockIdx.y, tiles per slice and per wave) arrives as
    // kernel arguments: read from the dispatch packet instead, the block size costs a second dependent memory round
    // trip and the balanced split two integer divisions before the first weight load can be issued, on every wave.
    const int lane = threadIdx.x & 63;
    // the wave index is uniform across the wave: keep it (and everything derived from it) in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kt_n = k / W4_TILE_K;
    const int kg_n = kt_n * GPT;
    const int nb0 = blockIdx.x * RB;
    const int glu_half = row_blocks >> 1;  // GLU: row block of rb is blockIdx.x + rb * glu_half
    auto row_block = [&](int rb) { return GLU ? (int)blockIdx.x + rb * glu_half : min(nb0 + rb, row_blocks - 1); };
    const int ky = blockIdx.y;  // k slice of this workgroup
    const int kt_lo = min(kt_n, ky * kt_per_slice), kt_hi = min(kt_n, kt_lo + kt_per_slice);
    const int kt0 = min(kt_hi, kt_lo + wave * kt_per_wave), kt1 = min(kt_hi, kt0 + kt_per_wave);
    const int m = lane & 15, g = lane >> 4;

    // Every load is a raw buffer load: an out-of-range offset returns zeros and costs no memory traffic, which
    // predicates token columns >= t without a branch.
    // x load l of a tile: lane (m, g) fetches, for token m % TPL, the 8 halves of chunk l*C + m / TPL at k offset g*8
    const int xtok = m % TPL, xchunk = m / TPL;
    const unsigned xoff = xtok < t ? ((unsigned)xtok * (unsigned)ldx + (unsigned)(xchunk * 32 + g * 8)) * 2u : W4_OOB;
    const unsigned q_bytes = (unsigned)row_blocks * (unsigned)kt_n * 1024u, s_bytes = (unsigned)row_blocks * (unsigned)kg_n * 32u,
                   x_bytes = ((unsigned)(t - 1) * (unsigned)ldx + (unsigned)k) * 2u;  // x rows are ldx halves apart
    f4_t acc[RB];
    unsigned qoff[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        acc[rb] = (f4_t){0.f, 0.f, 0.f, 0.f};
        const unsigned nb = (unsigned)row_block(rb);  // a tail block re-reads the last row block
        qoff[rb] = nb * (unsigned)kt_n * 1024u + (unsigned)lane * 16u;
    }
    // Scales of the wave's k slice, staged once: the wave's LDS area holds [row block][tile of the slice][group][16 rows],
    // aux_rb_bytes per row block (the stride is that of a full slice, so a shorter last slice leaves a gap); byte
    // o = lane*16 + a*1024 is fetched by lane `lane` of DMA instruction a (a lane past the slice fetches out of range:
    // zeros, no traffic).  AUX_PW bytes per wave, whole DMA instructions.
    const int aux_rb_bytes = kt_per_wave * (GPT * 32);
    const int AUX_PW = (RB * aux_rb_bytes + 1023) & ~1023;
    char* const aux_lds = reinterpret_cast<char*>(red) + W * RB * 1024 + wave * AUX_PW;
    {
        const __amdgpu_buffer_rsrc_t sr_ = w4_make_rsrc(st, s_bytes);
        const int slice_bytes = (kt1 - kt0) * (GPT * 32);
        for (int a = 0; a * 1024 < RB * aux_rb_bytes; a++) {
            const int o = lane * 16 + a * 1024;
            const int rb = o / aux_rb_bytes, rem = o - rb * aux_rb_bytes;
            const unsigned nb = (unsigned)row_block(min(rb, RB - 1));
            const unsigned off = (rb < RB && rem < slice_bytes) ? nb * (unsigned)kg_n * 32u + (unsigned)(kt0 * (GPT * 32) + rem) : W4_OOB;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(sr_, (__attribute__((address_space(3))) void*)(aux_lds + a * 1024), 16, off, 0,
                                                     0, 0);
        }
    }

    // Per-tile addressing costs no vector ALU work: the lane part of every offset is loop invariant, the k-tile part
    // travels in the scalar offset operand, and a tile past the wave's range is switched off by a zero-length
    // descriptor (the wave-uniform select is scalar work).
    DecodeStage<RB, XL> stage[DEPTH];
    auto load = [&](DecodeStage<RB, XL>& s_, int kt) {
        const bool live = kt < kt1;
        const __amdgpu_buffer_rsrc_t qr_ = w4_make_rsrc(qt, live ? q_bytes : 0u);
        const __amdgpu_buffer_rsrc_t xr_ = w4_make_rsrc(x, live ? x_bytes : 0u);
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
            s_.q[rb] = __builtin_amdgcn_raw_buffer_load_b128(qr_, qoff[rb], kt * 1024, 2 /* nt: read-once stream */);
#pragma unroll
        for (int l = 0; l < XL; l++)
            s_.x[l] = __builtin_amdgcn_raw_buffer_load_b128(xr_, xoff + (unsigned)(l * C * 32) * 2u, kt * (W4_TILE_K * 2), 0);
    };
    // sc = this lane's view of the scales of the round's first tile: rows 4g..4g+3 of (row block rb, tile d of the round,
    // group gi) are the 8 bytes at sc + rb*aux_rb_bytes + (d*GPT + gi)*32
    auto compute = [&](const DecodeStage<RB, XL>& s_, const char* sc, int d) {
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
                const u2_t sv = *reinterpret_cast<const u2_t*>(sc + rb * aux_rb_bytes + d * GPT * 32);
#pragma unroll
                for (int i = 0; i < 4; i++)
                    acc[rb][i] = __builtin_fmaf(w4_scale_fast<SBF>((sv[i >> 1] >> (16 * (i & 1))) & 0xFFFFu), part[i], acc[rb][i]);
            } else {
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    f4_t part = {0.f, 0.f, 0.f, 0.f};
                    part = __builtin_amdgcn_mfma_f32_16x16x32_f16(w4_deq8(s_.q[rb][w]),
                                                                  __builtin_bit_cast(h8_t, xb[w]), part, 0, 0, 0);
                    const u2_t sv = *reinterpret_cast<const u2_t*>(sc + rb * aux_rb_bytes + (d * GPT + w % GPT) * 32);
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        acc[rb][i] = __builtin_fmaf(w4_scale_fast<SBF>((sv[i >> 1] >> (16 * (i & 1))) & 0xFFFFu), part[i], acc[rb][i]);
                }
            }
        }
    };

    // Deferred RMS normalisation of the input (the linear commutes with a per-row factor): the launch that produced x
    // left n_stats_in partial sums of squares per row, [n_stats_in][16] floats.  Wave 0 turns them into this lane's
    // 1/sqrt(mean + 1e-6).  The entries of token columns 0..3 are fetched here, ahead of the ring, by LDS DMA (no
    // registers held across the fill) into a staging area behind the scale slots, 64 entries per instruction, lane l
    // entry c*64 + l; once the first weight tiles are in flight lane l adds its entries, a butterfly adds the lanes
    // (fixed order: the same bits on every run), and the factor is parked in the wave's own slot of `red`, which the
    // in-block reduction never writes.  The epilogue multiplies the sums by it.  Further token quads and entries
    // beyond the staging area (8 x 64) repeat the fetch inside input_scale.
    typedef __attribute__((address_space(3))) char lds_char_t;
    lds_char_t* const stage_lds = (lds_char_t*)(reinterpret_cast<char*>(red) + W * RB * 1024 + W * AUX_PW);
    const int stat_chunks = min((n_stats_in + 63) >> 6, 8);
    auto fetch_stats = [&](int c0, int qd) {
        const __amdgpu_buffer_rsrc_t sr_in = w4_make_rsrc(stats_in, (unsigned)n_stats_in * 64u);
        for (int c = 0; c < stat_chunks; c++)  // entries past n_stats_in read as zeros
            __builtin_amdgcn_raw_ptr_buffer_load_lds(sr_in, (__attribute__((address_space(3))) void*)(stage_lds + c * 1024), 16,
                                                     (unsigned)((c0 + c) * 64 + lane) * 64u + (unsigned)qd * 16u, 0, 0, 0);
    };
    if (stats_in != nullptr && wave == 0) fetch_stats(0, 0);
    auto input_scale = [&]() {
        const f4_t* const staged = reinterpret_cast<const f4_t*>(reinterpret_cast<char*>(red) + W * RB * 1024 + W * AUX_PW);
        float mine = 0.f;
        for (int qd = 0; qd * 4 < t; qd++) {  // a quad of token columns at a time
            f4_t sum = {0.f, 0.f, 0.f, 0.f};
            for (int c0 = 0; c0 * 64 < n_stats_in; c0 += 8) {
                if (qd > 0 || c0 > 0) {
                    fetch_stats(c0, qd);
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                } else {
                    // the first fetch is older than the ring fill's loads (DEPTH stages): wait for it alone
                    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DEPTH * (RB + XL) < 63 ? DEPTH * (RB + XL) : 63) : "memory");
                }
                for (int c = 0; c < stat_chunks; c++) sum += staged[c * 64 + lane];
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float v = sum[j];
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
                if (m == qd * 4 + j) mine = v;
            }
        }
        reinterpret_cast<float*>(red)[lane] = (float)(1.0 / sqrt((double)mine * (double)inv_cols_in + 1e-6));
    };

    // One counted loop does the pipeline fill (round -1, compute skipped) and the steady state, so on every path
    // into a stage's compute the outstanding loads are in ring order and the wait can leave the younger stages' loads
    // in flight (s_waitcnt vmcnt(N > 0)).  Tiles past kt1 load zeros and are never computed; the last partial round
    // is finished by the unrolled tail.  The scheduling barriers keep each stage's loads together.
    const int tiles = kt1 - kt0;
    const int rounds = tiles / DEPTH;
    const char* const sc0 = aux_lds + g * 8;
    for (int r = -1; r < rounds; r++) {
        const char* sc = sc0 + r * (DEPTH * GPT * 32);  // the staged scales are older than every ring load: no wait of their own
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            // A wave that holds a landed tile issues ahead of the waves that are only queueing their next loads, so the
            // tile's registers are free for the next load sooner: one row block per wave (seven resident waves per
            // SIMD), t = 1 on 5120 x 34816: 17.20 -> 17.05 us over four same-box rounds; four row blocks per wave,
            // 17408 x 5120 at t = 8 / 16: 13.65 -> 13.45 / 15.88 -> 15.76 us.  With two row blocks per wave the same
            // costs 0.6 % on the wide shape at t = 4 and is left out.
            if (RB != 2) __builtin_amdgcn_s_setprio(1);
            if (r >= 0) compute(stage[d], sc, d);
            __builtin_amdgcn_sched_barrier(0);
            if (RB != 2) __builtin_amdgcn_s_setprio(0);
            load(stage[d], kt0 + (r + 1) * DEPTH + d);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (r == -1 && stats_in != nullptr && wave == 0) input_scale();  // behind the first ring loads, once
    }
    {
        const char* sc = sc0 + rounds * (DEPTH * GPT * 32);
#pragma unroll
        for (int d = 0; d < DEPTH - 1; d++)
            if (rounds * DEPTH + d < tiles) compute(stage[d], sc, d);
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
    if (nks > 1) {  // wave 0 only from here
        // Hand-over of the partial tiles between workgroups (possibly on different XCDs, each with its own L2).
        // Every access to the workspace is a device-scope access: stores with sc1 are written through to memory, loads
        // with sc1 are served from memory — the instruction forms the compiler itself emits for agent-scope atomic
        // stores and loads — so no line of the workspace is ever valid in a non-coherent cache.  Order: the producer
        // waits until its stores have completed (s_waitcnt vmcnt(0): a write-through store is acknowledged by memory)
        // before it draws the ticket; the ticket is an agent-scope atomic; the consumer issues its loads only after
        // the atomic has returned the last ticket, behind an agent-scope acquire fence (buffer_inv sc1: nothing
        // fetched earlier can satisfy them).  A release fence on the producer side would write back the XCD's whole
        // L2 (buffer_wbl2) and cost more per workgroup than the slice itself; with write-through stores there is
        // nothing of this hand-over left in the L2 to write back.
        const __amdgpu_buffer_rsrc_t wr = w4_make_rsrc(ws, (unsigned)gridDim.x * (unsigned)nks * (RB * 1024u));
        const unsigned slice = (unsigned)gridDim.x * (RB * 1024u);  // bytes per k slice
        const unsigned mine = ((unsigned)blockIdx.x * RB * 64u + (unsigned)lane) * 16u;
        constexpr int DEV = 16;                                     // cache policy: device scope (sc1)
        // The slice offset travels in the vector offset and the scalar offset is the constant 0: for a store of more
        // than 8 bytes per lane the hardware reads its data registers after issue, and the compiler inserts the wait
        // state that a following write to them needs only for this form (with a register scalar offset it does not,
        // and its next instruction, v_mov_b32 of the first data register, gave one wrong dword in lanes 12..15 of every
        // 16).  The tiles are also kept live until the stores have completed.
        const unsigned park = mine + (unsigned)ky * slice;
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4_t, acc[rb]), wr, park + rb * 1024u, 0, DEV);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores have reached memory before the ticket is drawn
#pragma unroll
        for (int rb = 0; rb < RB; rb++) asm volatile("" ::"v"(acc[rb]));
        int ticket = 0;
        if (lane == 0) ticket = __hip_atomic_fetch_add(tickets + blockIdx.x, 1, W4_TICKET_ORDER, __HIP_MEMORY_SCOPE_AGENT);
        ticket = __builtin_amdgcn_readfirstlane(ticket);
        if (ticket != nks - 1) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            f4_t part[W4_DECODE_MAX_KSPLIT];
#pragma unroll
            for (int s_ = 0; s_ < W4_DECODE_MAX_KSPLIT; s_++)  // slices past nks: zero-length descriptor, zeros, no traffic
                part[s_] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                                        s_ < nks ? wr : w4_make_rsrc(ws, 0u), mine + rb * 1024u, s_ * slice, DEV));
            f4_t sum = part[0];
#pragma unroll
            for (int s_ = 1; s_ < W4_DECODE_MAX_KSPLIT; s_++) sum += part[s_];
            acc[rb] = sum;
        }
        if (lane == 0) __hip_atomic_store(tickets + blockIdx.x, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    }
    // Power-of-two factors of an f16 hand-over that could leave the f16 range otherwise: x arrives as its true value
    // times 1/in_scale, y leaves as its true value times out_scale (both exact; 1 = none).  in_scale joins the input's
    // 1/rms ahead of everything that looks at the values (statistics, residual, activation); out_scale is applied last.
    if (stats_in != nullptr || in_scale != 1.0f) {
        const float inv = (stats_in != nullptr ? reinterpret_cast<const float*>(red)[lane] : 1.0f) * in_scale;
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int i = 0; i < 4; i++) acc[rb][i] *= inv;
    }
    // The element-wise part of the reference's norm_resid (assets/norm.cu:9-23) that belongs to the producer of an
    // activation: the residual stream takes the linear's output (v = resid + y, written back) and, after the
    // statistics of v, the norm weight of each output row multiplies what the next linear will read.
    if (!GLU && resid != nullptr && m < t) {
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = (nb0 + rb) * 16 + 4 * g + i;
                if (nb0 + rb < row_blocks && row < n) {
                    float* const rp = resid + (size_t)m * n + row;
                    const float v = *rp + acc[rb][i];
                    *rp = v;
                    acc[rb][i] = v;
                }
            }
        }
    }
    if (!GLU && stats_out != nullptr) {
        // this block's share of the rows' sums of squares (rows below stat_rows only), for the launch that consumes y
        float p = 0.f;
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = (nb0 + rb) * 16 + 4 * g + i;
                if (nb0 + rb < row_blocks && row < stat_rows) p = __builtin_fmaf(acc[rb][i], acc[rb][i], p);
            }
        }
        p += __shfl_xor(p, 16);
        p += __shfl_xor(p, 32);
        if (g == 0 && m < t) stats_out[blockIdx.x * 16 + m] = p;
    }
    if (!GLU && nw != nullptr) {
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = (nb0 + rb) * 16 + 4 * g + i;
                if (nb0 + rb < row_blocks && row < n) acc[rb][i] *= nw[row];
            }
        }
    }
    if (m >= t) return;
    if (GLU) {
        const int n_ff = n >> 1;
        h4_t o;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float gt = acc[0][i], up = acc[RB - 1][i];
            float v = w4_act_mul(gt, up, act_kind);
            asm volatile("" : "+v"(v));  // the product is rounded to f32 before the f16 conversion, as in the separate kernel
            v *= out_scale;
            asm volatile("" : "+v"(v));
            o[i] = (_Float16)v;
        }
        *reinterpret_cast<h4_t*>(reinterpret_cast<_Float16*>(y) + (size_t)m * n_ff + blockIdx.x * 16 + 4 * g) = o;
        return;
    }
    if (out_scale != 1.0f) {
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                acc[rb][i] *= out_scale;
                asm volatile("" : "+v"(acc[rb][i]));  // rounded to f32 on its own, not fused into the f16 conversion
            }
    }
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        if (nb0 + rb >= row_blocks) break;
        const int row = (nb0 + rb) * 16 + 4 * g;
        // the part this row block belongs to (uniform: parts start at multiples of 16): its output, first row and end
        const int rb_row = (nb0 + rb) * 16;
        unsigned long long base = reinterpret_cast<unsigned long long>(y);
        int first = 0, end = n;
        if constexpr (MULTI) {
            end = min(mo.first[0], n);
#pragma unroll
            for (int j = 0; j < 3; j++)
                if (rb_row >= mo.first[j]) {
                    base = mo.out[j];
                    first = mo.first[j];
                    end = j < 2 ? min(mo.first[j + 1], n) : n;
                }
        }
        const size_t at = (size_t)m * (size_t)(end - first) + (size_t)(row - first);
        if (out_f16) {
            _Float16* yo = reinterpret_cast<_Float16*>(base) + at;
            if (row + 3 < end) {
                h4_t v = {(_Float16)acc[rb][0], (_Float16)acc[rb][1], (_Float16)acc[rb][2], (_Float16)acc[rb][3]};
                *reinterpret_cast<h4_t*>(yo) = v;
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (row + i < end) yo[i] = (_Float16)acc[rb][i];
            }
        } else {
            float* yo = reinterpret_cast<float*>(base) + at;
            if (row + 3 < end) {
                *reinterpret_cast<f4_t*>(yo) = acc[rb];
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (row + i < end) yo[i] = acc[rb][i];
            }
        }
    }
}

// Two register regimes, chosen per instantiation.  Measured on MI355X: what the streaming rate needs is many resident
// waves with a short ring each, not a deep ring in few waves — with <= 80 VGPRs six waves per SIMD are resident (6144
// on the chip: the whole grid of the 27B layer shapes at two row blocks per wave, 70 % of the gate+up grid at one),
// every wave gets its share of HBM and the generations are even (a deep-ring build at three waves per SIMD ran the
// grid in two uneven generations: 4.6 -> 5.0 TB/s at M = 1).
//   HI: ring sized for 24 VGPRs of load buffers, amdgpu_waves_per_eu(6,6)   — variants that fit 80 VGPRs unspilled
//   MID: the same ring at five waves per SIMD (<= 102 VGPRs)
//   LO: occupancy left to the compiler — the wide variants (4 row blocks, 4 x loads) and group size 32; their ring
//       is as short (a 64-register ring measured 11-18 % slower at group 32, M <= 4: 20.7 -> 18.4 us on the
//       5120 x 34816 shape, 14.8 -> 12.4 us on 17408 x 5120, and no faster anywhere)
#define DECODE_STAGE_REGS(G, RB, XL) (4 * RB + 4 * XL)
#define DECODE_DEPTH(BUDGET, G, RB, XL) \
    ((BUDGET / DECODE_STAGE_REGS(G, RB, XL)) < 2 ? 2 : (BUDGET / DECODE_STAGE_REGS(G, RB, XL)) > 8 ? 8 : (BUDGET / DECODE_STAGE_REGS(G, RB, XL)))

#define DECODE_KERNEL_X(NAME, G, SBF, RB, XL, BUDGET, ATTR)                                                          \
    extern "C" __global__ __launch_bounds__(512) ATTR void NAME##_x##XL(const u4_t* qt, const uint16_t* st,          \
                                                                        const uint16_t* x, void* y, int row_blocks,  \
                                                                        int k, int n, int t, int out_f16, f4_t* ws,  \
                                                                        int* tickets, int waves, int nks,            \
                                                                        int kt_per_slice, int kt_per_wave, int ldx,  \
                                                                        const float* stats_in, int n_stats_in,       \
                                                                        float inv_cols_in, float* stats_out,         \
                                                                        int stat_rows, float* resid,                 \
                                                                        const float* nw, int act_kind,               \
                                                                        float in_scale, float out_scale) {           \
        decode_body<G, SBF, RB, DECODE_DEPTH(BUDGET, G, RB, XL), XL>(                                                \
            qt, st, x, y, row_blocks, k, n, t, out_f16, ws, tickets, waves, nks, kt_per_slice, kt_per_wave, ldx,     \
            stats_in, n_stats_in, inv_cols_in, stats_out, stat_rows, resid, nw, act_kind, in_scale, out_scale,       \
            DECODE_ONE_OUTPUT);                                                                                      \
    }
// The same kernel with one output per part of a fused linear (two row blocks per wave): a symbol of its own, because
// the 40 more bytes of kernel arguments cost every launch 0.2 us, whether it has parts or not (measured on the 27B
// shapes at t = 1 and 4).
#define DECODE_MULTI_KERNEL_X(NAME, G, SBF, XL, BUDGET, ATTR)                                                         \
    extern "C" __global__ __launch_bounds__(512) ATTR void NAME##_x##XL(const u4_t* qt, const uint16_t* st,          \
                                                                        const uint16_t* x, void* y, int row_blocks,  \
                                                                        int k, int n, int t, int out_f16, f4_t* ws,  \
                                                                        int* tickets, int waves, int nks,            \
                                                                        int kt_per_slice, int kt_per_wave, int ldx,  \
                                                                        const float* stats_in, int n_stats_in,       \
                                                                        float inv_cols_in, float* stats_out,         \
                                                                        int stat_rows, float* resid,                 \
                                                                        const float* nw, int act_kind,               \
                                                                        float in_scale, float out_scale,             \
                                                                        DecodeMulti mo) {                            \
        decode_body<G, SBF, 2, DECODE_DEPTH(BUDGET, G, 2, XL), XL, false, true>(                                     \
            qt, st, x, y, row_blocks, k, n, t, out_f16, ws, tickets, waves, nks, kt_per_slice, kt_per_wave, ldx,     \
            stats_in, n_stats_in, inv_cols_in, stats_out, stat_rows, resid, nw, act_kind, in_scale, out_scale, mo);  \
    }
#define DECODE_GLU_KERNEL_X(NAME, G, SBF, XL, BUDGET, ATTR)                                                           \
    extern "C" __global__ __launch_bounds__(512) ATTR void NAME##_x##XL(const u4_t* qt, const uint16_t* st,          \
                                                                        const uint16_t* x, void* y, int row_blocks,  \
                                                                        int k, int n, int t, int out_f16, f4_t* ws,  \
                                                                        int* tickets, int waves, int nks,            \
                                                                        int kt_per_slice, int kt_per_wave, int ldx,  \
                                                                        const float* stats_in, int n_stats_in,       \
                                                                        float inv_cols_in, float* stats_out,         \
                                                                        int stat_rows, float* resid,                 \
                                                                        const float* nw, int act_kind,               \
                                                                        float in_scale, float out_scale) {           \
        decode_body<G, SBF, 2, DECODE_DEPTH(BUDGET, G, 2, XL), XL, true>(                                            \
            qt, st, x, y, row_blocks, k, n, t, out_f16, ws, tickets, waves, nks, kt_per_slice, kt_per_wave, ldx,     \
            stats_in, n_stats_in, inv_cols_in, stats_out, stat_rows, resid, nw, act_kind, in_scale, out_scale,       \
            DECODE_ONE_OUTPUT);                                                                                      \
    }
#define DECODE_HI __attribute__((amdgpu_waves_per_eu(6, 6)))
#define DECODE_MID __attribute__((amdgpu_waves_per_eu(5, 5)))
#define DECODE_LO
// rb1 at group 128: all three x widths fit the HI regime
#define DECODE_KERNEL_RB1(NAME, G, SBF)                                                       \
    DECODE_KERNEL_X(NAME, G, SBF, 1, 1, 24, DECODE_HI) DECODE_KERNEL_X(NAME, G, SBF, 1, 2, 24, DECODE_HI) \
    DECODE_KERNEL_X(NAME, G, SBF, 1, 4, 24, DECODE_HI)
// rb2 at group 128: x1 fits HI, x2 MID
#define DECODE_KERNEL_RB2_G128(NAME, SBF)                                                         \
    DECODE_KERNEL_X(NAME, 128, SBF, 2, 1, 24, DECODE_HI) DECODE_KERNEL_X(NAME, 128, SBF, 2, 2, 24, DECODE_MID) \
    DECODE_KERNEL_X(NAME, 128, SBF, 2, 4, 64, DECODE_LO)
#define DECODE_KERNEL_LO3(NAME, G, SBF, RB)                                                   \
    DECODE_KERNEL_X(NAME, G, SBF, RB, 1, 24, DECODE_LO) DECODE_KERNEL_X(NAME, G, SBF, RB, 2, 24, DECODE_LO) \
    DECODE_KERNEL_X(NAME, G, SBF, RB, 4, 24, DECODE_LO)

DECODE_KERNEL_RB1(w4a16_decode_g128_f16_rb1, 128, false)
DECODE_KERNEL_RB2_G128(w4a16_decode_g128_f16_rb2, false)
DECODE_KERNEL_LO3(w4a16_decode_g128_f16_rb4, 128, false, 4)
DECODE_KERNEL_LO3(w4a16_decode_g32_f16_rb1, 32, false, 1)
DECODE_KERNEL_LO3(w4a16_decode_g32_f16_rb2, 32, false, 2)
DECODE_KERNEL_LO3(w4a16_decode_g32_f16_rb4, 32, false, 4)
DECODE_KERNEL_RB1(w4a16_decode_g128_bf16_rb1, 128, true)
DECODE_KERNEL_RB2_G128(w4a16_decode_g128_bf16_rb2, true)
DECODE_KERNEL_LO3(w4a16_decode_g128_bf16_rb4, 128, true, 4)
DECODE_KERNEL_LO3(w4a16_decode_g32_bf16_rb1, 32, true, 1)
DECODE_KERNEL_LO3(w4a16_decode_g32_bf16_rb2, 32, true, 2)
DECODE_KERNEL_LO3(w4a16_decode_g32_bf16_rb4, 32, true, 4)
// one output per part of a fused linear
#define DECODE_MULTI_G128(NAME, SBF)                                                                       \
    DECODE_MULTI_KERNEL_X(NAME, 128, SBF, 1, 24, DECODE_HI) DECODE_MULTI_KERNEL_X(NAME, 128, SBF, 2, 24, DECODE_MID) \
    DECODE_MULTI_KERNEL_X(NAME, 128, SBF, 4, 64, DECODE_LO)
#define DECODE_MULTI_G32(NAME, SBF)                                                                      \
    DECODE_MULTI_KERNEL_X(NAME, 32, SBF, 1, 24, DECODE_LO) DECODE_MULTI_KERNEL_X(NAME, 32, SBF, 2, 24, DECODE_LO) \
    DECODE_MULTI_KERNEL_X(NAME, 32, SBF, 4, 24, DECODE_LO)
DECODE_MULTI_G128(w4a16_decode_g128_f16_multi, false)
DECODE_MULTI_G128(w4a16_decode_g128_bf16_multi, true)
DECODE_MULTI_G32(w4a16_decode_g32_f16_multi, false)
DECODE_MULTI_G32(w4a16_decode_g32_bf16_multi, true)
// fused gate|up with the SiLU*up epilogue (two row blocks per wave by construction)
#define DECODE_GLU_G128(NAME, SBF)                                                                     \
    DECODE_GLU_KERNEL_X(NAME, 128, SBF, 1, 24, DECODE_HI) DECODE_GLU_KERNEL_X(NAME, 128, SBF, 2, 24, DECODE_MID) \
    DECODE_GLU_KERNEL_X(NAME, 128, SBF, 4, 64, DECODE_LO)
#define DECODE_GLU_G32(NAME, SBF)                                                                    \
    DECODE_GLU_KERNEL_X(NAME, 32, SBF, 1, 24, DECODE_LO) DECODE_GLU_KERNEL_X(NAME, 32, SBF, 2, 24, DECODE_LO) \
    DECODE_GLU_KERNEL_X(NAME, 32, SBF, 4, 24, DECODE_LO)
DECODE_GLU_G128(w4a16_decode_g128_f16_glu, false)
DECODE_GLU_G128(w4a16_decode_g128_bf16_glu, true)
DECODE_GLU_G32(w4a16_decode_g32_f16_glu, false)
DECODE_GLU_G32(w4a16_decode_g32_bf16_glu, true)
