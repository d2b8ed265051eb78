// Operator layer of libw4a16hip.so: shape contract, weight registration with re-layout, regime dispatch.
// Stands in for Gptq4 (crates/backend-gpu/src/rawcuda/gptq4.rs) and for the W4a16Dec linear-op entry points
// upload_lin_g / lin_forward / gemv_t_launch / gemm_launch (w4a16_dec/upload.rs:15-65, kernels/mod.rs:121-144,
// kernels/gemv.rs:112-187, kernels/gemm.rs:4-51).
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>
#include <tuple>

#include "w4a16_internal.h"

static inline unsigned ceil_div(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

// ------------------------------------------------------------------------------------------------ contract
extern "C" int w4a16_check_shapes(size_t t, size_t qlen, size_t slen, size_t xlen, size_t n, size_t k, size_t group) {
    if ((group != 128 && group != 32) || k == 0 || k % group != 0 || t == 0 || n == 0 || qlen != n * (k / 8) ||
        slen != n * (k / group) || xlen != t * k) {
        return w4_fail(W4A16_ERR_SHAPE, "gptq4: shape contract violated q=%zu s=%zu x=%zu n=%zu k=%zu t=%zu group=%zu",
                       qlen, slen, xlen, n, k, t, group);
    }
    return 0;
}

extern "C" const char* w4a16_kernel_sym(int group, int scale_bf16) {
    if (group == 128) return scale_bf16 ? "w4a16_lane_g128_bf16" : "w4a16_lane_g128_f16";
    if (group == 32) return scale_bf16 ? "w4a16_lane_g32_bf16" : "w4a16_lane_g32_f16";
    w4_fail(W4A16_ERR_UNSUPPORTED, "gptq4: unsupported combination group=%d scale_bf16=%d", group, scale_bf16);
    return nullptr;
}

// ------------------------------------------------------------------------------------------------ launches
static int launch_lane(w4a16_ctx* ctx, uint64_t q, uint64_t s, uint64_t x, uint64_t out, size_t n, size_t k, size_t t,
                       size_t group, int scale_bf16) {
    const char* sym = w4a16_kernel_sym((int)group, scale_bf16);
    if (!sym) return W4A16_ERR_UNSUPPORTED;
    if (n > 0x7fffffffu || k > 0x7fffffffu || t > 8u * 65535u)
        return w4_fail(W4A16_ERR_SHAPE, "lane: n=%zu k=%zu t=%zu exceed the launch limits", n, k, t);
    int ni = (int)n, ki = (int)k, ti = (int)t;
    void* params[] = {&q, &s, &x, &out, &ni, &ki, &ti};
    return w4_launch(ctx, sym, ceil_div(n, 4), ceil_div(t, kW4LaneTt), 256, 0, params);
}

// Launch plan of the row-block decode kernel: a pure function of the linear's shape, the row count, the CU count and
// the pinned settings, so that a CPU test can ask for it (w4a16_plan_decode).
//
// Shape, measured on MI355X at the 27B layer shapes (gate+up 5120x34816, down 17408x5120, QKV 5120x7168, O 5120x5120).
// Wide outputs (>= 1024 row blocks): four waves per block; one row block per wave for one or two tokens (5.5 against
// 5.3 TB/s on gate+up), two up to six, four beyond (the more tokens, the more x bytes a weight byte drags through the
// L1 — wider waves share them).  Narrow outputs: two row blocks x eight waves, so that the few blocks still bring
// enough waves; a narrow output with a long k range (the 27B down projection, 320 row blocks x 136 k tiles) from seven
// tokens on runs four row blocks per wave, which share the x loads, with the k slices across workgroups bringing the
// workgroups back (t = 16: 21.6 -> 15.8 us, t = 12: 18.6 -> 14.9, t = 8: 14.2 -> 13.5; level at t = 6).
// k slices across workgroups (one launch; partial tiles and tickets in a workspace): only for a long k range over
// fewer workgroups than CUs (the 27B down projection: 160 blocks x 136 k tiles): slices of about 16 k tiles, four waves
// each (measured 12.4 -> 11.8 us at t = 1, 13.3 -> 12.4 us at t = 4).  Shorter k ranges lose more to the extra
// workgroups than they gain.
// LDS: the waves' staged scales grow with the k tiles per wave (kernels/decode.hip).  A plan that would pass the 160 KiB
// of a CU is shrunk — automatic row blocks per wave are halved first (keeps one launch without tickets), then the k
// range is cut into more slices — and only a shape that fits in no such plan is refused.
struct DecodePlanIn {
    size_t row_blocks = 0, k = 0, group = 128, t = 1;
    int cu_count = 256;
    int rows_per_wave = 0, waves_per_block = 0, ksplit = 0;  // pinned settings of the context, 0 = automatic
    bool glu = false;                                        // gated kernel: two row blocks per wave by construction
    unsigned extra_lds = 0;                                  // staging area of the input statistics
};
struct DecodePlan {
    int rb = 0, waves = 0, nks = 1, kt_per_slice = 0, kt_per_wave = 0;
    size_t blocks = 0;
    unsigned shmem = 0;
};

// LDS bytes of one wave's staged scales (kernels/decode.hip, AUX_PW)
static unsigned decode_scale_lds(size_t group, int rb, int kt_per_wave) {
    return ((unsigned)(rb * kt_per_wave * (128 / (int)group) * 32) + 1023u) / 1024u * 1024u;
}

static int plan_decode(const DecodePlanIn& in, DecodePlan* out) {
    const int kt_n = (int)(in.k / 128);
    if (kt_n <= 0 || in.row_blocks == 0) return w4_fail(W4A16_ERR_SHAPE, "decode: empty linear");
    const bool wide = in.row_blocks >= 1024;
    const bool long_k_narrow = !wide && kt_n >= 64 && in.t >= 7;
    int rb;
    bool rb_auto = false;
    if (in.glu) {
        rb = 2;
    } else if (in.rows_per_wave) {
        rb = in.rows_per_wave / 16;
        if (rb != 1 && rb != 2 && rb != 4) return w4_fail(W4A16_ERR_ARG, "decode: rows_per_wave must be 16, 32 or 64");
    } else {
        rb = wide ? (in.t <= 2 ? 1 : in.t <= 6 ? 2 : 4) : long_k_narrow ? 4 : 2;
        rb_auto = true;
    }
    while (!in.glu && rb > 1 && in.row_blocks < (size_t)rb) rb >>= 1;
    const int waves_auto = in.glu ? (in.t > 8 || wide ? 4 : 8) : wide ? 4 : (in.t > 8 || long_k_narrow ? 4 : 8);
    const int waves_want = std::max(1, std::min(std::min(in.waves_per_block ? in.waves_per_block : waves_auto, 8), kt_n));
    int nks_want = 1;
    bool nks_auto = false;
    int waves_cap = 8;
    if (in.ksplit > 0) {
        nks_want = in.ksplit;
    } else if (in.ksplit == 0) {
        nks_auto = true;
        const size_t blocks = in.glu ? in.row_blocks / 2 : (in.row_blocks + (size_t)rb - 1) / (size_t)rb;
        if (blocks < (size_t)std::max(in.cu_count, 1) && kt_n >= 64) {
            nks_want = std::min(kW4DecodeMaxKsplit, kt_n / 16);
            waves_cap = 4;
        }
    }
    for (;;) {
        DecodePlan P;
        P.rb = rb;
        P.blocks = in.glu ? in.row_blocks / 2 : (in.row_blocks + (size_t)rb - 1) / (size_t)rb;
        P.nks = std::max(1, std::min(nks_want, kt_n / 2));
        P.waves = std::min(waves_want, waves_cap);
        if (P.nks > 1) P.waves = std::max(1, std::min(P.waves, kt_n / P.nks));
        P.kt_per_slice = (kt_n + P.nks - 1) / P.nks;
        P.kt_per_wave = (P.kt_per_slice + P.waves - 1) / P.waves;
        // the split-K partial tiles [waves][rb][1 KiB]; then per wave the scales of its whole k slice (rb x tiles per
        // wave x groups per tile x 32 bytes, in whole 1 KiB DMA instructions); then the statistics staging area
        P.shmem = (unsigned)(P.waves * rb * 1024) + (unsigned)P.waves * decode_scale_lds(in.group, rb, P.kt_per_wave) + in.extra_lds;
        if (P.shmem <= 160u * 1024u) {
            *out = P;
            return 0;
        }
        if (rb_auto && rb > 1) {
            rb >>= 1;
        } else if (nks_auto && nks_want < kW4DecodeMaxKsplit && nks_want * 2 <= kt_n / 2) {
            nks_want = std::max(2, nks_want * 2);
        } else {
            return w4_fail(W4A16_ERR_SHAPE, "decode: k=%zu at group %zu needs %u bytes of LDS for the staged scales (limit 160 KiB) in every launch shape the settings allow: leave rows per wave and k slices automatic, or split k over more workgroups (w4a16_set_decode_ksplit)",
                           in.k, in.group, P.shmem);
        }
    }
}

extern "C" int w4a16_plan_decode(size_t n, size_t k, size_t group, size_t t, int cu_count, int glu, int* rows_per_wave,
                                 int* waves_per_block, int* k_slices, size_t* lds_bytes) {
    if ((group != 128 && group != 32) || n == 0 || k == 0 || k % 128 != 0 || t == 0 || t > 16 || cu_count <= 0)
        return w4_fail(W4A16_ERR_SHAPE, "plan_decode: n=%zu k=%zu group=%zu t=%zu cus=%d", n, k, group, t, cu_count);
    if (glu && n % 32 != 0) return w4_fail(W4A16_ERR_SHAPE, "plan_decode: a gated linear needs n %% 32 == 0");
    DecodePlanIn in;
    in.row_blocks = (n + 15) / 16;
    in.k = k;
    in.group = group;
    in.t = t;
    in.cu_count = cu_count;
    in.glu = glu != 0;
    DecodePlan P;
    W4_TRY(plan_decode(in, &P));
    if (rows_per_wave) *rows_per_wave = P.rb * 16;
    if (waves_per_block) *waves_per_block = P.waves;
    if (k_slices) *k_slices = P.nks;
    if (lds_bytes) *lds_bytes = P.shmem;
    return 0;
}

// Workspace of a launch split over k across workgroups: partial tiles and one ticket per workgroup of a slice.  The
// tickets are zero when (re)allocated and every launch leaves them zero.  With `fixed` the workspace is the caller's (a
// buffer of stated size that cannot grow): a launch that needs more is refused, nothing is allocated.
struct DecodeWorkspace {
    uint64_t ws = 0, tickets = 0;
    size_t ws_cap = 0, tickets_cap = 0;  // bytes
};

static int decode_workspace(w4a16_ctx* ctx, const DecodePlan& P, DecodeWorkspace* out, const DecodeWorkspace* fixed) {
    if (P.nks > 1) {
        const size_t ws_need = P.blocks * (size_t)P.rb * 1024 * (size_t)P.nks, tk_need = P.blocks * 4;
        if (fixed) {
            if (ws_need > fixed->ws_cap || tk_need > fixed->tickets_cap)
                return w4_fail(W4A16_ERR_SHAPE, "decode: the split over k needs %zu bytes of partial tiles and %zu of tickets, the fixed workspace holds %zu and %zu",
                               ws_need, tk_need, fixed->ws_cap, fixed->tickets_cap);
        } else {
            W4_TRY(w4_ensure(ctx, &ctx->decode_ws, &ctx->decode_ws_cap, ws_need));
            if (tk_need > ctx->decode_tickets_cap) {
                W4_TRY(w4_ensure(ctx, &ctx->decode_tickets, &ctx->decode_tickets_cap, std::max<size_t>(tk_need, 16384)));
                W4_TRY(w4a16_memset0(ctx, ctx->decode_tickets, ctx->decode_tickets_cap));
            }
        }
    }
    if (fixed) {
        *out = *fixed;
    } else {
        out->ws = ctx->decode_ws;
        out->tickets = ctx->decode_tickets;
    }
    return 0;
}

// RMS normalisation deferred across a decode launch (kernels/decode.hip): the input's 1/rms comes from the partial
// sums of squares its producer left (stats_in, n_stats_in entries of 16 floats) and multiplies the output; the
// launch leaves its own partial sums over output rows below stat_rows in stats_out.  Zero pointers switch either off.
struct DecodeNorm {
    size_t ldx = 0;  // halves between x rows, 0 = k
    uint64_t stats_in = 0;
    size_t n_stats_in = 0, in_cols = 0;
    uint64_t stats_out = 0;
    size_t stat_rows = 0;
    size_t n_stats_out = 0;  // set by the launch: entries written to stats_out
    uint64_t resid = 0;      // f32 [t][n] residual stream, takes the output: v = resid + y, written back
    uint64_t nw = 0;         // f32 [n] norm weight of the output rows, multiplies what y_dev receives
    int act = 0;             // gated projection only: W4A16_ACT_*
    int in_exp = 0, out_exp = 0;  // x holds its true value times 2^-in_exp, y receives its true value times 2^-out_exp
};

static unsigned decode_stats_lds(const DecodeNorm& nm) {
    return nm.stats_in ? (unsigned)std::min<size_t>((nm.n_stats_in + 63) / 64, 8) * 1024u : 0u;
}

static int check_decode_norm(const W4Lin& L, size_t t, const DecodeNorm& nm) {
    const size_t ldx = nm.ldx ? nm.ldx : L.k;
    if (ldx < L.k || ldx % 8 != 0) return w4_fail(W4A16_ERR_SHAPE, "decode: ldx=%zu must be a multiple of 8 and >= k=%zu", ldx, L.k);
    if (((t - 1) * ldx + L.k) * 2 >= 0x80000000ull) return w4_fail(W4A16_ERR_SHAPE, "decode: x reaches 2 GiB");
    if (nm.stats_in && (nm.n_stats_in == 0 || nm.n_stats_in > 0x7fffffffu / 16 || nm.in_cols == 0))
        return w4_fail(W4A16_ERR_ARG, "decode: input statistics need n_stats_in and in_cols (got %zu, %zu)", nm.n_stats_in, nm.in_cols);
    if (nm.stats_out && nm.stat_rows == 0) return w4_fail(W4A16_ERR_ARG, "decode: output statistics over zero rows");
    if (nm.in_exp < -120 || nm.in_exp > 120 || nm.out_exp < -120 || nm.out_exp > 120)
        return w4_fail(W4A16_ERR_ARG, "decode: hand-over exponents %d, %d outside -120..120", nm.in_exp, nm.out_exp);
    return 0;
}

// Host mirror of DecodeMulti (kernels/decode.hip): outputs and first rows of parts 1..3 of a fused linear; a first row
// of INT_MAX means "no such part" (the value every single-output launch passes).
struct DecodeMultiHost {
    uint64_t out[3] = {0, 0, 0};
    int first[3] = {0x7fffffff, 0x7fffffff, 0x7fffffff};
    int reserved = 0;
};
static_assert(sizeof(DecodeMultiHost) == 40, "DecodeMulti is three pointers and four ints");

static int launch_decode(w4a16_ctx* ctx, const W4Lin& L, uint64_t x, uint64_t y, size_t t, int out_f16,
                         DecodeNorm* norm = nullptr, const DecodeWorkspace* fixed_ws = nullptr,
                         const DecodeMultiHost* multi = nullptr) {
    if (t == 0 || t > 16) return w4_fail(W4A16_ERR_SHAPE, "decode: t=%zu outside 1..16", t);
    if (!L.q_tiled) return w4_fail(W4A16_ERR_UNSUPPORTED, "decode: linear has no tiled copy (needs k %% 128 == 0)");
    if (L.row_blocks * (L.k / 128) * 1024 >= 0x80000000ull)
        return w4_fail(W4A16_ERR_SHAPE, "decode: tiled weights of 2 GiB or more exceed the buffer-descriptor range");
    DecodeNorm none;
    DecodeNorm& nm = norm ? *norm : none;
    W4_TRY(check_decode_norm(L, t, nm));
    DecodePlanIn in;
    in.row_blocks = L.row_blocks;
    in.k = L.k;
    in.group = L.group;
    in.t = t;
    in.cu_count = ctx->cu_count;
    in.rows_per_wave = multi ? 32 : ctx->decode_rows_per_wave;  // the kernels with one output per part are built for two row blocks per wave
    in.waves_per_block = ctx->decode_waves_per_block;
    in.ksplit = ctx->decode_ksplit;
    in.extra_lds = decode_stats_lds(nm);
    DecodePlan P;
    W4_TRY(plan_decode(in, &P));
    const int rb = P.rb;
    int waves = P.waves, nks = P.nks, kt_per_slice = P.kt_per_slice, kt_per_wave = P.kt_per_wave;
    const size_t blocks = P.blocks;
    // x loads per k tile: one serves up to 4 token rows, two up to 8, four up to 16 (kernels/decode.hip)
    const int xl = t <= 4 ? 1 : t <= 8 ? 2 : 4;
    char sym[64];
    if (multi)
        snprintf(sym, sizeof sym, "w4a16_decode_g%zu_%s_multi_x%d", L.group, L.scale_bf16 ? "bf16" : "f16", xl);
    else
        snprintf(sym, sizeof sym, "w4a16_decode_g%zu_%s_rb%d_x%d", L.group, L.scale_bf16 ? "bf16" : "f16", rb, xl);
    uint64_t qt = L.q_tiled, st = L.s_tiled;
    int row_blocks = (int)L.row_blocks, ki = (int)L.k, ni = (int)L.n, ti = (int)t, of = out_f16 ? 1 : 0;
    DecodeWorkspace W;
    W4_TRY(decode_workspace(ctx, P, &W, fixed_ws));
    uint64_t ws = W.ws, tk = W.tickets;
    int ldx = (int)(nm.ldx ? nm.ldx : L.k), n_in = (int)nm.n_stats_in, stat_rows = (int)std::min<size_t>(nm.stat_rows, L.n);
    float inv_cols = nm.in_cols ? 1.0f / (float)nm.in_cols : 0.0f;
    uint64_t s_in = nm.stats_in, s_out = nm.stats_out, resid = nm.resid, nw = nm.nw;
    int act_kind = 0;  // no activation in the plain linear
    float in_scale = std::ldexp(1.0f, nm.in_exp), out_scale = std::ldexp(1.0f, -nm.out_exp);
    nm.n_stats_out = s_out ? std::min(blocks, (size_t)ceil_div((size_t)stat_rows, (size_t)rb * 16)) : 0;
    DecodeMultiHost mo;
    if (multi) {
        if (s_out || resid || nw) return w4_fail(W4A16_ERR_UNSUPPORTED, "decode: a launch with one output per part takes no statistics, residual or norm weight");
        mo = *multi;
    }
    // the last entry is read by the kernels with one output per part only (the argument count is the kernel's own)
    void* params[] = {&qt, &st, &x, &y, &row_blocks, &ki, &ni, &ti, &of, &ws, &tk, &waves, &nks, &kt_per_slice, &kt_per_wave,
                      &ldx, &s_in, &n_in, &inv_cols, &s_out, &stat_rows, &resid, &nw, &act_kind, &in_scale, &out_scale, &mo};
    return w4_launch(ctx, sym, (unsigned)blocks, (unsigned)nks, (unsigned)(waves * 64), P.shmem, params);
}

// Fused gate|up projection with the SiLU*up epilogue (decode regime): y f16 [t][n/2].
static int launch_decode_glu(w4a16_ctx* ctx, const W4Lin& L, uint64_t x, uint64_t y, size_t t, DecodeNorm* norm = nullptr) {
    if (t == 0 || t > 16) return w4_fail(W4A16_ERR_SHAPE, "decode glu: t=%zu outside 1..16", t);
    if (!L.q_tiled) return w4_fail(W4A16_ERR_UNSUPPORTED, "decode glu: linear has no tiled copy (needs k %% 128 == 0)");
    if (L.n % 32 != 0) return w4_fail(W4A16_ERR_SHAPE, "decode glu: n=%zu must be a multiple of 32 (gate and up halves of whole row blocks)", L.n);
    if (L.row_blocks * (L.k / 128) * 1024 >= 0x80000000ull)
        return w4_fail(W4A16_ERR_SHAPE, "decode: tiled weights of 2 GiB or more exceed the buffer-descriptor range");
    DecodeNorm none;
    DecodeNorm& nm = norm ? *norm : none;
    W4_TRY(check_decode_norm(L, t, nm));
    DecodePlanIn in;
    in.row_blocks = L.row_blocks;
    in.k = L.k;
    in.group = L.group;
    in.t = t;
    in.cu_count = ctx->cu_count;
    in.waves_per_block = ctx->decode_waves_per_block;
    in.ksplit = ctx->decode_ksplit;
    in.glu = true;
    in.extra_lds = decode_stats_lds(nm);
    DecodePlan P;
    W4_TRY(plan_decode(in, &P));
    int waves = P.waves, nks = P.nks, kt_per_slice = P.kt_per_slice, kt_per_wave = P.kt_per_wave;
    const size_t blocks = P.blocks;
    const int xl = t <= 4 ? 1 : t <= 8 ? 2 : 4;
    char sym[64];
    snprintf(sym, sizeof sym, "w4a16_decode_g%zu_%s_glu_x%d", L.group, L.scale_bf16 ? "bf16" : "f16", xl);
    uint64_t qt = L.q_tiled, st = L.s_tiled;
    int row_blocks = (int)L.row_blocks, ki = (int)L.k, ni = (int)L.n, ti = (int)t, of = 1;
    DecodeWorkspace W;
    W4_TRY(decode_workspace(ctx, P, &W, nullptr));
    uint64_t ws = W.ws, tk = W.tickets;
    if (nm.stats_out || nm.resid || nm.nw)
        return w4_fail(W4A16_ERR_UNSUPPORTED, "decode glu: the gated output takes no statistics, residual or norm weight");
    int ldx = (int)(nm.ldx ? nm.ldx : L.k), n_in = (int)nm.n_stats_in, stat_rows = 0;
    float inv_cols = nm.in_cols ? 1.0f / (float)nm.in_cols : 0.0f;
    uint64_t s_in = nm.stats_in, s_out = 0, resid = 0, nw = 0;
    if (nm.act != W4A16_ACT_SILU && nm.act != W4A16_ACT_GELU_TANH)
        return w4_fail(W4A16_ERR_ARG, "decode glu: activation %d (0 = silu, 1 = gelu, tanh form)", nm.act);
    int act_kind = nm.act;
    float in_scale = std::ldexp(1.0f, nm.in_exp), out_scale = std::ldexp(1.0f, -nm.out_exp);
    void* params[] = {&qt, &st, &x, &y, &row_blocks, &ki, &ni, &ti, &of, &ws, &tk, &waves, &nks, &kt_per_slice, &kt_per_wave,
                      &ldx, &s_in, &n_in, &inv_cols, &s_out, &stat_rows, &resid, &nw, &act_kind, &in_scale, &out_scale};
    return w4_launch(ctx, sym, (unsigned)blocks, (unsigned)nks, (unsigned)(waves * 64), P.shmem, params);
}

// Launch plan of the prefill GEMM (kernels/prefill.hip): a pure function of (t, n, k), the CU count and the pinned
// settings, so that a CPU test can pin what it chooses at the layer shapes (w4a16_plan_prefill).
// Block tile 128 x 256 (two workgroups per CU), 96 x 256 or 64 x 256 (three per CU, 96 / 64 accumulator registers), the
// k range whole or cut into 2, 3, 4, 6 or 8 slices (split-K: f32 partials in a context-owned workspace, added in slice order by a
// second launch — deterministic), and the super-tile shape: every combination is priced and the cheapest runs.
struct PrefillSuper {
    size_t sup_m, sup_n, supers, load;
};
struct PrefillPlan {
    size_t bm, nks;
    PrefillSuper sup;
    double us;  // the price it won with
};

static PrefillPlan plan_prefill(size_t t, size_t n, size_t k, size_t group, size_t cus, int tile_m_forced, int ksplit_forced,
                                bool glu = false) {
    // a gated launch tiles the n/2 output columns by 128 (each block tile holds the matching 128 up columns as well)
    const size_t tiles_n = glu ? (n / 2 + kW4PfBn / 2 - 1) / (kW4PfBn / 2) : (n + kW4PfBn - 1) / kW4PfBn, kt_n = k / 128;
    // Super-tile shape for a grid of tiles_m x tiles_n block tiles: sup_m <= 8 along m, sup_n in {8, 4, 2, 1} along n.
    // Super-tiles are dealt round-robin to the 8 XCDs (m fastest), so every candidate is priced by the block tiles its
    // busiest XCD ends up with — counted exactly, partial super-tiles at the edges included — and the shape with the
    // lightest busiest XCD wins, the larger one on ties for L2 reuse.  (A fixed 8 along m left 10 tile rows as 8 + 2:
    // the XCDs that drew the 2-row super-tiles idled, 298 against 227 us on the down projection at t = 1280.)
    auto super_for = [&](size_t tiles_m) {
        PrefillSuper best{std::min<size_t>(8, tiles_m), 8, 0, ~(size_t)0};
        for (size_t cm = std::min<size_t>(8, tiles_m); cm >= 1; cm--) {
            for (size_t cn : {8, 4, 2, 1}) {
                const size_t sm = (tiles_m + cm - 1) / cm, sn = (tiles_n + cn - 1) / cn, sp = sm * sn;
                size_t per_xcd[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (size_t sidx = 0; sidx < sp; sidx++)
                    per_xcd[sidx & 7] += std::min(cm, tiles_m - (sidx % sm) * cm) * std::min(cn, tiles_n - (sidx / sm) * cn);
                const size_t load = *std::max_element(per_xcd, per_xcd + 8);
                if (load < best.load || (load == best.load && cm * cn > best.sup_m * best.sup_n)) best = PrefillSuper{cm, cn, sp, load};
            }
        }
        return best;
    };
    // Price of a launch in microseconds, from measurements on MI355X (grids of exactly 256 x j workgroups of each tile,
    // k = 17408 and 5120).  A CU holds c workgroups at once (3 of the 64-row tile, 2 of the 128-row tile); j workgroups
    // per CU (of the busiest XCD) run as floor(j / c) full generations, `full` microseconds per k tile each, and a last
    // partial one whose cost depends on how many workgroups share the CU — a workgroup alone runs nearly twice as fast
    // as one of a full set (the chip is power-limited under this kernel), so the cost of a partial generation starts at
    // more than half a full one and grows from there.  Plus a fixed cost per generation (first loads, epilogue), and for a
    // split launch the second launch and the partial sums written and read back.  The constants started from those
    // measurements and were then fitted to a sweep of tile x slices over 108 (n, k, t) shapes (nine linears, t = 128
    // to 4096), minimising the time lost against the best choice of the sweep: 0.8 % lost on average, 9 % at worst,
    // where the earlier rule (generations x slice length x a tile factor, slices by doubling) lost 3 % and 22 %; fitted
    // on four of the linears only it lost 0.9 % / 11 % on the other five.  The 96-row tile joined later with constants of
    // its own fitted to a sweep of that tile over the same 108 shapes (the others kept): the plans gain 0.5 % on average,
    // up to 14 % where its grid fills the generations better (11008 x 4096 at t = 1536, 17408 x 5120 at t = 1024,
    // 5120 x 34816 at t = 1024: 4 %), and lose at most 3 % against the two-tile plans.
    auto us_per_k_tile = [](size_t rows, double per_cu) {
        static const double at[7] = {0.0, 0.5, 1.0, 1.5, 2.0, 2.5, 3.0};
        static const double part64[7] = {1.0, 1.006, 1.595, 1.738, 1.95, 2.552, 2.903}, part128[5] = {1.5, 1.6, 2.416, 2.9, 3.37},
                            part96[7] = {1.25, 1.258, 1.994, 2.494, 2.729, 3.787, 4.077};
        const double c = rows == 128 ? 2.0 : 3.0, full = rows == 64 ? 2.745 : rows == 96 ? 4.126 : 3.497;
        const double* part = rows == 64 ? part64 : rows == 96 ? part96 : part128;
        const double gens = std::floor(per_cu / c), rem = per_cu - gens * c;
        double us = gens * full;
        if (rem > 1e-9) {
            const int last = rows == 128 ? 4 : 6;
            int i = 1;
            while (i < last && rem > at[i]) i++;
            us += part[i - 1] + (part[i] - part[i - 1]) * (rem - at[i - 1]) / (at[i] - at[i - 1]);
        }
        return us;
    };
    PrefillPlan best{128, 1, PrefillSuper{1, 1, 0, 0}, 1e30};
    for (size_t rows : {(size_t)128, (size_t)96, (size_t)64}) {
        if (tile_m_forced && (size_t)tile_m_forced != rows) continue;
        if (rows == 96 && group != 128 && !tile_m_forced) continue;  // the group-32 builds of that tile spill: only when pinned
        const size_t tiles_m = (t + rows - 1) / rows;
        const PrefillSuper sup = super_for(tiles_m);
        const size_t forced = ksplit_forced > 0 ? std::max<size_t>(1, std::min<size_t>((size_t)ksplit_forced, kt_n / 4)) : 0;
        for (size_t cand : {1, 2, 3, 4, 6, 8}) {
            const size_t nks = forced ? forced : cand;  // a pinned slice count is the only candidate
            if (forced && cand != 1) break;
            if (ksplit_forced < 0 && nks != 1) continue;
            if (!forced && nks > 1 && (n % (glu ? 8 : 4) != 0 || nks > kt_n / 4)) continue;
            const double per_cu = (double)(sup.load * nks) * 8.0 / (double)cus;  // of the busiest XCD
            const double gens = std::ceil(per_cu / (rows == 128 ? 2.0 : 3.0));
            double us = (double)((kt_n + nks - 1) / nks) * us_per_k_tile(rows, per_cu) + 5.7 * gens;
            if (nks > 1) us += 6.0 + (double)nks * (double)t * (double)n * 8.0 / 9.76e6;
            if (us < best.us) best = PrefillPlan{rows, nks, sup, us};
        }
    }
    return best;
}

extern "C" int w4a16_plan_prefill(size_t t, size_t n, size_t k, size_t group, int cu_count, int tile_rows, int k_slices,
                                  size_t out[5], double* price_us) {
    if (t == 0 || n == 0 || k == 0 || k % 128 != 0 || (group != 128 && group != 32) || cu_count <= 0 || !out ||
        (tile_rows != 0 && tile_rows != 64 && tile_rows != 96 && tile_rows != 128) || k_slices < -1 || k_slices > 16)
        return w4_fail(W4A16_ERR_ARG, "plan_prefill: t=%zu n=%zu k=%zu cus=%d tile=%d slices=%d", t, n, k, cu_count, tile_rows, k_slices);
    const PrefillPlan P = plan_prefill(t, n, k, group, (size_t)cu_count, tile_rows, k_slices);
    out[0] = P.bm;
    out[1] = P.nks;
    out[2] = P.sup.sup_m;
    out[3] = P.sup.sup_n;
    out[4] = P.sup.supers;
    if (price_us) *price_us = P.us;
    return 0;
}

// Host mirror of PfEpi (kernels/prefill.hip): same members in the same order.
struct PfEpiHost {
    uint64_t stats_in = 0, stats_out = 0, resid = 0, nw = 0;
    int n_stats_in = 0, ld_stats = 0, stat_cols = 0, ldx = 0;
    float inv_cols_in = 0.f, in_scale = 1.f, out_scale = 1.f;
};
static_assert(sizeof(PfEpiHost) == 64, "PfEpi is four pointers, four ints and three floats, padded to 64 bytes");

// Floats between the rows' entries of a statistics array: 16 in the decode regime (kernels/decode.hip), the row count
// rounded up to 4 beyond it.
static size_t stats_ld(size_t t) { return t <= 16 ? 16 : (t + 3) / 4 * 4; }

// Prefill GEMM (kernels/prefill.hip).  glu_act >= 0: the linear is a fused gate|up projection and y receives
// f16 [t][n/2] = act(gate) * up (W4A16_ACT_*), the element-wise kernel folded into the epilogue.  norm != null: the
// parts of a normalisation deferred across this linear (row factor from the producer's statistics, residual, norm
// weight, statistics of the output, power-of-two hand-over factors), as in the decode kernel.
static int launch_prefill(w4a16_ctx* ctx, const W4Lin& L, uint64_t x, uint64_t y, size_t t, int out_f16, int glu_act = -1,
                          DecodeNorm* norm = nullptr) {
    const bool glu = glu_act >= 0;
    if (glu && L.n % 32 != 0) return w4_fail(W4A16_ERR_SHAPE, "prefill glu: n=%zu must be a multiple of 32 (gate and up halves of whole row blocks)", L.n);
    if (!L.q_tiled) return w4_fail(W4A16_ERR_UNSUPPORTED, "prefill: linear has no tiled copy (needs k %% 128 == 0)");
    if (!L.scales_regular)
        return w4_fail(W4A16_ERR_UNSUPPORTED, "prefill: linear has a zero or non-finite scale (use the decode path)");
    PfEpiHost epi;
    size_t ldx = L.k;
    bool has_epi = false;
    if (norm) {
        W4_TRY(check_decode_norm(L, t, *norm));
        if (glu && (norm->stats_out || norm->resid || norm->nw))
            return w4_fail(W4A16_ERR_UNSUPPORTED, "prefill glu: the gated output takes no statistics, residual or norm weight");
        ldx = norm->ldx ? norm->ldx : L.k;
        epi.stats_in = norm->stats_in;
        epi.n_stats_in = (int)norm->n_stats_in;
        epi.inv_cols_in = norm->in_cols ? 1.0f / (float)norm->in_cols : 0.0f;
        epi.ld_stats = (int)stats_ld(t);
        epi.stats_out = norm->stats_out;
        epi.stat_cols = norm->stats_out ? (int)std::min<size_t>(norm->stat_rows, L.n) : 0;
        epi.resid = norm->resid;
        epi.nw = norm->nw;
        epi.ldx = (int)ldx;
        epi.in_scale = std::ldexp(1.0f, norm->in_exp);
        epi.out_scale = std::ldexp(1.0f, -norm->out_exp);
        has_epi = epi.stats_in || epi.stats_out || epi.resid || epi.nw || norm->in_exp != 0 || norm->out_exp != 0;
        norm->n_stats_out = 0;
    }
    if (((t - 1) * ldx + L.k) * 2 >= 0x80000000ull || L.row_blocks * (L.k / 128) * 1024 >= 0x80000000ull)
        return w4_fail(W4A16_ERR_SHAPE, "prefill: x or the tiled weights reach 2 GiB, beyond the buffer-descriptor range");
    // A split launch finishes in a second kernel.  With epilogue options that kernel works on whole 1024-column
    // chunks of a row; where the shape does not allow it (or for the gated form) the k range stays whole.
    int ksplit = ctx->prefill_ksplit;
    if (has_epi && (glu || L.n % 1024 != 0)) ksplit = -1;
    // the plan depends on (t, n, k) and the pinned settings only and is kept per shape
    PrefillPlan plan;
    {
        const auto key = std::make_tuple(t, L.n, L.k, ctx->prefill_tile_m + (glu ? 1000 : 0), ksplit);
        const auto hit = ctx->prefill_plans.find(key);
        if (hit != ctx->prefill_plans.end()) {
            plan = PrefillPlan{hit->second[0], hit->second[1], PrefillSuper{hit->second[2], hit->second[3], hit->second[4], 0}, 0.0};
        } else {
            plan = plan_prefill(t, L.n, L.k, L.group, (size_t)std::max(ctx->cu_count, 1), ctx->prefill_tile_m, ksplit, glu);
            ctx->prefill_plans[key] = {plan.bm, plan.nks, plan.sup.sup_m, plan.sup.sup_n, plan.sup.supers};
        }
    }
    const size_t bm = plan.bm, nks = plan.nks, sup_m = plan.sup.sup_m, sup_n = plan.sup.sup_n, supers = plan.sup.supers;
    const size_t grid = ((supers + 7) / 8) * (sup_m * sup_n) * 8;
    char sym[64];
    snprintf(sym, sizeof sym, "w4a16_prefill_g%zu_%s%s%s", L.group, L.scale_bf16 ? "bf16" : "f16", bm == 64 ? "_m64" : bm == 96 ? "_m96" : "", glu ? "_glu" : "");
    // two stages of bm rows x PF_KS halves, then bm words (row factors of the dense kernels)
    const unsigned shmem = (unsigned)(2 * bm * kW4PfKs * 2 + bm * 4);
    uint64_t qt = L.q_tiled, st = L.s_tiled;
    int row_blocks = (int)L.row_blocks, ki = (int)L.k, ni = (int)L.n, ti = (int)t, of = (out_f16 || glu) ? 1 : 0;
    int spm = (int)sup_m, spn = (int)sup_n, act = glu ? glu_act : 0, glu_i = glu ? 1 : 0;
    if (nks == 1) {
        if (norm && epi.stats_out) norm->n_stats_out = ((size_t)epi.stat_cols + 63) / 64;  // one entry per wave's 64 columns
        void* params[] = {&qt, &st, &x, &y, &row_blocks, &ki, &ni, &ti, &of, &spm, &spn, &act, &epi};
        return w4_launch(ctx, sym, (unsigned)grid, 1, kW4PfThreads, shmem, params);
    }
    if (L.n % (glu ? 8 : 4) != 0) return w4_fail(W4A16_ERR_UNSUPPORTED, "prefill: split-K needs n %% %d == 0", glu ? 8 : 4);
    const size_t count = t * L.n;
    W4_TRY(w4_ensure(ctx, &ctx->prefill_ws, &ctx->prefill_ws_cap, count * 4 * nks));
    uint64_t ws = ctx->prefill_ws;
    int zero = 0;
    PfEpiHost slice_epi;  // the slices only need the row stride of x; the finish kernel applies the options
    slice_epi.ldx = (int)ldx;
    void* params[] = {&qt, &st, &x, &ws, &row_blocks, &ki, &ni, &ti, &zero, &spm, &spn, &act, &slice_epi};
    W4_TRY(w4_launch(ctx, sym, (unsigned)grid, (unsigned)nks, kW4PfThreads, shmem, params));
    int nksi = (int)nks;
    if (has_epi) {
        if (t * (L.n / 1024) > 0x7fffffffu) return w4_fail(W4A16_ERR_SHAPE, "prefill: t=%zu n=%zu exceed the finish launch", t, L.n);
        if (norm && epi.stats_out) norm->n_stats_out = ((size_t)epi.stat_cols + 1023) / 1024;  // one entry per 1024-column chunk
        void* fp[] = {&ws, &y, &nksi, &ti, &ni, &of, &epi};
        return w4_launch(ctx, "w4a16_prefill_splitk_finish", (unsigned)(t * (L.n / 1024)), 1, 256, 0, fp);
    }
    size_t cnt = count;
    void* rp[] = {&ws, &y, &nksi, &cnt, &of, &glu_i, &ni, &act};
    return w4_launch(ctx, "w4a16_prefill_splitk_sum", std::min<unsigned>(ceil_div(count / (glu ? 8 : 4), 256), 4096), 1, 256, 0, rp);
}

// ------------------------------------------------------------------------------------------------ Gptq4::gemm
extern "C" int w4a16_gemm_host(w4a16_ctx* ctx, const uint16_t* x_f16, size_t t, const uint32_t* q, const uint16_t* s,
                               size_t n, size_t k, size_t group, int scale_bf16, float* out_f32) {
    if (!ctx || !x_f16 || !q || !s || !out_f32) return w4_fail(W4A16_ERR_ARG, "gemm_host: null argument");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    if ((group != 128 && group != 32) || k == 0 || k % group != 0 || t == 0 || n == 0)
        return w4_fail(W4A16_ERR_SHAPE, "gptq4: shape contract violated n=%zu k=%zu t=%zu group=%zu", n, k, t, group);
    if (!w4a16_kernel_sym((int)group, scale_bf16)) return W4A16_ERR_UNSUPPORTED;
    const size_t qb = n * (k / 8) * 4, sb = n * (k / group) * 2, xb = t * k * 2, ob = t * n * 4;
    uint64_t dq = 0, ds = 0, dx = 0, dout = 0;
    int rc = w4a16_alloc(ctx, qb, &dq);
    if (!rc) rc = w4a16_alloc(ctx, sb, &ds);
    if (!rc) rc = w4a16_alloc(ctx, xb, &dx);
    if (!rc) rc = w4a16_alloc(ctx, ob, &dout);
    if (!rc) rc = w4a16_h2d(ctx, dq, q, qb);
    if (!rc) rc = w4a16_h2d(ctx, ds, s, sb);
    if (!rc) rc = w4a16_h2d(ctx, dx, x_f16, xb);
    if (!rc) rc = launch_lane(ctx, dq, ds, dx, dout, n, k, t, group, scale_bf16);
    if (!rc) rc = w4a16_d2h(ctx, out_f32, dout, ob);
    const std::string keep = w4_err_save();
    (void)w4a16_free(ctx, dq);
    (void)w4a16_free(ctx, ds);
    (void)w4a16_free(ctx, dx);
    (void)w4a16_free(ctx, dout);
    if (rc) w4_err_restore(keep);
    return rc;
}

// ------------------------------------------------------------------------------------------------ registration
// The MFMA prefill kernels multiply their accumulators by s_prev / s_cur at every group boundary and hold sum / s_cur:
// every scale must be finite and non-zero, and a bf16 scale inside [2^-60, 2^60], so that neither a quotient of two
// scales nor an accumulator expressed in the smallest one leaves the f32 range (f16 scales span 2^-24 .. 2^16 and
// always qualify; a bf16 subnormal or 1e-38 does not).
bool w4_scales_regular(const uint16_t* sp, size_t count, int scale_bf16) {
    const unsigned expmask = scale_bf16 ? 0x7F80u : 0x7C00u;
    for (size_t i = 0; i < count; i++) {
        const unsigned b = sp[i];
        if ((b & 0x7FFFu) == 0 || (b & expmask) == expmask) return false;
        if (scale_bf16) {
            const unsigned e = (b >> 7) & 0xFFu;  // biased exponent, 127 = 2^0
            if (e < 127u - 60u || e > 127u + 60u) return false;
        }
    }
    return true;
}

static void free_lin(w4a16_ctx* ctx, W4Lin& L) {
    (void)w4a16_free(ctx, L.q_raw);
    (void)w4a16_free(ctx, L.s_raw);
    (void)w4a16_free(ctx, L.q_tiled);
    (void)w4a16_free(ctx, L.s_tiled);
    L = W4Lin();
}

extern "C" int w4a16_upload_lin(w4a16_ctx* ctx, const char* name, const void* q, size_t qlen_bytes, const void* s,
                                size_t slen_bytes, size_t n, size_t k, size_t group, int scale_bf16) {
    if (!ctx || !name || !q || !s) return w4_fail(W4A16_ERR_ARG, "upload_lin: null argument");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    if (group != 128 && group != 32)
        return w4_fail(W4A16_ERR_UNSUPPORTED, "gptq4: unsupported combination group=%zu scale_bf16=%d", group, scale_bf16);
    if (n == 0 || k == 0 || k % group != 0 || qlen_bytes != n * (k / 2) || slen_bytes != n * (k / group) * 2)
        return w4_fail(W4A16_ERR_SHAPE, "upload_lin_g %s: q=%zu s=%zu != n%zu k%zu g%zu contract", name, qlen_bytes,
                       slen_bytes, n, k, group);
    if (n > 0x7fffffffu || k > 0x7fffffffu) return w4_fail(W4A16_ERR_SHAPE, "upload_lin_g %s: n or k too large", name);
    W4Lin L;
    L.n = n;
    L.k = k;
    L.group = group;
    L.scale_bf16 = scale_bf16 ? 1 : 0;
    // "regular": what the MFMA prefill kernel can carry as a running unit (w4_scales_regular).  Other linears are served
    // by the streaming kernels, which only ever multiply by a scale.
    L.scales_regular = w4_scales_regular(static_cast<const uint16_t*>(s), slen_bytes / 2, scale_bf16);
    int rc = w4a16_alloc(ctx, qlen_bytes, &L.q_raw);
    if (!rc) rc = w4a16_alloc(ctx, slen_bytes, &L.s_raw);
    if (!rc) rc = w4a16_h2d(ctx, L.q_raw, q, qlen_bytes);
    if (!rc) rc = w4a16_h2d(ctx, L.s_raw, s, slen_bytes);
    if (rc) {
        const std::string keep = w4_err_save();
        free_lin(ctx, L);
        w4_err_restore(keep);
        return rc;
    }
    return w4_register_lin(ctx, name, L);
}

// Several linears that read the same x become one (rows concatenated in the order given), so that one launch serves
// them all: the as-given operands are row-major, so the fused operands are plain concatenations.
extern "C" int w4a16_lin_fuse(w4a16_ctx* ctx, const char* name, const char* const* parts, size_t n_parts,
                              int drop_parts) {
    if (!ctx || !name || !parts || n_parts == 0) return w4_fail(W4A16_ERR_ARG, "lin_fuse: null argument");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    std::vector<W4Lin*> P(n_parts);
    W4Lin F;
    for (size_t i = 0; i < n_parts; i++) {
        if (!parts[i]) return w4_fail(W4A16_ERR_ARG, "lin_fuse %s: part %zu is null", name, i);
        if (std::string(parts[i]) == name) return w4_fail(W4A16_ERR_ARG, "lin_fuse %s: a part has the fused name", name);
        for (size_t j = 0; j < i; j++)
            if (std::string(parts[i]) == parts[j]) return w4_fail(W4A16_ERR_ARG, "lin_fuse %s: part %s twice", name, parts[i]);
        W4_TRY(w4_find_lin(ctx, parts[i], &P[i]));
        const W4Lin& L = *P[i];
        if (!L.q_raw) return w4_fail(W4A16_ERR_NOT_FOUND, "lin_fuse %s: part %s has dropped its as-given operands", name, parts[i]);
        if (i == 0) {
            F.k = L.k;
            F.group = L.group;
            F.scale_bf16 = L.scale_bf16;
        } else if (L.k != F.k || L.group != F.group || L.scale_bf16 != F.scale_bf16) {
            return w4_fail(W4A16_ERR_SHAPE, "lin_fuse %s: part %s (k=%zu g=%zu bf16=%d) does not match k=%zu g=%zu bf16=%d",
                           name, parts[i], L.k, L.group, L.scale_bf16, F.k, F.group, F.scale_bf16);
        }
        F.n += L.n;
        F.part_n.push_back(L.n);
        F.scales_regular = F.scales_regular && L.scales_regular;
    }
    if (F.n > 0x7fffffffu) return w4_fail(W4A16_ERR_SHAPE, "lin_fuse %s: n=%zu too large", name, F.n);
    const size_t q_row = F.k / 2, s_row = (F.k / F.group) * 2;
    int rc = w4a16_alloc(ctx, F.n * q_row, &F.q_raw);
    if (!rc) rc = w4a16_alloc(ctx, F.n * s_row, &F.s_raw);
    size_t row = 0;
    for (size_t i = 0; i < n_parts && !rc; i++) {
        rc = w4a16_d2d(ctx, F.q_raw + row * q_row, P[i]->q_raw, P[i]->n * q_row);
        if (!rc) rc = w4a16_d2d(ctx, F.s_raw + row * s_row, P[i]->s_raw, P[i]->n * s_row);
        row += P[i]->n;
    }
    if (rc) {
        const std::string keep = w4_err_save();
        free_lin(ctx, F);
        w4_err_restore(keep);
        return rc;
    }
    W4_TRY(w4_register_lin(ctx, name, F));  // builds the tiled copy and waits for the stream
    if (drop_parts)
        for (size_t i = 0; i < n_parts; i++) {
            auto it = ctx->lins.find(parts[i]);
            if (it != ctx->lins.end()) {
                free_lin(ctx, it->second);
                ctx->lins.erase(it);
            }
        }
    return 0;
}

// One decode launch over a fused linear with one output per part (the reference's multi-linear GEMV: a table of
// {weights, scales, out, n, k} segments, w4a16_dec/buffers.rs:229-366, launched by kernels/gemv.rs:189-332).
extern "C" int w4a16_lin_forward_multi(w4a16_ctx* ctx, const char* name, uint64_t x_dev, const uint64_t* outs_dev,
                                       size_t n_outs, size_t t, int out_f16) {
    if (!ctx || !name || !outs_dev) return w4_fail(W4A16_ERR_ARG, "lin_forward_multi: null argument");
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (L->part_n.size() < 2)
        return w4_fail(W4A16_ERR_ARG, "lin_forward_multi %s: not a fused linear (w4a16_lin_fuse makes one)", name);
    if (n_outs != L->part_n.size())
        return w4_fail(W4A16_ERR_ARG, "lin_forward_multi %s: %zu outputs for %zu parts", name, n_outs, L->part_n.size());
    if (n_outs > 4)
        return w4_fail(W4A16_ERR_UNSUPPORTED, "lin_forward_multi %s: %zu parts (one launch writes up to four outputs)", name, n_outs);
    if (!x_dev) return w4_fail(W4A16_ERR_ARG, "lin_forward_multi %s: null x", name);
    if (t == 0) return w4_fail(W4A16_ERR_SHAPE, "lin_forward_multi %s: t=0", name);
    if (t > 16)
        return w4_fail(W4A16_ERR_UNSUPPORTED, "lin_forward_multi %s: t=%zu: one output per part exists for decode steps (t <= 16); beyond, w4a16_lin_forward writes the parts side by side in one [t][n] tensor", name, t);
    DecodeMultiHost mo;
    size_t first = 0;
    for (size_t i = 0; i < n_outs; i++) {
        if (!outs_dev[i]) return w4_fail(W4A16_ERR_ARG, "lin_forward_multi %s: output %zu is null", name, i);
        if (L->part_n[i] % 16 != 0)
            return w4_fail(W4A16_ERR_SHAPE, "lin_forward_multi %s: part %zu has %zu rows; parts must be multiples of 16 rows (a 16-row block writes one output)", name, i, L->part_n[i]);
        if (i > 0) {
            mo.out[i - 1] = outs_dev[i];
            mo.first[i - 1] = (int)first;
        }
        first += L->part_n[i];
    }
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    return launch_decode(ctx, *L, x_dev, outs_dev[0], t, out_f16, nullptr, nullptr, &mo);
}

// Second half of a registration: build the tiled copy from the as-given operands already on the device and enter
// the linear under its name.  Frees L's buffers on failure.
int w4_register_lin(w4a16_ctx* ctx, const char* name, W4Lin& L) {
    int rc = 0;
    if (L.k % 128 == 0) {
        L.row_blocks = (L.n + 15) / 16;
        const size_t kt_n = L.k / 128, kg_n = L.k / L.group;
        const size_t qt_bytes = L.row_blocks * kt_n * 1024, st_bytes = L.row_blocks * kg_n * 16 * 2;
        rc = w4a16_alloc(ctx, qt_bytes, &L.q_tiled);
        if (!rc) rc = w4a16_alloc(ctx, st_bytes, &L.s_tiled);
        if (!rc) {
            int ni = (int)L.n, ki = (int)L.k, rbi = (int)L.row_blocks, kgi = (int)kg_n;
            void* pq[] = {&L.q_raw, &L.q_tiled, &ni, &ki, &rbi};
            rc = w4_launch(ctx, "w4a16_tile_q", ceil_div(qt_bytes / 4, 256), 1, 256, 0, pq);
            void* ps[] = {&L.s_raw, &L.s_tiled, &ni, &kgi, &rbi};
            if (!rc) rc = w4_launch(ctx, "w4a16_tile_s", ceil_div(st_bytes / 2, 256), 1, 256, 0, ps);
            if (!rc) rc = w4a16_sync(ctx);
        }
    }
    if (rc) {
        const std::string keep = w4_err_save();
        free_lin(ctx, L);
        w4_err_restore(keep);
        return rc;
    }
    auto it = ctx->lins.find(name);
    if (it != ctx->lins.end()) free_lin(ctx, it->second);  // re-registration frees the old buffers (upload.rs:53-56)
    ctx->lins[name] = L;
    return 0;
}

int w4_find_lin(w4a16_ctx* ctx, const char* name, W4Lin** out) {
    if (!ctx || !name) return w4_fail(W4A16_ERR_ARG, "lin: null argument");
    auto it = ctx->lins.find(std::string_view(name));  // transparent comparator: no std::string is built
    if (it == ctx->lins.end()) return w4_fail(W4A16_ERR_NOT_FOUND, "lin %s: not registered", name);
    *out = &it->second;
    return 0;
}

extern "C" int w4a16_lin_drop_raw(w4a16_ctx* ctx, const char* name) {
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (!L->q_tiled) return w4_fail(W4A16_ERR_UNSUPPORTED, "lin %s: no tiled copy, the operands as given must stay", name);
    W4_TRY(w4a16_free(ctx, L->q_raw));
    W4_TRY(w4a16_free(ctx, L->s_raw));
    L->q_raw = L->s_raw = 0;
    return 0;
}

extern "C" int w4a16_lin_info(w4a16_ctx* ctx, const char* name, size_t* n, size_t* k, size_t* group, int* scale_bf16,
                              int* has_tiled, int* has_raw) {
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (n) *n = L->n;
    if (k) *k = L->k;
    if (group) *group = L->group;
    if (scale_bf16) *scale_bf16 = L->scale_bf16;
    if (has_tiled) *has_tiled = L->q_tiled != 0;
    if (has_raw) *has_raw = L->q_raw != 0;
    return 0;
}

// ------------------------------------------------------------------------------------------------ forward
extern "C" int w4a16_lin_forward(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t y_dev, size_t t, int out_f16,
                                 int path) {
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (!x_dev || !y_dev || t == 0) return w4_fail(W4A16_ERR_ARG, "lin_forward %s: null operand or t=0", name);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    if (path == W4A16_PATH_AUTO) {
        if (!L->q_tiled)
            path = W4A16_PATH_LANE;
        else if (t <= 16)
            path = W4A16_PATH_DECODE;
        else if (t <= 64 || !L->scales_regular)
            // a few dozen rows are still bound by the weight stream (measured on the 27B shapes: 33 vs 57 us at t = 32
            // on gate|up, 22 vs 43 us on the down projection; level with the MFMA tiles at t = 128).  A linear with a
            // zero or non-finite scale always comes here: the prefill kernel divides by scales.
            path = W4A16_PATH_STREAM;
        else
            path = W4A16_PATH_PREFILL;
    }
    switch (path) {
        case W4A16_PATH_LANE:
            if (!L->q_raw) return w4_fail(W4A16_ERR_NOT_FOUND, "lin %s: operands as given were dropped", name);
            if (out_f16) return w4_fail(W4A16_ERR_UNSUPPORTED, "lin_forward %s: the bit-exact path writes f32 only", name);
            return launch_lane(ctx, L->q_raw, L->s_raw, x_dev, y_dev, L->n, L->k, t, L->group, L->scale_bf16);
        case W4A16_PATH_DECODE:
            return launch_decode(ctx, *L, x_dev, y_dev, t, out_f16);
        case W4A16_PATH_PREFILL:
            return launch_prefill(ctx, *L, x_dev, y_dev, t, out_f16);
        case W4A16_PATH_STREAM:
            return w4_dense_grouped(ctx, *L, x_dev, y_dev, t, out_f16);
        default:
            return w4_fail(W4A16_ERR_ARG, "lin_forward %s: unknown path %d", name, path);
    }
}

// Decode-regime lin_forward whose split-K workspace is the fixed per-device buffer of w4a16_noalloc.hip: no allocation
// on any path (the linear and the kernel are looked up without building a std::string).
int w4_lin_forward_fixed_ws(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t y_dev, size_t t, int out_f16,
                            uint64_t ws, size_t ws_bytes, uint64_t tickets, size_t ticket_bytes) {
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (!x_dev || !y_dev || t == 0) return w4_fail(W4A16_ERR_ARG, "lin_forward_noalloc %s: null operand or t=0", name);
    if (t > 16)
        return w4_fail(W4A16_ERR_SHAPE, "lin_forward_noalloc %s: t=%zu, the entry point serves the decode regime (1..16 rows)", name, t);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    DecodeWorkspace W;
    W.ws = ws;
    W.ws_cap = ws_bytes;
    W.tickets = tickets;
    W.tickets_cap = ticket_bytes;
    return launch_decode(ctx, *L, x_dev, y_dev, t, out_f16, nullptr, &W);
}

extern "C" int w4a16_lin_forward_glu(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t y_f16_dev, size_t t) {
    return w4a16_lin_forward_glu_act(ctx, name, x_dev, y_f16_dev, t, W4A16_ACT_SILU);
}

extern "C" int w4a16_lin_forward_glu_act(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t y_f16_dev, size_t t,
                                         int act) {
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (!x_dev || !y_f16_dev || t == 0) return w4_fail(W4A16_ERR_ARG, "lin_forward_glu %s: null operand or t=0", name);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    if (act != W4A16_ACT_SILU && act != W4A16_ACT_GELU_TANH)
        return w4_fail(W4A16_ERR_ARG, "lin_forward_glu %s: activation %d (0 = silu, 1 = gelu, tanh form)", name, act);
    if (t <= 16) {
        DecodeNorm nm;
        nm.act = act;
        return launch_decode_glu(ctx, *L, x_dev, y_f16_dev, t, &nm);
    }
    // beyond the decode regime the same split as w4a16_lin_forward's AUTO: the weight-streaming kernel up to 64 rows
    // (and for scales the MFMA kernel cannot divide by), the tiled MFMA GEMM above — each with the gated epilogue
    if (L->n % 32 != 0) return w4_fail(W4A16_ERR_SHAPE, "lin_forward_glu %s: n=%zu must be a multiple of 32", name, L->n);
    if (!L->q_tiled) return w4_fail(W4A16_ERR_UNSUPPORTED, "lin_forward_glu %s: linear has no tiled copy (needs k %% 128 == 0)", name);
    if (t <= 64 || !L->scales_regular) return w4_dense_grouped(ctx, *L, x_dev, y_f16_dev, t, 1, act);
    return launch_prefill(ctx, *L, x_dev, y_f16_dev, t, 1, act);
}

// Largest row norm of the dequantised weights (kernels/layout.hip, w4a16_row_norm_max_*), computed on the first request
// and kept with the linear.  The one device word it is reduced into belongs to the context.
extern "C" int w4a16_lin_row_norm_max(w4a16_ctx* ctx, const char* name, float* out) {
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (!out) return w4_fail(W4A16_ERR_ARG, "lin_row_norm_max %s: null output", name);
    if (L->row_norm_max < 0.0f) {
        if (!L->q_tiled) return w4_fail(W4A16_ERR_UNSUPPORTED, "lin_row_norm_max %s: linear has no tiled copy (needs k %% 128 == 0)", name);
        if (ctx->capturing)
            return w4_fail(W4A16_ERR_ARG, "lin_row_norm_max %s: first request while the launch stream is capturing (it reads a word back): ask once before the capture", name);
        W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
        W4_TRY(w4_ensure(ctx, &ctx->norm_word, &ctx->norm_word_cap, 256));
        W4_TRY(w4a16_memset0(ctx, ctx->norm_word, 256));
        int rbi = (int)L->row_blocks, kt_n = (int)(L->k / 128), gi = (int)L->group;
        void* p[] = {&L->q_tiled, &L->s_tiled, &ctx->norm_word, &rbi, &kt_n, &gi};
        W4_TRY(w4_launch(ctx, L->scale_bf16 ? "w4a16_row_norm_max_bf16" : "w4a16_row_norm_max_f16",
                         ceil_div(L->row_blocks, 4), 1, 256, 0, p));
        float v = 0.0f;
        W4_TRY(w4a16_d2h(ctx, &v, ctx->norm_word, 4));
        if (!std::isfinite(v)) return w4_fail(W4A16_ERR_UNSUPPORTED, "lin_row_norm_max %s: a scale is not finite", name);
        L->row_norm_max = v;
    }
    *out = L->row_norm_max;
    return 0;
}

extern "C" int w4a16_lin_forward_deferred_norm(w4a16_ctx* ctx, const char* name, uint64_t x_dev, size_t ldx, size_t t,
                                               uint64_t stats_in_dev, size_t n_stats_in, size_t in_cols, uint64_t y_dev,
                                               int out_f16, uint64_t stats_out_dev, size_t stat_rows,
                                               size_t* n_stats_out, uint64_t resid_dev, uint64_t nw_dev) {
    return w4a16_lin_forward_deferred_norm_scaled(ctx, name, x_dev, ldx, t, stats_in_dev, n_stats_in, in_cols, 0, y_dev,
                                                  out_f16, 0, stats_out_dev, stat_rows, n_stats_out, resid_dev, nw_dev);
}

extern "C" int w4a16_lin_forward_deferred_norm_scaled(w4a16_ctx* ctx, const char* name, uint64_t x_dev, size_t ldx,
                                                      size_t t, uint64_t stats_in_dev, size_t n_stats_in, size_t in_cols,
                                                      int in_exp, uint64_t y_dev, int out_f16, int out_exp,
                                                      uint64_t stats_out_dev, size_t stat_rows, size_t* n_stats_out,
                                                      uint64_t resid_dev, uint64_t nw_dev) {
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (!x_dev || !y_dev || t == 0) return w4_fail(W4A16_ERR_ARG, "lin_forward_deferred_norm %s: null operand or t=0", name);
    if (stats_out_dev && !n_stats_out) return w4_fail(W4A16_ERR_ARG, "lin_forward_deferred_norm %s: n_stats_out is null", name);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    DecodeNorm nm;
    nm.ldx = ldx;
    nm.stats_in = stats_in_dev;
    nm.n_stats_in = n_stats_in;
    nm.in_cols = in_cols;
    nm.stats_out = stats_out_dev;
    nm.stat_rows = stat_rows;
    nm.resid = resid_dev;
    nm.nw = nw_dev;
    nm.in_exp = in_exp;
    nm.out_exp = out_exp;
    if (t <= 16) {
        W4_TRY(launch_decode(ctx, *L, x_dev, y_dev, t, out_f16, &nm));
    } else {
        // beyond the decode regime the MFMA-tiled kernel carries the same options in its epilogue (statistics arrays
        // are then [entries][t rounded up to 4] floats); it needs scales it can divide by
        if (!L->scales_regular)
            return w4_fail(W4A16_ERR_UNSUPPORTED, "lin_forward_deferred_norm %s: t=%zu runs the MFMA-tiled kernel, which cannot take this linear's zero, non-finite or out-of-range scale", name, t);
        W4_TRY(launch_prefill(ctx, *L, x_dev, y_dev, t, out_f16, -1, &nm));
    }
    if (n_stats_out) *n_stats_out = nm.n_stats_out;
    return 0;
}

extern "C" int w4a16_lin_forward_glu_deferred_norm(w4a16_ctx* ctx, const char* name, uint64_t x_dev, size_t ldx, size_t t,
                                                   uint64_t stats_in_dev, size_t n_stats_in, size_t in_cols,
                                                   uint64_t y_f16_dev, int act) {
    return w4a16_lin_forward_glu_deferred_norm_scaled(ctx, name, x_dev, ldx, t, stats_in_dev, n_stats_in, in_cols, 0,
                                                      y_f16_dev, 0, act);
}

extern "C" int w4a16_lin_forward_glu_deferred_norm_scaled(w4a16_ctx* ctx, const char* name, uint64_t x_dev, size_t ldx,
                                                          size_t t, uint64_t stats_in_dev, size_t n_stats_in,
                                                          size_t in_cols, int in_exp, uint64_t y_f16_dev, int out_exp,
                                                          int act) {
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (!x_dev || !y_f16_dev || t == 0) return w4_fail(W4A16_ERR_ARG, "lin_forward_glu_deferred_norm %s: null operand or t=0", name);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    DecodeNorm nm;
    nm.ldx = ldx;
    nm.stats_in = stats_in_dev;
    nm.n_stats_in = n_stats_in;
    nm.in_cols = in_cols;
    nm.act = act;
    nm.in_exp = in_exp;
    nm.out_exp = out_exp;
    if (t <= 16) return launch_decode_glu(ctx, *L, x_dev, y_f16_dev, t, &nm);
    if (act != W4A16_ACT_SILU && act != W4A16_ACT_GELU_TANH)
        return w4_fail(W4A16_ERR_ARG, "lin_forward_glu_deferred_norm %s: activation %d (0 = silu, 1 = gelu, tanh form)", name, act);
    if (!L->scales_regular)
        return w4_fail(W4A16_ERR_UNSUPPORTED, "lin_forward_glu_deferred_norm %s: t=%zu runs the MFMA-tiled kernel, which cannot take this linear's zero, non-finite or out-of-range scale", name, t);
    return launch_prefill(ctx, *L, x_dev, y_f16_dev, t, 1, act, &nm);
}

extern "C" int w4a16_lin_forward_host(w4a16_ctx* ctx, const char* name, const uint16_t* x_f16, void* y, size_t t,
                                      int out_f16, int path) {
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (!x_f16 || !y || t == 0) return w4_fail(W4A16_ERR_ARG, "lin_forward_host %s: null operand or t=0", name);
    const size_t xb = t * L->k * 2, yb = t * L->n * (out_f16 ? 2 : 4);
    uint64_t dx = 0, dy = 0;
    int rc = w4a16_alloc(ctx, xb, &dx);
    if (!rc) rc = w4a16_alloc(ctx, yb, &dy);
    if (!rc) rc = w4a16_h2d(ctx, dx, x_f16, xb);
    if (!rc) rc = w4a16_lin_forward(ctx, name, dx, dy, t, out_f16, path);
    if (!rc) rc = w4a16_d2h(ctx, y, dy, yb);
    const std::string keep = w4_err_save();
    (void)w4a16_free(ctx, dx);
    (void)w4a16_free(ctx, dy);
    if (rc) w4_err_restore(keep);
    return rc;
}

extern "C" int w4a16_dequant_dump(w4a16_ctx* ctx, const char* name, int from_tiled, uint64_t out_f32_dev) {
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (!out_f32_dev) return w4_fail(W4A16_ERR_ARG, "dequant_dump %s: null output", name);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    int ni = (int)L->n, ki = (int)L->k, gi = (int)L->group, rbi = (int)L->row_blocks;
    if (from_tiled) {
        if (!L->q_tiled) return w4_fail(W4A16_ERR_NOT_FOUND, "lin %s: no tiled copy", name);
        void* p[] = {&L->q_tiled, &L->s_tiled, &out_f32_dev, &ni, &ki, &gi, &rbi};
        return w4_launch(ctx, L->scale_bf16 ? "w4a16_dump_tiled_bf16" : "w4a16_dump_tiled_f16",
                         ceil_div(L->row_blocks * (L->k / 128) * 256, 256), 1, 256, 0, p);
    }
    if (!L->q_raw) return w4_fail(W4A16_ERR_NOT_FOUND, "lin %s: operands as given were dropped", name);
    void* p[] = {&L->q_raw, &L->s_raw, &out_f32_dev, &ni, &ki, &gi};
    return w4_launch(ctx, L->scale_bf16 ? "w4a16_dump_raw_bf16" : "w4a16_dump_raw_f16", ceil_div(L->n * (L->k / 8), 256),
                     1, 256, 0, p);
}

extern "C" int w4a16_lin_untile(w4a16_ctx* ctx, const char* name, uint64_t q_out_dev, uint64_t s_out_dev) {
    W4Lin* L = nullptr;
    W4_TRY(w4_find_lin(ctx, name, &L));
    if (!q_out_dev || !s_out_dev) return w4_fail(W4A16_ERR_ARG, "lin_untile %s: null output", name);
    if (!L->q_tiled) return w4_fail(W4A16_ERR_NOT_FOUND, "lin %s: no tiled copy", name);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    int ni = (int)L->n, ki = (int)L->k, kgi = (int)(L->k / L->group);
    void* pq[] = {&L->q_tiled, &q_out_dev, &ni, &ki};
    W4_TRY(w4_launch(ctx, "w4a16_untile_q", ceil_div(L->n * (L->k / 8), 256), 1, 256, 0, pq));
    void* ps[] = {&L->s_tiled, &s_out_dev, &ni, &kgi};
    return w4_launch(ctx, "w4a16_untile_s", ceil_div(L->n * (L->k / L->group), 256), 1, 256, 0, ps);
}

extern "C" int w4a16_set_prefill_ksplit(w4a16_ctx* ctx, int ksplit) {
    if (!ctx) return w4_fail(W4A16_ERR_ARG, "set_prefill_ksplit: null context");
    if (ksplit < -1 || ksplit > 16) return w4_fail(W4A16_ERR_ARG, "set_prefill_ksplit: -1 (never), 0 (automatic) or 1..16");
    ctx->prefill_ksplit = ksplit;
    return 0;
}

extern "C" int w4a16_set_decode_shape(w4a16_ctx* ctx, int rows_per_wave, int waves_per_block) {
    if (!ctx) return w4_fail(W4A16_ERR_ARG, "set_decode_shape: null context");
    if ((rows_per_wave != 0 && rows_per_wave != 16 && rows_per_wave != 32 && rows_per_wave != 64) ||
        waves_per_block < 0 || waves_per_block > 8)
        return w4_fail(W4A16_ERR_ARG, "set_decode_shape: rows_per_wave in {0,16,32,64}, waves_per_block in 0..8");
    ctx->decode_rows_per_wave = rows_per_wave;
    ctx->decode_waves_per_block = waves_per_block;
    return 0;
}

extern "C" int w4a16_set_prefill_tile(w4a16_ctx* ctx, int rows) {
    if (!ctx) return w4_fail(W4A16_ERR_ARG, "set_prefill_tile: null context");
    if (rows != 0 && rows != 64 && rows != 96 && rows != 128) return w4_fail(W4A16_ERR_ARG, "set_prefill_tile: 0 = automatic, 64, 96 or 128 rows");
    ctx->prefill_tile_m = rows;
    return 0;
}

extern "C" int w4a16_set_decode_ksplit(w4a16_ctx* ctx, int ksplit) {
    if (!ctx) return w4_fail(W4A16_ERR_ARG, "set_decode_ksplit: null context");
    if (ksplit < -1 || ksplit > kW4DecodeMaxKsplit)
        return w4_fail(W4A16_ERR_ARG, "set_decode_ksplit: -1 = never, 0 = automatic, 1..%d slices", kW4DecodeMaxKsplit);
    ctx->decode_ksplit = ksplit;
    return 0;
}

// ------------------------------------------------------------------------------------------------ bench probe
extern "C" int w4a16_bench_forward(w4a16_ctx* ctx, const char* const* names, size_t n_names, uint64_t x_dev,
                                   uint64_t y_dev, size_t t, int out_f16, int path, size_t warmup, size_t reps,
                                   float* ms_events, double* ms_wall) {
    if (!ctx || !names || n_names == 0 || reps == 0) return w4_fail(W4A16_ERR_ARG, "bench_forward: null argument");
    W4Lin* first = nullptr;
    W4_TRY(w4_find_lin(ctx, names[0], &first));
    for (size_t i = 1; i < n_names; i++) {
        W4Lin* L = nullptr;
        W4_TRY(w4_find_lin(ctx, names[i], &L));
        if (L->n != first->n || L->k != first->k || L->group != first->group)
            return w4_fail(W4A16_ERR_SHAPE, "bench_forward: %s and %s differ in shape", names[0], names[i]);
    }
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    W4_TRY(w4_hip(hipEventCreate(&e0), "hipEventCreate"));
    int rc = w4_hip(hipEventCreate(&e1), "hipEventCreate");
    for (size_t i = 0; i < warmup && !rc; i++)
        rc = w4a16_lin_forward(ctx, names[i % n_names], x_dev, y_dev, t, out_f16, path);
    if (!rc) rc = w4_hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    auto w0 = std::chrono::steady_clock::now();
    if (!rc) rc = w4_hip(hipEventRecord(e0, ctx->stream), "hipEventRecord");
    for (size_t i = 0; i < reps && !rc; i++)
        rc = w4a16_lin_forward(ctx, names[(warmup + i) % n_names], x_dev, y_dev, t, out_f16, path);
    if (!rc) rc = w4_hip(hipEventRecord(e1, ctx->stream), "hipEventRecord");
    if (!rc) rc = w4_hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    auto w1 = std::chrono::steady_clock::now();
    float ms = 0.f;
    if (!rc) rc = w4_hip(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
    if (ms_events) *ms_events = ms;
    if (ms_wall) *ms_wall = std::chrono::duration<double, std::milli>(w1 - w0).count();
    const std::string keep = w4_err_save();
    (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (rc) w4_err_restore(keep);
    return rc;
}
