// MoE layer of libw4a16hip.so: expert arenas, routing, slot alignment and the routed-expert FFN.
// Stands in for build_marlin_moe_arenas (w4a16_dec/upload.rs:1116-1235), moe_topk (w4a16_dec/mod.rs:168-185),
// moe_align_launch (moe/moe_align.rs:4-22) and marlin_moe_ffn_dev (kernels/marlin_moe.rs:290-422).
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>

#include "w4a16_internal.h"

static inline unsigned ceil_div(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

// ------------------------------------------------------------------------------------------------ arenas
static void free_experts(w4a16_ctx* ctx, W4Experts& E) {
    (void)w4a16_free(ctx, E.q13);
    (void)w4a16_free(ctx, E.s13);
    (void)w4a16_free(ctx, E.q2);
    (void)w4a16_free(ctx, E.s2);
    E = W4Experts();
}

// Tile one projection of every expert: raw [n_exp][n][k/8] + [n_exp][n][k/group] on the host -> arena on the device.
static int tile_arena(w4a16_ctx* ctx, const void* q, const void* s, size_t n_exp, size_t n, size_t k, size_t group,
                      uint64_t* q_arena, uint64_t* s_arena, size_t* q_stride, size_t* s_stride) {
    const size_t row_blocks = (n + 15) / 16, kt_n = k / 128, kg_n = k / group;
    const size_t q_raw_e = n * (k / 2), s_raw_e = n * kg_n * 2;
    *q_stride = row_blocks * kt_n * 1024;
    *s_stride = row_blocks * kg_n * 32;
    W4_TRY(w4a16_alloc(ctx, *q_stride * n_exp, q_arena));
    W4_TRY(w4a16_alloc(ctx, *s_stride * n_exp, s_arena));
    // stage the operands through a bounded device buffer, a few experts at a time
    const size_t per = std::max<size_t>(1, std::min<size_t>(n_exp, (size_t)(256u << 20) / (q_raw_e + s_raw_e)));
    uint64_t dq = 0, ds = 0;
    int rc = w4a16_alloc(ctx, per * q_raw_e, &dq);
    if (!rc) rc = w4a16_alloc(ctx, per * s_raw_e, &ds);
    for (size_t e0 = 0; e0 < n_exp && !rc; e0 += per) {
        const size_t cnt = std::min(per, n_exp - e0);
        rc = w4a16_h2d(ctx, dq, static_cast<const char*>(q) + e0 * q_raw_e, cnt * q_raw_e);
        if (!rc) rc = w4a16_h2d(ctx, ds, static_cast<const char*>(s) + e0 * s_raw_e, cnt * s_raw_e);
        for (size_t i = 0; i < cnt && !rc; i++) {
            uint64_t qr = dq + i * q_raw_e, sr = ds + i * s_raw_e;
            uint64_t qt = *q_arena + (e0 + i) * *q_stride, st = *s_arena + (e0 + i) * *s_stride;
            int ni = (int)n, ki = (int)k, rbi = (int)row_blocks, kgi = (int)kg_n;
            void* pq[] = {&qr, &qt, &ni, &ki, &rbi};
            rc = w4_launch(ctx, "w4a16_tile_q", ceil_div(*q_stride / 4, 256), 1, 256, 0, pq);
            void* ps[] = {&sr, &st, &ni, &kgi, &rbi};
            if (!rc) rc = w4_launch(ctx, "w4a16_tile_s", ceil_div(*s_stride / 2, 256), 1, 256, 0, ps);
        }
        if (!rc) rc = w4a16_sync(ctx);  // the staging buffer is reused by the next batch
    }
    const std::string keep = w4_err_save();
    (void)w4a16_free(ctx, dq);
    (void)w4a16_free(ctx, ds);
    if (rc) w4_err_restore(keep);
    return rc;
}

extern "C" int w4a16_upload_experts(w4a16_ctx* ctx, const char* name, size_t n_experts, const void* q13,
                                    size_t q13_bytes, const void* s13, size_t s13_bytes, const void* q2,
                                    size_t q2_bytes, const void* s2, size_t s2_bytes, size_t h, size_t n_ff,
                                    size_t group, int scale_bf16) {
    if (!ctx || !name || !q13 || !s13 || !q2 || !s2) return w4_fail(W4A16_ERR_ARG, "upload_experts: null argument");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    if (group != 128 && group != 32)
        return w4_fail(W4A16_ERR_UNSUPPORTED, "upload_experts %s: unsupported group=%zu", name, group);
    if (n_experts == 0 || n_experts > 1024 || h == 0 || n_ff == 0 || h % 128 != 0 || n_ff % 128 != 0)
        return w4_fail(W4A16_ERR_SHAPE, "upload_experts %s: experts=%zu h=%zu n_ff=%zu (1..1024 experts, h and n_ff multiples of 128)",
                       name, n_experts, h, n_ff);
    if (q13_bytes != n_experts * 2 * n_ff * (h / 2) || s13_bytes != n_experts * 2 * n_ff * (h / group) * 2 ||
        q2_bytes != n_experts * h * (n_ff / 2) || s2_bytes != n_experts * h * (n_ff / group) * 2)
        return w4_fail(W4A16_ERR_SHAPE, "upload_experts %s: q13=%zu s13=%zu q2=%zu s2=%zu != experts%zu h%zu n_ff%zu g%zu contract",
                       name, q13_bytes, s13_bytes, q2_bytes, s2_bytes, n_experts, h, n_ff, group);
    if (2 * n_ff * (h / 2) >= 0x80000000ull || h * (n_ff / 2) >= 0x80000000ull)
        return w4_fail(W4A16_ERR_SHAPE, "upload_experts %s: one expert reaches 2 GiB", name);
    W4Experts E;
    E.n_exp = n_experts;
    E.h = h;
    E.n_ff = n_ff;
    E.group = group;
    E.scale_bf16 = scale_bf16 ? 1 : 0;
    // the MFMA-tiled grouped kernels carry the running unit of the prefill kernel: they are taken only for arenas
    // whose every scale that kernel can divide by (the streaming kernels only multiply by scales and take any)
    E.scales_regular = w4_scales_regular(static_cast<const uint16_t*>(s13), s13_bytes / 2, scale_bf16) &&
                       w4_scales_regular(static_cast<const uint16_t*>(s2), s2_bytes / 2, scale_bf16);
    int rc = tile_arena(ctx, q13, s13, n_experts, 2 * n_ff, h, group, &E.q13, &E.s13, &E.q13_stride, &E.s13_stride);
    if (!rc) rc = tile_arena(ctx, q2, s2, n_experts, h, n_ff, group, &E.q2, &E.s2, &E.q2_stride, &E.s2_stride);
    if (rc) {
        const std::string keep = w4_err_save();
        free_experts(ctx, E);
        w4_err_restore(keep);
        return rc;
    }
    auto it = ctx->experts.find(name);
    if (it != ctx->experts.end()) free_experts(ctx, it->second);
    ctx->experts[name] = E;
    return 0;
}

static int find_experts(w4a16_ctx* ctx, const char* name, W4Experts** out) {
    if (!ctx || !name) return w4_fail(W4A16_ERR_ARG, "experts: null argument");
    auto it = ctx->experts.find(name);
    if (it == ctx->experts.end()) return w4_fail(W4A16_ERR_NOT_FOUND, "experts %s: not registered", name);
    *out = &it->second;
    return 0;
}

extern "C" int w4a16_experts_info(w4a16_ctx* ctx, const char* name, size_t* n_experts, size_t* h, size_t* n_ff,
                                  size_t* group, int* scale_bf16) {
    W4Experts* E = nullptr;
    W4_TRY(find_experts(ctx, name, &E));
    if (n_experts) *n_experts = E->n_exp;
    if (h) *h = E->h;
    if (n_ff) *n_ff = E->n_ff;
    if (group) *group = E->group;
    if (scale_bf16) *scale_bf16 = E->scale_bf16;
    return 0;
}

extern "C" int w4a16_experts_dequant_dump(w4a16_ctx* ctx, const char* name, int which, size_t expert,
                                          uint64_t out_f32_dev) {
    W4Experts* E = nullptr;
    W4_TRY(find_experts(ctx, name, &E));
    if (!out_f32_dev || (which != 0 && which != 1) || expert >= E->n_exp)
        return w4_fail(W4A16_ERR_ARG, "experts_dequant_dump %s: which=%d expert=%zu", name, which, expert);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    const size_t n = which == 0 ? 2 * E->n_ff : E->h, k = which == 0 ? E->h : E->n_ff;
    uint64_t qt = (which == 0 ? E->q13 + expert * E->q13_stride : E->q2 + expert * E->q2_stride);
    uint64_t st = (which == 0 ? E->s13 + expert * E->s13_stride : E->s2 + expert * E->s2_stride);
    int ni = (int)n, ki = (int)k, gi = (int)E->group, rbi = (int)((n + 15) / 16);
    void* p[] = {&qt, &st, &out_f32_dev, &ni, &ki, &gi, &rbi};
    return w4_launch(ctx, E->scale_bf16 ? "w4a16_dump_tiled_bf16" : "w4a16_dump_tiled_f16",
                     ceil_div((size_t)rbi * (k / 128) * 256, 256), 1, 256, 0, p);
}

// ------------------------------------------------------------------------------------------------ routing
extern "C" int w4a16_moe_topk_host(const float* logits, size_t t, size_t n_exp, size_t top_k, int32_t* idx, float* w) {
    if (!logits || !idx || !w) return w4_fail(W4A16_ERR_ARG, "moe_topk: null argument");
    if (n_exp == 0 || top_k == 0 || top_k > n_exp)
        return w4_fail(W4A16_ERR_SHAPE, "moe_topk: n_exp=%zu top_k=%zu", n_exp, top_k);
    std::vector<float> p(n_exp);
    std::vector<char> taken(n_exp);
    for (size_t ti = 0; ti < t; ti++) {
        const float* l = logits + ti * n_exp;
        float mx = -INFINITY;
        for (size_t i = 0; i < n_exp; i++) mx = std::fmax(mx, l[i]);
        float sum = 0.0f;
        for (size_t i = 0; i < n_exp; i++) {
            p[i] = std::exp(l[i] - mx);
            sum += p[i];
        }
        for (size_t i = 0; i < n_exp; i++) p[i] /= sum;
        std::fill(taken.begin(), taken.end(), 0);
        float wsum = 0.0f;
        for (size_t r = 0; r < top_k; r++) {  // descending probability, ties to the lower index
            size_t best = n_exp;
            for (size_t i = 0; i < n_exp; i++)
                if (!taken[i] && (best == n_exp || p[i] > p[best])) best = i;
            taken[best] = 1;
            idx[ti * top_k + r] = (int32_t)best;
            wsum += p[best];
        }
        for (size_t r = 0; r < top_k; r++) w[ti * top_k + r] = p[(size_t)idx[ti * top_k + r]] / wsum;
    }
    return 0;
}

extern "C" int w4a16_moe_route(w4a16_ctx* ctx, uint64_t logits_dev, size_t t, size_t n_exp, size_t top_k,
                               uint64_t idx_dev, uint64_t wt_dev) {
    if (!ctx || !logits_dev || !idx_dev || !wt_dev) return w4_fail(W4A16_ERR_ARG, "moe_route: null argument");
    if (t == 0 || n_exp == 0 || n_exp > 1024 || top_k == 0 || top_k > 64 || top_k > n_exp || t > 0x7fffffffu / n_exp)
        return w4_fail(W4A16_ERR_SHAPE, "moe_route: t=%zu n_exp=%zu top_k=%zu (n_exp <= 1024, top_k <= min(64, n_exp))", t,
                       n_exp, top_k);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    int ti = (int)t, ni = (int)n_exp, ki = (int)top_k;
    void* p[] = {&logits_dev, &idx_dev, &wt_dev, &ti, &ni, &ki};
    return w4_launch(ctx, "w4a16_moe_topk_t", ceil_div(t, 4), 1, 256, 0, p);
}

extern "C" int w4a16_moe_align(w4a16_ctx* ctx, uint64_t idx_dev, size_t ns, size_t n_exp, size_t block,
                               uint64_t sorted_dev, uint64_t expert_ids_dev, uint64_t num_post_dev) {
    if (!ctx || !idx_dev || !sorted_dev || !expert_ids_dev || !num_post_dev)
        return w4_fail(W4A16_ERR_ARG, "moe_align: null argument");
    if (ns == 0 || ns > 0x3fffffffu || n_exp == 0 || n_exp > 1024 || block == 0 || block > 1024)
        return w4_fail(W4A16_ERR_SHAPE, "moe_align: ns=%zu n_exp=%zu block=%zu", ns, n_exp, block);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    int nsi = (int)ns, ni = (int)n_exp, bi = (int)block;
    void* p[] = {&idx_dev, &nsi, &ni, &bi, &sorted_dev, &expert_ids_dev, &num_post_dev};
    // LDS: 16 per-wave count rows, totals and offsets, one entry per expert each
    return w4_launch(ctx, "w4a16_moe_align", 1, 1, 64 * kW4MoeAlignWaves, (unsigned)((kW4MoeAlignWaves + 2) * n_exp * 4), p);
}

// ------------------------------------------------------------------------------------------------ FFN
int w4_ensure(w4a16_ctx* ctx, uint64_t* buf, size_t* cap, size_t bytes) {
    if (bytes <= *cap) return 0;
    if (ctx->capturing)
        return w4_fail(W4A16_ERR_ARG, "a scratch buffer would grow to %zu bytes while the launch stream is capturing: run the sequence once before the capture", bytes);
    if (*buf) {
        W4_TRY(w4a16_sync(ctx));  // earlier launches may still read the old buffer
        ctx->scratch_gen++;       // graphs captured so far hold its address: w4a16_graph_launch refuses them from now on
    }
    (void)w4a16_free(ctx, *buf);
    *buf = 0;
    *cap = 0;
    W4_TRY(w4a16_alloc(ctx, bytes, buf));
    *cap = bytes;
    return 0;
}

// Segment size (slots of one expert per workgroup).  Up to 15 tokens (top_k <= 8) skip the alignment; otherwise up to 8
// tokens run the streaming kernel on 16-slot segments; beyond that the LDS-staged kernel, whose segment size follows
// the mean run per expert: 32 slots below a mean of 24, 48 below 40, else 64.  The reference picks the smallest of
// 16/32/48/64 that the mean run fills to under 90 % (kernels/marlin_moe.rs:309-315); measured here (128 experts,
// top-8, T = 16..1024) 32-slot segments beat 16-slot ones at every T, and the larger sizes win once most experts would
// need a second segment.
static size_t pick_block(const w4a16_ctx* ctx, size_t t, size_t ns, size_t n_exp, size_t top_k) {
    if (ctx->moe_block) return (size_t)ctx->moe_block;
    // direct mode (no alignment, two launches, see w4a16_moe_ffn): streams an expert once per token that chose it,
    // which still beats the two extra launches up to fifteen tokens (128 experts, top-8: 35.6 vs 52.9 us at t = 8,
    // 49.3 vs 61.3 us at t = 12, 62.9 vs 64.7 us at t = 15, level at t = 16, 79.3 vs 65.4 us at t = 20)
    if (t <= 15 && top_k <= 8) return 1;
    if (t <= 4) return 4;
    if (t <= 8) return 16;
    const double mean = (double)ns / (double)n_exp;
    return mean < 24.0 ? 32 : mean < 40.0 ? 48 : 64;
}

static int launch_moe_gemm(w4a16_ctx* ctx, const W4Experts& E, bool glu, uint64_t x, size_t x_rows, size_t x_div,
                           uint64_t y, int y_f16, uint64_t topw, size_t ns, size_t block, size_t max_segs,
                           uint64_t sorted, uint64_t eids, uint64_t npost, size_t nks = 1, bool tiled = false) {
    const size_t n = glu ? 2 * E.n_ff : E.h, k = glu ? E.h : E.n_ff;
    const size_t row_blocks = (n + 15) / 16, kt_n = k / 128;
    const size_t units = glu ? row_blocks / 2 : (row_blocks + 1) / 2;
    if (x_rows * k * 2 >= 0x80000000ull)
        return w4_fail(W4A16_ERR_SHAPE, "moe: activations reach 2 GiB, beyond the buffer-descriptor range");
    uint64_t qa = glu ? E.q13 : E.q2, sa = glu ? E.s13 : E.s2;
    unsigned long long qs = glu ? E.q13_stride : E.q2_stride, ss = glu ? E.s13_stride : E.s2_stride;
    int xr = (int)x_rows, xd = (int)x_div, yf = y_f16, blk = (int)block, nsi = (int)ns, rbi = (int)row_blocks,
        ki = (int)k, ni = (int)n, nei = (int)E.n_exp;
    uint64_t ws = 0, tk = 0;
    int waves = 0;  // set below, before the launch reads it
    int act_kind = ctx->moe_act_kind;  // read by the gate|up kernels only
    void* p[] = {&qa, &sa, &qs, &ss, &x, &xr, &xd, &y, &yf, &topw, &sorted, &eids, &npost, &blk, &nsi, &rbi, &ki, &ni, &nei,
                 &ws, &tk, &waves, &act_kind};
    char sym[80];
    const char* fam = E.scale_bf16 ? "bf16" : "f16";
    if (tiled) {
        // MFMA-tiled grouped kernel (kernels/prefill.hip, MODE 1 / 2): block tile = one 64-slot segment x 256 columns
        // (gate|up: 128 gate + the 128 matching up columns); LDS = two x stages of 64 rows x 64 k and the slot ids
        if (block != 64) return w4_fail(W4A16_ERR_ARG, "moe: the tiled grouped kernel needs 64-slot segments (got %zu)", block);
        if (max_segs > 65535) return w4_fail(W4A16_ERR_SHAPE, "moe: %zu segments exceed the grid", max_segs);
        const size_t cols = glu ? E.n_ff : n, per_tile = glu ? 128 : 256;
        snprintf(sym, sizeof sym, "w4a16_moe_g%zu_%s_pf_%s", E.group, fam, glu ? "glu" : "lin");
        return w4_launch(ctx, sym, (unsigned)((cols + per_tile - 1) / per_tile), (unsigned)max_segs, 256, 2 * 64 * 64 * 2 + 256, p);
    }
    if (block <= 16) {
        // in-block split-K: each wave needs at least one k tile
        waves = ctx->moe_waves ? ctx->moe_waves : 4;
        waves = std::max(1, std::min(std::min(waves, 8), (int)kt_n));
        snprintf(sym, sizeof sym, "w4a16_moe_g%zu_%s_dec_%s_x%d", E.group, fam, glu ? "glu" : "lin", block <= 4 ? 1 : 4);
        const unsigned shmem = waves > 1 ? (unsigned)(waves * 2 * 64 * 16) : 0;
        return w4_launch(ctx, sym, (unsigned)(max_segs * units), 1, (unsigned)(waves * 64), shmem, p);
    }
    const int tt = (int)(block / 16);
    waves = ctx->moe_waves ? ctx->moe_waves : 4;
    waves = waves >= 8 ? 8 : 4;  // the x staging needs at least 4 waves
    const size_t blocks = max_segs * ((units + (size_t)waves - 1) / (size_t)waves);
    nks = std::max<size_t>(1, std::min<size_t>(std::min<size_t>(nks, kW4MoeMaxKsplit), kt_n / 2));
    if (nks > 1) {
        // split over k across workgroups: partial tiles and per-(block, wave) tickets, shared with the decode kernel
        W4_TRY(w4_ensure(ctx, &ctx->decode_ws, &ctx->decode_ws_cap, blocks * (size_t)waves * 2 * (size_t)tt * 1024 * nks));
        if (blocks * (size_t)waves * 4 > ctx->decode_tickets_cap) {
            W4_TRY(w4_ensure(ctx, &ctx->decode_tickets, &ctx->decode_tickets_cap,
                             std::max<size_t>(blocks * (size_t)waves * 4, 16384)));
            W4_TRY(w4a16_memset0(ctx, ctx->decode_tickets, ctx->decode_tickets_cap));
        }
        ws = ctx->decode_ws;
        tk = ctx->decode_tickets;
    }
    if (nks > 1 && glu) return w4_fail(W4A16_ERR_UNSUPPORTED, "moe: the gate|up kernel does not split over k");
    snprintf(sym, sizeof sym, "w4a16_moe_g%zu_%s_mm_%s_t%d%s", E.group, fam, glu ? "glu" : "lin", tt, nks > 1 ? "_ks" : "");
    const unsigned shmem = (unsigned)(2 * 16 * tt * kW4MoeLdx * 2);
    return w4_launch(ctx, sym, (unsigned)blocks, (unsigned)nks, (unsigned)(waves * 64), shmem, p);
}

// A dense linear at a few dozen rows through the LDS-staged grouped kernel: one "expert" (the linear itself), slot =
// token, segments of up to 64 tokens.  Between the streaming decode kernel (t <= 16: x operands straight from global
// memory) and the 128-row MFMA tiles of the prefill kernel, this regime is still bound by the weight stream, and the
// grouped kernel shares each x tile among all waves of a workgroup through LDS.
int w4_dense_grouped(w4a16_ctx* ctx, const W4Lin& L, uint64_t x_dev, uint64_t y_dev, size_t t, int out_f16, int glu_act) {
    if (!L.q_tiled) return w4_fail(W4A16_ERR_UNSUPPORTED, "stream: linear has no tiled copy (needs k %% 128 == 0)");
    if (t > 0x7fffffffu / 2) return w4_fail(W4A16_ERR_SHAPE, "stream: t=%zu too large", t);
    W4MoeScratch& S = ctx->moe;
    const size_t block = ctx->moe_block >= 16 ? (size_t)ctx->moe_block : t <= 16 ? 16 : t <= 32 ? 32 : t <= 48 ? 48 : 64;
    const size_t segs = (t + block - 1) / block, padded = segs * block;
    // identity slot table (entries >= t are the padding sentinel by themselves), all-zero expert table, padded total
    if (S.iota_cap < padded) {
        const size_t cap = std::max<size_t>(padded, 4096);
        std::vector<int32_t> host(cap);
        for (size_t i = 0; i < cap; i++) host[i] = (int32_t)i;
        size_t bytes_cap = S.iota_cap * 4;
        W4_TRY(w4_ensure(ctx, &S.iota, &bytes_cap, cap * 4));
        W4_TRY(w4a16_h2d(ctx, S.iota, host.data(), cap * 4));
        S.iota_cap = cap;
    }
    if (S.zeros_cap < segs) {
        const size_t cap = std::max<size_t>(segs, 1024);
        size_t bytes_cap = S.zeros_cap * 4;
        W4_TRY(w4_ensure(ctx, &S.zeros, &bytes_cap, cap * 4));
        W4_TRY(w4a16_memset0(ctx, S.zeros, cap * 4));
        S.zeros_cap = cap;
    }
    if (!S.always) {
        const int32_t big[2] = {0x7fffffff, 0};
        W4_TRY(w4a16_alloc(ctx, 8, &S.always));
        W4_TRY(w4a16_h2d(ctx, S.always, big, 8));
    }
    const bool glu = glu_act >= 0;
    W4Experts E;
    E.n_exp = 1;
    E.group = L.group;
    E.scale_bf16 = L.scale_bf16;
    if (glu) {  // the linear is the "gate|up arena" of its one expert: n = 2 n_ff rows over k = h
        if (L.n % 32 != 0) return w4_fail(W4A16_ERR_SHAPE, "stream glu: n=%zu must be a multiple of 32", L.n);
        E.q13 = L.q_tiled;
        E.s13 = L.s_tiled;
        E.h = L.k;
        E.n_ff = L.n / 2;
    } else {
        E.q2 = L.q_tiled;
        E.s2 = L.s_tiled;
        E.h = L.n;
        E.n_ff = L.k;
    }
    // k slices until the launch has a few workgroups per CU
    const size_t waves = ctx->moe_waves >= 8 ? 8 : 4, units = glu ? L.row_blocks / 2 : (L.row_blocks + 1) / 2;
    const size_t groups = (units + waves - 1) / waves;
    size_t nks = 1;
    if (glu) {
        nks = 1;  // the gated kernel does not split over k
    } else if (ctx->decode_ksplit > 0) {
        nks = (size_t)ctx->decode_ksplit;
    } else if (ctx->decode_ksplit == 0) {
        // only while the launch has fewer workgroups than CUs: the 27B down projection (40 unit groups) runs 8 slices
        // (78 -> 22 us at t = 32), the wide gate|up (272 groups) none (slices cost it 1-3 us, measured)
        while (groups * segs * nks < (size_t)std::max(ctx->cu_count, 1) && nks < 8) nks *= 2;
    }
    // the grid covers exactly `segs` segments, so the "padded total" may be the constant no segment start reaches
    if (glu) {
        // bit 1: the activation takes the f32 sums (the expert FFN rounds gate and up to f16 first)
        const int keep = ctx->moe_act_kind;
        ctx->moe_act_kind = glu_act | 2;
        const int rc = launch_moe_gemm(ctx, E, true, x_dev, t, 1, y_dev, 1, 0, t, block, segs, S.iota, S.zeros, S.always, 1);
        ctx->moe_act_kind = keep;
        return rc;
    }
    return launch_moe_gemm(ctx, E, false, x_dev, t, 1, y_dev, out_f16, 0, t, block, segs, S.iota, S.zeros, S.always, nks);
}

// Direct mode for decode steps: no alignment pass.  The gate|up GEMM runs one segment per slot — the segment table is
// the identity, the expert table is idx itself, the "padded total" a constant no slot index reaches — and
// w4a16_moe_*_down_sum folds the down projection of a token's experts, the routing-weight multiply, the f16 rounding
// of c2 and the slot-order sum into one launch of top_k waves per block.  Experts chosen by several tokens are
// streamed once per token, which is cheaper than the two extra launches for a handful of tokens.
static int moe_ffn_direct(w4a16_ctx* ctx, const char* name, const W4Experts& E, uint64_t x_dev, uint64_t idx_dev,
                          uint64_t wt_dev, size_t t, size_t top_k, uint64_t y_dev) {
    if (top_k > 8) return w4_fail(W4A16_ERR_UNSUPPORTED, "moe_ffn %s: direct mode needs top_k <= 8 (got %zu)", name, top_k);
    const size_t ns = t * top_k;
    W4MoeScratch& S = ctx->moe;
    S.block = 1;
    S.sorted_len = S.expert_len = S.c2_len = 0;
    S.act_len = ns * E.n_ff * 2;
    W4_TRY(w4_ensure(ctx, &S.act, &S.act_cap, S.act_len));
    if (S.iota_cap < ns) {
        const size_t cap = std::max<size_t>(ns, 256);
        std::vector<int32_t> host(cap);
        for (size_t i = 0; i < cap; i++) host[i] = (int32_t)i;
        size_t bytes_cap = S.iota_cap * 4;
        W4_TRY(w4_ensure(ctx, &S.iota, &bytes_cap, cap * 4));
        W4_TRY(w4a16_h2d(ctx, S.iota, host.data(), cap * 4));
        S.iota_cap = cap;
    }
    if (!S.always) {
        const int32_t big[2] = {0x7fffffff, 0};
        W4_TRY(w4a16_alloc(ctx, 8, &S.always));
        W4_TRY(w4a16_h2d(ctx, S.always, big, 8));
    }
    // gate|up with the SiLU*up epilogue, one slot per segment
    W4_TRY(launch_moe_gemm(ctx, E, true, x_dev, t, top_k, S.act, 1, 0, ns, 1, ns, S.iota, idx_dev, S.always));
    // down + routing weight + f16 rounding + slot-order sum
    // units of one row block while units of two would leave CUs without a workgroup
    const size_t row_blocks = (E.h + 15) / 16;
    const size_t rbu = (ctx->moe_waves == 2 || (ctx->moe_waves == 0 && t * ((row_blocks + 1) / 2) < (size_t)std::max(ctx->cu_count, 1))) ? 1 : 2;
    const size_t units = (row_blocks + rbu - 1) / rbu;
    uint64_t qa = E.q2, sa = E.s2;
    unsigned long long qs = E.q2_stride, ss = E.s2_stride;
    int tk = (int)top_k, nsi = (int)ns, rbi = (int)row_blocks, ki = (int)E.n_ff, ni = (int)E.h, nei = (int)E.n_exp;
    void* p[] = {&qa, &sa, &qs, &ss, &S.act, &idx_dev, &wt_dev, &y_dev, &tk, &nsi, &rbi, &ki, &ni, &nei};
    char sym[80];
    snprintf(sym, sizeof sym, "w4a16_moe_g%zu_%s_down_sum%s", E.group, E.scale_bf16 ? "bf16" : "f16", rbu == 1 ? "1" : "");
    return w4_launch(ctx, sym, (unsigned)(t * units), 1, (unsigned)(top_k * 64), (unsigned)(top_k * rbu * 64 * 16), p);
}

extern "C" int w4a16_moe_ffn(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t idx_dev, uint64_t wt_dev,
                             size_t t, size_t top_k, uint64_t y_dev) {
    return w4a16_moe_ffn_act(ctx, name, x_dev, idx_dev, wt_dev, t, top_k, y_dev, W4A16_ACT_SILU);
}

extern "C" int w4a16_moe_ffn_act(w4a16_ctx* ctx, const char* name, uint64_t x_dev, uint64_t idx_dev, uint64_t wt_dev,
                                 size_t t, size_t top_k, uint64_t y_dev, int act) {
    W4Experts* E = nullptr;
    W4_TRY(find_experts(ctx, name, &E));
    if (!x_dev || !idx_dev || !wt_dev || !y_dev) return w4_fail(W4A16_ERR_ARG, "moe_ffn %s: null operand", name);
    if (act != W4A16_ACT_SILU && act != W4A16_ACT_GELU_TANH)
        return w4_fail(W4A16_ERR_ARG, "moe_ffn %s: activation %d (0 = silu, 1 = gelu, tanh form)", name, act);
    ctx->moe_act_kind = act;  // read by the gate|up launches of this call
    if (t == 0 || top_k == 0 || top_k > E->n_exp || t > 0x3fffffffu / top_k)
        return w4_fail(W4A16_ERR_SHAPE, "moe_ffn %s: t=%zu top_k=%zu experts=%zu", name, t, top_k, E->n_exp);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    const size_t ns = t * top_k;
    // From a mean run of 96 slots per expert on, 64-slot segments are mostly full and the MFMA-tiled grouped kernel
    // (one segment x 256 columns per workgroup, x through LDS, 32x32x16 tiles) takes over from the streaming kernels.
    if (ctx->moe_tiled > 0 && !E->scales_regular)
        return w4_fail(W4A16_ERR_UNSUPPORTED, "moe_ffn %s: the MFMA-tiled grouped kernels were requested (set_moe_tiled 1) but the experts hold a zero, non-finite or out-of-range scale; the streaming kernels serve them", name);
    const bool tiled = ctx->moe_tiled > 0 || (ctx->moe_tiled == 0 && ctx->moe_block == 0 && E->scales_regular && ns >= 96 * E->n_exp);
    const size_t block = tiled ? 64 : pick_block(ctx, t, ns, E->n_exp, top_k);
    if (block != 1 && block != 4 && block != 16 && block != 32 && block != 48 && block != 64)
        return w4_fail(W4A16_ERR_ARG, "moe_ffn %s: segment size %zu not in {1,4,16,32,48,64}", name, block);
    if (block == 1) return moe_ffn_direct(ctx, name, *E, x_dev, idx_dev, wt_dev, t, top_k, y_dev);
    // every expert's run is padded to a multiple of block: at most ns/block full segments plus one partial per expert
    const size_t max_segs = std::min(ns, ns / block + E->n_exp);
    W4MoeScratch& S = ctx->moe;
    S.block = block;
    S.sorted_len = (ns + E->n_exp * block) * 4;
    S.expert_len = (ns / block + E->n_exp + 1) * 4;
    S.act_len = ns * E->n_ff * 2;
    S.c2_len = ns * E->h * 2;
    W4_TRY(w4_ensure(ctx, &S.sorted, &S.sorted_cap, S.sorted_len));
    W4_TRY(w4_ensure(ctx, &S.expert_ids, &S.expert_cap, S.expert_len));
    size_t np_cap = S.num_post ? 8 : 0;
    W4_TRY(w4_ensure(ctx, &S.num_post, &np_cap, 8));
    W4_TRY(w4_ensure(ctx, &S.act, &S.act_cap, S.act_len));
    W4_TRY(w4_ensure(ctx, &S.c2, &S.c2_cap, S.c2_len));
    W4_TRY(w4a16_moe_align(ctx, idx_dev, ns, E->n_exp, block, S.sorted, S.expert_ids, S.num_post));
    // gate|up with the SiLU*up epilogue: slot j reads token j / top_k
    W4_TRY(launch_moe_gemm(ctx, *E, true, x_dev, t, top_k, S.act, 1, 0, ns, block, max_segs, S.sorted, S.expert_ids,
                           S.num_post, 1, tiled));
    // down, multiplied by the routing weight: slot j reads act row j
    W4_TRY(launch_moe_gemm(ctx, *E, false, S.act, ns, 1, S.c2, 1, wt_dev, ns, block, max_segs, S.sorted, S.expert_ids,
                           S.num_post, 1, tiled));
    int ti = (int)t, hi = (int)E->h, ki = (int)top_k;
    void* p[] = {&S.c2, &y_dev, &ti, &hi, &ki};
    return w4_launch(ctx, "w4a16_moe_topk_sum_f16", std::min<unsigned>(ceil_div(t * E->h / (E->h % 8 == 0 ? 8 : 1), 256), 4096), 1, 256, 0, p);
}

extern "C" int w4a16_moe_scratch(w4a16_ctx* ctx, int which, uint64_t* dptr, size_t* bytes, size_t* block) {
    if (!ctx || !dptr || !bytes) return w4_fail(W4A16_ERR_ARG, "moe_scratch: null argument");
    const W4MoeScratch& S = ctx->moe;
    switch (which) {
        case 0: *dptr = S.sorted; *bytes = S.sorted_len; break;
        case 1: *dptr = S.expert_ids; *bytes = S.expert_len; break;
        case 2: *dptr = S.num_post; *bytes = S.num_post ? 8 : 0; break;
        case 3: *dptr = S.act; *bytes = S.act_len; break;
        case 4: *dptr = S.c2; *bytes = S.c2_len; break;
        default: return w4_fail(W4A16_ERR_ARG, "moe_scratch: which=%d outside 0..4", which);
    }
    if (!*dptr) return w4_fail(W4A16_ERR_NOT_FOUND, "moe_scratch: no MoE call has run on this context");
    if (block) *block = S.block;
    return 0;
}

extern "C" int w4a16_set_moe_shape(w4a16_ctx* ctx, int block, int waves) {
    if (!ctx) return w4_fail(W4A16_ERR_ARG, "set_moe_shape: null context");
    if ((block != 0 && block != 1 && block != 4 && block != 16 && block != 32 && block != 48 && block != 64) || waves < 0 ||
        waves > 8)
        return w4_fail(W4A16_ERR_ARG, "set_moe_shape: block in {0,1,4,16,32,48,64}, waves in 0..8");
    ctx->moe_block = block;
    ctx->moe_waves = waves;
    return 0;
}

extern "C" int w4a16_set_moe_tiled(w4a16_ctx* ctx, int mode) {
    if (!ctx) return w4_fail(W4A16_ERR_ARG, "set_moe_tiled: null context");
    if (mode < -1 || mode > 1) return w4_fail(W4A16_ERR_ARG, "set_moe_tiled: -1 = never, 0 = automatic, 1 = always");
    ctx->moe_tiled = mode;
    return 0;
}

extern "C" int w4a16_bench_moe(w4a16_ctx* ctx, const char* const* names, size_t n_names, uint64_t x_dev,
                               uint64_t idx_dev, uint64_t wt_dev, size_t t, size_t top_k, uint64_t y_dev, size_t warmup,
                               size_t reps, float* ms_events, double* ms_wall) {
    if (!ctx || !names || n_names == 0 || reps == 0) return w4_fail(W4A16_ERR_ARG, "bench_moe: null argument");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    W4_TRY(w4_hip(hipEventCreate(&e0), "hipEventCreate"));
    int rc = w4_hip(hipEventCreate(&e1), "hipEventCreate");
    for (size_t i = 0; i < warmup && !rc; i++)
        rc = w4a16_moe_ffn(ctx, names[i % n_names], x_dev, idx_dev, wt_dev, t, top_k, y_dev);
    if (!rc) rc = w4_hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    auto w0 = std::chrono::steady_clock::now();
    if (!rc) rc = w4_hip(hipEventRecord(e0, ctx->stream), "hipEventRecord");
    for (size_t i = 0; i < reps && !rc; i++)
        rc = w4a16_moe_ffn(ctx, names[(warmup + i) % n_names], x_dev, idx_dev, wt_dev, t, top_k, y_dev);
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
