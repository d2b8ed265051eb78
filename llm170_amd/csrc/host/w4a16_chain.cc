// Layer chain of libw4a16hip.so: device-generated synthetic linears, the elementwise glue, and the decoder-layer
// sequence of linears.  Stands in for chain_device_body (w4a16_dec/chains.rs:195-304), norm_resid_dev / ew_dev_fused
// (the glue launches around it) and decode_bench (w4a16_dec/probe.rs:1123-1289).
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstring>

#include "w4a16_internal.h"

static inline unsigned ceil_div(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

extern "C" int w4a16_upload_lin_synth(w4a16_ctx* ctx, const char* name, size_t n, size_t k, size_t group,
                                      uint64_t seed_q, uint64_t seed_s, float lo, float hi) {
    if (!ctx || !name) return w4_fail(W4A16_ERR_ARG, "upload_lin_synth: null argument");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    if (group != 128 && group != 32)
        return w4_fail(W4A16_ERR_UNSUPPORTED, "gptq4: unsupported combination group=%zu scale_bf16=0", group);
    if (n == 0 || k == 0 || k % group != 0 || n > 0x7fffffffu || k > 0x7fffffffu)
        return w4_fail(W4A16_ERR_SHAPE, "upload_lin_synth %s: n%zu k%zu g%zu contract", name, n, k, group);
    if (!(lo > 0.0f) || !(hi >= lo) || !std::isfinite(hi) || hi > 65504.0f)
        return w4_fail(W4A16_ERR_ARG, "upload_lin_synth %s: scale range [%g, %g) must be positive and finite in f16", name,
                       (double)lo, (double)hi);
    W4Lin L;
    L.n = n;
    L.k = k;
    L.group = group;
    L.scale_bf16 = 0;
    L.scales_regular = true;
    unsigned long long words = (unsigned long long)n * (k / 8), scales = (unsigned long long)n * (k / group);
    int rc = w4a16_alloc(ctx, words * 4, &L.q_raw);
    if (!rc) rc = w4a16_alloc(ctx, scales * 2, &L.s_raw);
    if (!rc) {
        unsigned long long sq = seed_q, ss = seed_s;
        float span = hi - lo;
        void* pq[] = {&L.q_raw, &words, &sq};
        rc = w4_launch(ctx, "w4a16_synth_q", std::min<unsigned>(ceil_div(words, 256), 65536), 1, 256, 0, pq);
        void* ps[] = {&L.s_raw, &scales, &ss, &lo, &span};
        if (!rc) rc = w4_launch(ctx, "w4a16_synth_s", std::min<unsigned>(ceil_div(scales, 256), 65536), 1, 256, 0, ps);
    }
    if (rc) {
        const std::string keep = w4_err_save();
        (void)w4a16_free(ctx, L.q_raw);
        (void)w4a16_free(ctx, L.s_raw);
        w4_err_restore(keep);
        return rc;
    }
    return w4_register_lin(ctx, name, L);
}

extern "C" int w4a16_rms_rescale_f16(w4a16_ctx* ctx, uint64_t v_f32_dev, size_t ld, size_t ncols, size_t t,
                                     uint64_t out_f16_dev) {
    if (!ctx || !v_f32_dev || !out_f16_dev) return w4_fail(W4A16_ERR_ARG, "rms_rescale: null argument");
    if (t == 0 || ncols == 0 || ncols > ld || ld > 0x7fffffffu || t > 0x7fffffffu)
        return w4_fail(W4A16_ERR_SHAPE, "rms_rescale: t=%zu ncols=%zu ld=%zu", t, ncols, ld);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    int ldi = (int)ld, nc = (int)ncols;
    void* p[] = {&v_f32_dev, &ldi, &nc, &out_f16_dev};
    return w4_launch(ctx, "w4a16_rms_rescale_f16", (unsigned)t, 1, kW4RmsLanes, 0, p);
}

extern "C" int w4a16_norm_resid(w4a16_ctx* ctx, uint64_t x_dev, uint64_t nw_dev, uint64_t ab_dev, uint64_t xn_dev,
                                uint64_t xn32_dev, uint64_t xn16_dev, size_t t, size_t w_off, size_t hidden) {
    if (!ctx || !x_dev || !nw_dev || !ab_dev || !xn_dev) return w4_fail(W4A16_ERR_ARG, "norm_resid: null argument");
    if (t == 0 || hidden == 0 || hidden > 8192 || t > 0x7fffffffu || w_off > 0x7fffffffu - hidden)
        return w4_fail(W4A16_ERR_SHAPE, "norm_resid: t=%zu hidden=%zu (1..8192) w_off=%zu", t, hidden, w_off);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    int wo = (int)w_off, hd = (int)hidden;
    void* p[] = {&x_dev, &nw_dev, &ab_dev, &xn_dev, &xn32_dev, &xn16_dev, &wo, &hd};
    return w4_launch(ctx, "w4a16_norm_resid", (unsigned)t, 1, 1024, 0, p);
}

extern "C" int w4a16_silu_mul_f16(w4a16_ctx* ctx, uint64_t gu_f32_dev, size_t n_ff, size_t t, uint64_t out_f16_dev) {
    return w4a16_act_mul_f16(ctx, gu_f32_dev, n_ff, t, out_f16_dev, W4A16_ACT_SILU);
}

extern "C" int w4a16_act_mul_f16(w4a16_ctx* ctx, uint64_t gu_f32_dev, size_t n_ff, size_t t, uint64_t out_f16_dev, int act) {
    if (!ctx || !gu_f32_dev || !out_f16_dev) return w4_fail(W4A16_ERR_ARG, "silu_mul: null argument");
    if (act != W4A16_ACT_SILU && act != W4A16_ACT_GELU_TANH)
        return w4_fail(W4A16_ERR_ARG, "act_mul: activation %d (0 = silu, 1 = gelu, tanh form)", act);
    if (t == 0 || n_ff == 0 || n_ff > 0x3fffffffu || t > 0x7fffffffu)
        return w4_fail(W4A16_ERR_SHAPE, "silu_mul: t=%zu n_ff=%zu", t, n_ff);
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    int nf = (int)n_ff, ti = (int)t;
    void* p[] = {&gu_f32_dev, &nf, &ti, &out_f16_dev, &act};
    return w4_launch(ctx, "w4a16_silu_mul_f16", std::min<unsigned>(ceil_div(t * n_ff / (n_ff % 4 == 0 ? 4 : 1), 256), 4096), 1, 256, 0, p);
}

extern "C" int w4a16_chain_forward(w4a16_ctx* ctx, const char* prefix, size_t layer0, size_t n_layers, uint64_t x_dev,
                                   size_t t, uint64_t y_dev) {
    if (!ctx || !prefix || !x_dev || !y_dev) return w4_fail(W4A16_ERR_ARG, "chain_forward: null argument");
    if (n_layers == 0 || t == 0) return w4_fail(W4A16_ERR_SHAPE, "chain_forward: n_layers=%zu t=%zu", n_layers, t);
    W4ChainScratch& S = ctx->chain;
    uint64_t cur = x_dev;
    for (size_t l = layer0; l < layer0 + n_layers; l++) {
        char nm[4][160];
        const char* role[4] = {"attn_qkv", "attn_output", "ffn_gate_up", "ffn_down"};
        W4Lin* L[4];
        for (int i = 0; i < 4; i++) {
            snprintf(nm[i], sizeof nm[i], "%s.%zu.%s", prefix, l, role[i]);
            W4_TRY(w4_find_lin(ctx, nm[i], &L[i]));
        }
        const size_t hidden = L[0]->k, n_ff = L[3]->k;
        if (L[0]->n < hidden || L[1]->k != hidden || L[1]->n != hidden || L[2]->k != hidden || L[2]->n != 2 * n_ff ||
            L[3]->n != hidden)
            return w4_fail(W4A16_ERR_SHAPE, "chain_forward %s.%zu: linears do not chain (hidden %zu, n_ff %zu)", prefix, l,
                           hidden, n_ff);
        const size_t widest = std::max(std::max(L[0]->n, L[2]->n), hidden);
        W4_TRY(w4_ensure(ctx, &S.y32, &S.y32_cap, t * widest * 4));
        W4_TRY(w4_ensure(ctx, &S.h16a, &S.h16a_cap, t * hidden * 2));
        W4_TRY(w4_ensure(ctx, &S.h16b, &S.h16b_cap, t * n_ff * 2));
        const bool last = l + 1 == layer0 + n_layers;
        uint64_t out = y_dev;
        if (!last) {
            const int pp = (int)(l & 1);
            W4_TRY(w4_ensure(ctx, &S.ping[pp], &S.ping_cap[pp], t * hidden * 2));
            out = S.ping[pp];
        }
        W4_TRY(w4a16_lin_forward(ctx, nm[0], cur, S.y32, t, 0, W4A16_PATH_AUTO));
        W4_TRY(w4a16_rms_rescale_f16(ctx, S.y32, L[0]->n, hidden, t, S.h16a));
        W4_TRY(w4a16_lin_forward(ctx, nm[1], S.h16a, S.y32, t, 0, W4A16_PATH_AUTO));
        W4_TRY(w4a16_rms_rescale_f16(ctx, S.y32, hidden, hidden, t, S.h16a));
        if (L[2]->q_tiled && L[2]->n % 32 == 0) {
            // SiLU*up is the epilogue of the gate|up kernel in every regime (decode, streaming, MFMA tiles): same bits
            // as the linear followed by the element-wise launch, without the [t][2 n_ff] f32 round trip
            W4_TRY(w4a16_lin_forward_glu(ctx, nm[2], S.h16a, S.h16b, t));
        } else {
            W4_TRY(w4a16_lin_forward(ctx, nm[2], S.h16a, S.y32, t, 0, W4A16_PATH_AUTO));
            W4_TRY(w4a16_silu_mul_f16(ctx, S.y32, n_ff, t, S.h16b));
        }
        W4_TRY(w4a16_lin_forward(ctx, nm[3], S.h16b, S.y32, t, 0, W4A16_PATH_AUTO));
        W4_TRY(w4a16_rms_rescale_f16(ctx, S.y32, hidden, hidden, t, out));
        cur = out;
    }
    return 0;
}

// Smallest e >= 0 with bound * 2^-e <= 32768 (half the f16 range), for a bound on the magnitude of what is handed over.
static int handover_exp(double bound) {
    int e = 0;
    while (e < 120 && std::ldexp(bound, -e) > 32768.0) e++;
    return e;
}

// The same chain with the three normalisations inside a layer deferred across the linears that follow them
// (w4a16_lin_forward_deferred_norm_scaled): four launches per layer instead of seven.  The activations cross from launch
// to launch as f16 WITHOUT their 1/rms factor, so each hand-over carries a power-of-two factor that keeps it inside
// the f16 range whatever the input: a linear fed rows of unit root mean square over k columns gives no element above
// (largest row norm of W) x sqrt(k) (Cauchy-Schwarz; w4a16_lin_row_norm_max), the gated product none above the square
// of that, and the down projection none above its own row-norm bound times sqrt(n_ff) times the bound of its input.
// The producer multiplies by 2^-e before rounding to f16 and the consumer by 2^e after its MFMA sums, both exact, so the
// values are those of the un-scaled statement wherever that one stays in range.
extern "C" int w4a16_chain_forward_fused(w4a16_ctx* ctx, const char* prefix, size_t layer0, size_t n_layers,
                                         uint64_t x_dev, size_t t, uint64_t y_dev) {
    if (!ctx || !prefix || !x_dev || !y_dev) return w4_fail(W4A16_ERR_ARG, "chain_forward_fused: null argument");
    if (n_layers == 0 || t == 0) return w4_fail(W4A16_ERR_SHAPE, "chain_forward_fused: n_layers=%zu t=%zu", n_layers, t);
    W4ChainScratch& S = ctx->chain;
    uint64_t cur = x_dev;
    size_t n_prev = 0;  // partial sums the previous layer's down projection left in S.stats[2]
    int e_prev = 0;     // and the exponent of its hand-over
    for (size_t l = layer0; l < layer0 + n_layers; l++) {
        char nm[4][160];
        const char* role[4] = {"attn_qkv", "attn_output", "ffn_gate_up", "ffn_down"};
        W4Lin* L[4];
        for (int i = 0; i < 4; i++) {
            snprintf(nm[i], sizeof nm[i], "%s.%zu.%s", prefix, l, role[i]);
            W4_TRY(w4_find_lin(ctx, nm[i], &L[i]));
        }
        const size_t hidden = L[0]->k, n_ff = L[3]->k, n_qkv = L[0]->n;
        if (n_qkv < hidden || n_qkv % 8 != 0 || L[1]->k != hidden || L[1]->n != hidden || L[2]->k != hidden ||
            L[2]->n != 2 * n_ff || L[3]->n != hidden)
            return w4_fail(W4A16_ERR_SHAPE, "chain_forward_fused %s.%zu: linears do not chain (hidden %zu, n_ff %zu)", prefix,
                           l, hidden, n_ff);
        W4_TRY(w4_ensure(ctx, &S.y32, &S.y32_cap, t * hidden * 4));
        W4_TRY(w4_ensure(ctx, &S.a16, &S.a16_cap, t * n_qkv * 2));
        W4_TRY(w4_ensure(ctx, &S.h16a, &S.h16a_cap, t * hidden * 2));
        W4_TRY(w4_ensure(ctx, &S.h16b, &S.h16b_cap, t * n_ff * 2));
        W4_TRY(w4_ensure(ctx, &S.ping[0], &S.ping_cap[0], t * hidden * 2));
        for (int i = 0; i < 3; i++)
            // decode regime: one entry of 16 floats per 16 output rows at most; beyond it one entry of t (rounded up to
            // 4) floats per 64 output columns at most
            W4_TRY(w4_ensure(ctx, &S.stats[i], &S.stats_cap[i],
                             t <= 16 ? ((std::max(n_qkv, hidden) + 15) / 16) * 64
                                     : ((std::max(n_qkv, hidden) + 63) / 64) * ((t + 3) / 4 * 4) * 4));
        const bool last = l + 1 == layer0 + n_layers;
        size_t n_a = 0, n_b = 0, n_d = 0;
        float rn[4];
        for (int i = 0; i < 4; i++) W4_TRY(w4a16_lin_row_norm_max(ctx, nm[i], &rn[i]));
        const double b_qkv = (double)rn[0] * std::sqrt((double)hidden), b_o = (double)rn[1] * std::sqrt((double)hidden),
                     b_gu = (double)rn[2] * std::sqrt((double)hidden), b_act = b_gu * b_gu,
                     b_down = (double)rn[3] * std::sqrt((double)n_ff) * b_act;
        const int e_a = handover_exp(b_qkv), e_b = handover_exp(b_o), e_c = handover_exp(b_act), e_d = handover_exp(b_down);
        // a = qkv(x)[:, :hidden], its statistics over those columns only.  The chain's own input is taken as given
        // (e_prev = 0); the previous layer's down projection handed over 2^-e_prev times its output
        W4_TRY(w4a16_lin_forward_deferred_norm_scaled(ctx, nm[0], cur, 0, t, n_prev ? S.stats[2] : 0, n_prev, hidden, e_prev,
                                                      S.a16, 1, e_a, S.stats[0], hidden, &n_a, 0, 0));
        W4_TRY(w4a16_lin_forward_deferred_norm_scaled(ctx, nm[1], S.a16, n_qkv, t, S.stats[0], n_a, hidden, e_a, S.h16a, 1,
                                                      e_b, S.stats[1], hidden, &n_b, 0, 0));
        W4_TRY(w4a16_lin_forward_glu_deferred_norm_scaled(ctx, nm[2], S.h16a, 0, t, S.stats[1], n_b, hidden, e_b, S.h16b, e_c,
                                                          W4A16_ACT_SILU));
        if (last) {
            // the chain's output is normalised: one launch per call, not per layer
            W4_TRY(w4a16_lin_forward_deferred_norm_scaled(ctx, nm[3], S.h16b, 0, t, 0, 0, 0, e_c, S.y32, 0, 0, 0, 0, nullptr, 0, 0));
            W4_TRY(w4a16_rms_rescale_f16(ctx, S.y32, hidden, hidden, t, y_dev));
        } else {
            W4_TRY(w4a16_lin_forward_deferred_norm_scaled(ctx, nm[3], S.h16b, 0, t, 0, 0, 0, e_c, S.ping[0], 1, e_d, S.stats[2],
                                                          hidden, &n_d, 0, 0));
            cur = S.ping[0];
            n_prev = n_d;
            e_prev = e_d;
        }
    }
    return 0;
}

extern "C" int w4a16_chain_graph_create(w4a16_ctx* ctx, const char* prefix, size_t layer0, size_t n_layers, uint64_t x_dev,
                                        size_t t, uint64_t y_dev, int fused, w4a16_graph** out) {
    if (!ctx || !prefix || !out) return w4_fail(W4A16_ERR_ARG, "chain_graph_create: null argument");
    *out = nullptr;
    auto pass = [&]() {
        return fused ? w4a16_chain_forward_fused(ctx, prefix, layer0, n_layers, x_dev, t, y_dev)
                     : w4a16_chain_forward(ctx, prefix, layer0, n_layers, x_dev, t, y_dev);
    };
    W4_TRY(pass());  // sizes the scratch (a capture cannot allocate) and checks the arguments
    W4_TRY(w4a16_capture_begin(ctx));
    const int frc = pass();
    const std::string keep = w4_err_save();
    w4a16_graph* g = nullptr;
    const int erc = w4a16_capture_end(ctx, &g);
    if (frc) {  // the failing step's message, not the one of ending the capture
        if (g) w4a16_graph_destroy(ctx, g);
        w4_err_restore(keep);
        return frc;
    }
    W4_TRY(erc);
    *out = g;
    return 0;
}

extern "C" int w4a16_bench_chain(w4a16_ctx* ctx, const char* prefix, size_t n_layers, uint64_t x_dev, size_t t,
                                 uint64_t y_dev, size_t warmup, size_t reps, int use_graph, int fused, float* ms_events,
                                 double* ms_wall) {
    if (!ctx || !prefix || reps == 0) return w4_fail(W4A16_ERR_ARG, "bench_chain: null argument");
    W4_TRY(w4_hip(hipSetDevice(ctx->device), "hipSetDevice"));
    auto pass = [&]() {
        return fused ? w4a16_chain_forward_fused(ctx, prefix, 0, n_layers, x_dev, t, y_dev)
                     : w4a16_chain_forward(ctx, prefix, 0, n_layers, x_dev, t, y_dev);
    };
    for (size_t i = 0; i < std::max<size_t>(warmup, 1); i++) W4_TRY(pass());
    W4_TRY(w4_hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"));
    w4a16_graph* graph = nullptr;
    int rc = 0;
    if (use_graph) {
        rc = w4a16_chain_graph_create(ctx, prefix, 0, n_layers, x_dev, t, y_dev, fused, &graph);
        if (!rc) rc = w4a16_graph_launch(ctx, graph);  // one untimed replay
        if (!rc) rc = w4_hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (!rc) rc = w4_hip(hipEventCreate(&e0), "hipEventCreate");
    if (!rc) rc = w4_hip(hipEventCreate(&e1), "hipEventCreate");
    auto w0 = std::chrono::steady_clock::now();
    if (!rc) rc = w4_hip(hipEventRecord(e0, ctx->stream), "hipEventRecord");
    for (size_t i = 0; i < reps && !rc; i++) rc = use_graph ? w4a16_graph_launch(ctx, graph) : pass();
    if (!rc) rc = w4_hip(hipEventRecord(e1, ctx->stream), "hipEventRecord");
    if (!rc) rc = w4_hip(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    auto w1 = std::chrono::steady_clock::now();
    float ms = 0.f;
    if (!rc) rc = w4_hip(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
    if (ms_events) *ms_events = ms;
    if (ms_wall) *ms_wall = std::chrono::duration<double, std::milli>(w1 - w0).count();
    const std::string keep = w4_err_save();
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (graph) w4a16_graph_destroy(ctx, graph);
    if (rc) w4_err_restore(keep);
    return rc;
}
