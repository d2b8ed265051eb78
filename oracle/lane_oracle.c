/*
 * lane_oracle.c — CPU restatement of the reference's W4A16 numeric contract.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against and the thing timed as the CPU baseline.  Nothing in the
 * product library may link, load or call it; the product path has no CPU
 * fallback.
 *
 * Every function cites the reference lines it follows (paths relative to the
 * reference checkout).  Build: gcc -O2 -ffp-contract=off -fno-fast-math —
 * the reference accumulates with a separate f32 multiply and f32 add, so no
 * FMA contraction may be introduced by the compiler.
 *
 * Pinning status (what checks each function independently of this text):
 *   orc_half_to_f32 ....... exhaustive 65536 patterns vs numpy float16, KATs lane.rs:140-145
 *   orc_f32_to_f16 ........ round trip over all non-NaN halves + 13 edge KATs (probes/w4a16/gpu.rs:953-982)
 *   orc_bf16_to_f32 ....... closed form bits<<16
 *   orc_dequant_row_split . KAT rows matmul/cpu.rs:227-271, packer order scripts/gen_tiny_w4a16.py:44-48
 *   orc_lane_parts ........ numpy float32 emulation (separately rounded mul/add), exact-rational brute force,
 *                           closed forms (nibble 8 => 0; scale 1, x 1 => integer sum), lane.rs:98-193 test inputs
 *   orc_tree64 ............ math.fsum on exactly-summable inputs + a pairing-order vector that distinguishes orders
 *   orc_moe_topk .......... KATs qwen35/stages/moe.rs:135-155
 *   orc_exact_dot ......... exact-rational brute force (quant/exact.rs:77-135 precedent)
 *   orc_exact_dot_sample .. the row function above, call for call; plain f64 dot of the dequantised row
 *   orc_moe_act_silu_f16 .. float64 evaluation of g/(1+exp(-g))*u within one f16 step; special cases g = 0, u = 0,
 *                           large |g| (silu -> g, -> 0)
 *   orc_moe_act_gelu_f16 .. float64 evaluation of 0.5 g (1 + tanh(0.7978846 (g + 0.044715 g^3))) u within one f16 step;
 *                           against the erf form of gelu to 1e-3; g = 0, large |g| (-> g, -> 0); swapped operands fail
 *   orc_moe_topk_sum_f16 .. numpy float32 sequential sum; exactly-summable inputs
 *   orc_moe_align ......... numpy stable argsort by expert + padding arithmetic; tiny hand-worked case
 *   orc_rms_rescale_f16 ... float64 v / sqrt(mean(v^2) + 1e-6) within one f16 step, >= 99.9 % identical; constant rows;
 *                           invariance of the output under scaling the row by a power of two
 *   orc_silu_mul_f16_rows . float64 evaluation within one f16 step; layout (gate | up) by a crafted row
 *   orc_gelu_mul_f16_rows . float64 evaluation of the tanh form within one f16 step; swapped operands fail
 *   orc_norm_resid ........ numpy float32 restatement whose fused multiply-add is built from exact f64 products and a
 *                           round-to-odd sum (independent of libm's fmaf); float64 v/sqrt(mean v^2 + 1e-6)*w to a few f32
 *                           ulp; x + ab exact; an un-fused sum of squares and a sequential (non-tree) sum are shown to
 *                           give different bits; f16 copies against numpy float16
 * No function here is "parity unpinned".
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- crates/core/src/quant/deq.rs:4-27 (half_to_f32); same routine as gptq4.rs:5-27 (h2f) ---- */
float orc_half_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h >> 15) & 1u;
    uint32_t exp = (uint32_t)(h >> 10) & 0x1fu;
    uint32_t frac = (uint32_t)h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (frac == 0) {
            bits = sign << 31;
        } else {
            uint32_t e = 127 - 15 + 1;
            uint32_t f = frac;
            while ((f & 0x400u) == 0) {
                f <<= 1;
                e -= 1;
            }
            f &= 0x3ffu;
            bits = (sign << 31) | (e << 23) | (f << 13);
        }
    } else if (exp == 0x1f) {
        bits = (sign << 31) | (0xffu << 23) | (frac << 13);
    } else {
        bits = (sign << 31) | ((exp + 112u) << 23) | (frac << 13);
    }
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

/* Bit pattern of the result (a float return value passing through a foreign-function layer that widens to double
 * would quiet signalling NaNs; the payload rule of deq.rs:23 is checked on the raw bits). */
uint32_t orc_half_to_f32_bits(uint16_t h) {
    float f = orc_half_to_f32(h);
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

/* ---- crates/core/src/quant/deq.rs:29-31 ---- */
float orc_bf16_to_f32(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

/* ---- crates/backend-gpu/src/rawcuda/w4a16_dec/mod.rs:187-219 (f32_to_f16, round to nearest even) ---- */
uint16_t orc_f32_to_f16(float v) {
    uint32_t b;
    memcpy(&b, &v, 4);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
    int32_t exp = (int32_t)((b >> 23) & 0xFFu);
    uint32_t man = b & 0x7FFFFFu;
    if (exp == 0xFF) {
        return (uint16_t)(sign | 0x7C00u | (man != 0 ? 0x200u : 0u));
    }
    int32_t e = exp - 127 + 15;
    if (e >= 31) {
        return (uint16_t)(sign | 0x7C00u);
    }
    if (e <= 0) {
        if (e < -10) {
            return sign;
        }
        uint32_t m = man | 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half = 1u << (shift - 1);
        uint32_t sub = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        if (rem > half || (rem == half && (sub & 1u) == 1u)) {
            sub += 1;
        }
        return (uint16_t)(sign | (uint16_t)sub);
    }
    uint32_t h = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u) == 1u)) {
        h += 1;
    }
    return (uint16_t)(sign | (uint16_t)h);
}

/* ---- crates/core/src/quant/lane.rs:2-13 (tree64) ---- */
double orc_tree64(const double v[64]) {
    double a[64];
    memcpy(a, v, sizeof a);
    for (int i = 0; i < 32; i++) a[i] += a[i + 32];
    static const int offs[5] = {16, 8, 4, 2, 1};
    for (int o = 0; o < 5; o++) {
        int off = offs[o];
        for (int i = 0; i < off; i++) a[i] += a[i + off];
    }
    return a[0];
}

/* ---- crates/core/src/quant/lane.rs:42-70 (lane_parts_scale) ----
 * zrow: zero point per group (8 for the symmetric format, gates.rs:113); srow_f32: scale per group already
 * widened to f32 (f16 via half_to_f32 as in lane.rs:15-18,29, or bf16 via bf16_to_f32 as in gates.rs:98-107).
 * Returns -1 when the shape contract asserted at lane.rs:50-55 does not hold (the caller passes the lengths). */
int orc_lane_parts(const uint32_t* qrow, size_t qlen, const uint32_t* zrow, size_t zlen, const float* srow_f32,
                   const uint16_t* x, size_t k, size_t group, double lane[64]) {
    if (!(group >= 32 && group % 32 == 0 && k % group == 0)) return -1;
    if (qlen != k / 8 || zlen != k / group) return -1;
    for (size_t l = 0; l < 64; l++) {
        float acc = 0.0f;
        for (size_t i = l; i < k; i += 64) {
            size_t g = i / group;
            int32_t q = (int32_t)((qrow[i >> 3] >> (4 * (i & 7))) & 0xFu);
            float w = (float)(q - (int32_t)zrow[g]) * srow_f32[g];
            float p = w * orc_half_to_f32(x[i]);
            acc = acc + p;
        }
        lane[l] = (double)acc;
    }
    return 0;
}

/* ---- crates/core/src/quant/lane.rs:32-40 (dot_row_w4a16_lane_group) ---- */
int orc_dot_row_lane_group(const uint32_t* qrow, size_t qlen, const uint32_t* zrow, size_t zlen,
                           const float* srow_f32, const uint16_t* x, size_t k, size_t group, float* out) {
    double lane[64];
    if (orc_lane_parts(qrow, qlen, zrow, zlen, srow_f32, x, k, group, lane) != 0) return -1;
    *out = (float)orc_tree64(lane);
    return 0;
}

/* ---- crates/core/src/quant/lane.rs:20-30 (dot_row_w4a16_lane: g128, f16 scales) ---- */
int orc_dot_row_lane(const uint32_t* qrow, size_t qlen, const uint32_t* zrow, size_t zlen, const uint16_t* srow,
                     size_t slen, const uint16_t* x, size_t k, float* out) {
    if (k % 128 != 0 || qlen != k / 8 || slen != k / 128) return -1;
    float sf[k / 128 ? k / 128 : 1];
    for (size_t g = 0; g < k / 128; g++) sf[g] = orc_half_to_f32(srow[g]);
    return orc_dot_row_lane_group(qrow, qlen, zrow, zlen, sf, x, k, 128, out);
}

/* ---- crates/core/src/matmul/cpu.rs:167-194 (dequant_row_w4a16_split), byte-addressed operands ---- */
void orc_dequant_row_split(const uint8_t* q, const uint8_t* s, size_t row, size_t k, size_t group, int scale_bf16,
                           float* out) {
    size_t nb = k / group;
    const uint8_t* qrow = q + row * (k / 2);
    const uint8_t* srow = s + row * (k * 2 / group);
    for (size_t b = 0; b < nb; b++) {
        uint16_t bits = (uint16_t)(srow[2 * b] | ((uint16_t)srow[2 * b + 1] << 8));
        float sc = scale_bf16 ? orc_bf16_to_f32(bits) : orc_half_to_f32(bits);
        for (size_t i = 0; i < group; i++) {
            size_t woff = 4 * (b * (group / 8) + i / 8);
            uint32_t w = (uint32_t)qrow[woff] | ((uint32_t)qrow[woff + 1] << 8) | ((uint32_t)qrow[woff + 2] << 16) |
                         ((uint32_t)qrow[woff + 3] << 24);
            int32_t nib = (int32_t)((w >> (4 * (i % 8))) & 0xFu);
            out[b * group + i] = (float)(nib - 8) * sc;
        }
    }
}

/* ---- crates/core/src/quant/exact.rs:4-53 (Neumaier-compensated f64 dot over f32 activations) ---- */
double orc_exact_dot(const uint8_t* qrow, const uint8_t* srow, const float* x, size_t k, size_t group,
                     int scale_bf16) {
    double sum = 0.0, c = 0.0;
    size_t nb = k / group;
    for (size_t b = 0; b < nb; b++) {
        uint16_t bits = (uint16_t)(srow[2 * b] | ((uint16_t)srow[2 * b + 1] << 8));
        double sc = (double)(scale_bf16 ? orc_bf16_to_f32(bits) : orc_half_to_f32(bits));
        for (size_t i = 0; i < group; i++) {
            size_t woff = 4 * (b * (group / 8) + i / 8);
            uint32_t w = (uint32_t)qrow[woff] | ((uint32_t)qrow[woff + 1] << 8) | ((uint32_t)qrow[woff + 2] << 16) |
                         ((uint32_t)qrow[woff + 3] << 24);
            int32_t nib = (int32_t)((w >> (4 * (i % 8))) & 0xFu);
            double v = (double)(nib - 8) * sc * (double)x[b * group + i];
            double t = sum + v;
            if (fabs(sum) >= fabs(v)) {
                c += (sum - t) + v;
            } else {
                c += (v - t) + sum;
            }
            sum = t;
        }
    }
    return sum + c;
}

/* ---- whole GEMM the way the parity gate builds its expectation (probes/w4a16/gates.rs:113-132):
 * out[ti*n + o] = dot_row_w4a16_lane_group(q row o, z = 8, scales widened to f32, x row ti).
 * Rows [n0, n1) only, so callers can sample or partition. ---- */
typedef struct {
    const uint32_t* q;
    const uint16_t* s;
    const uint16_t* x;
    float* out;
    size_t t, n, k, group;
    int scale_bf16;
    size_t n0, n1;
    int rc;
} orc_gemm_job;

static void* orc_gemm_rows(void* arg) {
    orc_gemm_job* j = (orc_gemm_job*)arg;
    size_t ng = j->k / j->group;
    uint32_t* z8 = (uint32_t*)malloc(ng * sizeof(uint32_t));
    float* sf = (float*)malloc(ng * sizeof(float));
    for (size_t g = 0; g < ng; g++) z8[g] = 8;
    j->rc = 0;
    for (size_t o = j->n0; o < j->n1; o++) {
        const uint32_t* qrow = j->q + o * (j->k / 8);
        const uint16_t* srow = j->s + o * ng;
        for (size_t g = 0; g < ng; g++)
            sf[g] = j->scale_bf16 ? orc_bf16_to_f32(srow[g]) : orc_half_to_f32(srow[g]);
        for (size_t ti = 0; ti < j->t; ti++) {
            float v;
            if (orc_dot_row_lane_group(qrow, j->k / 8, z8, ng, sf, j->x + ti * j->k, j->k, j->group, &v) != 0) {
                j->rc = -1;
                v = NAN;
            }
            j->out[ti * j->n + o] = v;
        }
    }
    free(z8);
    free(sf);
    return NULL;
}

/* Row chunks over `threads` workers — the reference's CPU engine partitions output rows the same way over
 * min(cores, 32) pool threads (crates/core/src/matmul/cpu.rs:2-10, 21-23). threads <= 1 runs inline. */
int orc_gemm_lane(const uint16_t* x, size_t t, const uint32_t* q, const uint16_t* s, size_t n, size_t k,
                  size_t group, int scale_bf16, float* out, int threads) {
    if ((group != 128 && group != 32) || k % group != 0 || t == 0) return -1;
    if (threads < 1) threads = 1;
    if ((size_t)threads > n) threads = (int)(n ? n : 1);
    orc_gemm_job* jobs = (orc_gemm_job*)calloc((size_t)threads, sizeof(orc_gemm_job));
    pthread_t* th = (pthread_t*)calloc((size_t)threads, sizeof(pthread_t));
    size_t per = (n + (size_t)threads - 1) / (size_t)threads;
    int rc = 0;
    for (int i = 0; i < threads; i++) {
        size_t a = (size_t)i * per, b = a + per;
        if (a > n) a = n;
        if (b > n) b = n;
        jobs[i] = (orc_gemm_job){q, s, x, out, t, n, k, group, scale_bf16, a, b, 0};
        if (threads == 1) {
            orc_gemm_rows(&jobs[i]);
        } else {
            pthread_create(&th[i], NULL, orc_gemm_rows, &jobs[i]);
        }
    }
    for (int i = 0; i < threads; i++) {
        if (threads != 1) pthread_join(th[i], NULL);
        if (jobs[i].rc != 0) rc = -1;
    }
    free(jobs);
    free(th);
    return rc;
}

/* Sampled outputs: out[j] = dot(row rows[j], x row toks[j]).  Used where the full shape is ~1e12 scalar MACs. */
int orc_gemm_lane_sample(const uint16_t* x, const uint32_t* q, const uint16_t* s, size_t k, size_t group,
                         int scale_bf16, const uint32_t* rows, const uint32_t* toks, size_t count, float* out) {
    if ((group != 128 && group != 32) || k % group != 0) return -1;
    size_t ng = k / group;
    uint32_t* z8 = (uint32_t*)malloc(ng * sizeof(uint32_t));
    float* sf = (float*)malloc(ng * sizeof(float));
    for (size_t g = 0; g < ng; g++) z8[g] = 8;
    int rc = 0;
    for (size_t j = 0; j < count; j++) {
        const uint16_t* srow = s + (size_t)rows[j] * ng;
        for (size_t g = 0; g < ng; g++) sf[g] = scale_bf16 ? orc_bf16_to_f32(srow[g]) : orc_half_to_f32(srow[g]);
        if (orc_dot_row_lane_group(q + (size_t)rows[j] * (k / 8), k / 8, z8, ng, sf, x + (size_t)toks[j] * k, k,
                                   group, &out[j]) != 0)
            rc = -1;
    }
    free(z8);
    free(sf);
    return rc;
}

/* Sampled outputs of the compensated f64 dot (orc_exact_dot, quant/exact.rs:27-53), activations widened from f16
 * exactly: out[j] = exact(row rows[j], x row toks[j]).  The yardstick that tells summation-order noise of the f32
 * lane sum from a kernel's own error. */
int orc_exact_dot_sample(const uint16_t* x, const uint32_t* q, const uint16_t* s, size_t k, size_t group,
                         int scale_bf16, const uint32_t* rows, const uint32_t* toks, size_t count, double* out) {
    if ((group != 128 && group != 32) || k % group != 0) return -1;
    size_t ng = k / group;
    float* xf = (float*)malloc(k * sizeof(float));
    for (size_t j = 0; j < count; j++) {
        const uint16_t* xr = x + (size_t)toks[j] * k;
        for (size_t i = 0; i < k; i++) xf[i] = orc_half_to_f32(xr[i]);
        out[j] = orc_exact_dot((const uint8_t*)(q + (size_t)rows[j] * (k / 8)), (const uint8_t*)(s + (size_t)rows[j] * ng),
                               xf, k, group, scale_bf16);
    }
    free(xf);
    return 0;
}

/* ---- crates/backend-gpu/src/rawcuda/w4a16_dec/mod.rs:168-185 (moe_topk) ≡ qwen35/stages/moe.rs:8-31:
 * softmax over all experts in f32, k largest probabilities, ties to the lower index, weights renormalised by
 * the selected sum (summed in selection order). ---- */
void orc_moe_topk(const float* logits, size_t n, size_t k, uint32_t* idx_out, float* w_out) {
    float mx = -INFINITY;
    for (size_t i = 0; i < n; i++) mx = fmaxf(mx, logits[i]);
    float* p = (float*)malloc(n * sizeof(float));
    uint8_t* used = (uint8_t*)calloc(n, 1);
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++) {
        p[i] = expf(logits[i] - mx);
        sum = sum + p[i];
    }
    for (size_t i = 0; i < n; i++) p[i] = p[i] / sum;
    if (k > n) k = n;
    for (size_t j = 0; j < k; j++) {
        size_t best = n;
        for (size_t i = 0; i < n; i++) {
            if (used[i]) continue;
            if (best == n || p[i] > p[best]) best = i; /* strict > keeps the lower index on ties */
        }
        used[best] = 1;
        idx_out[j] = (uint32_t)best;
    }
    float wsum = 0.0f;
    for (size_t j = 0; j < k; j++) wsum = wsum + p[idx_out[j]];
    for (size_t j = 0; j < k; j++) w_out[j] = p[idx_out[j]] / wsum;
    free(p);
    free(used);
}

/* ---- elementwise glue between the two expert GEMMs: silu(g)*u computed in f32, rounded to f16
 * (crates/backend-gpu/src/rawcuda/assets/moe.cu:1649-1660; CPU engine order qwen35/stages/moe.rs:79-83) ---- */
uint16_t orc_silu_mul_f16(float g, float u) {
    float sg = g / (1.0f + expf(-g));
    return orc_f32_to_f16(sg * u);
}

/* ---- w4a16_moe_act_silu_f16 (crates/backend-gpu/src/rawcuda/assets/moe.cu:1649-1660): c13 is f16 [ns][2*n_ff],
 * gate in columns 0..n_ff, up in n_ff..2*n_ff; act[r][c] = f16(silu(gate) * up) with f32 arithmetic. ---- */
void orc_moe_act_silu_f16(const uint16_t* c13, size_t ns, size_t n_ff, uint16_t* act) {
    for (size_t r = 0; r < ns; r++)
        for (size_t c = 0; c < n_ff; c++) {
            const float g = orc_half_to_f32(c13[r * 2 * n_ff + c]);
            const float u = orc_half_to_f32(c13[r * 2 * n_ff + n_ff + c]);
            act[r * n_ff + c] = orc_silu_mul_f16(g, u);
        }
}

/* ---- w4a16_moe_act_gelu_f16 (crates/backend-gpu/src/rawcuda/assets/moe.cu:1635-1647): the tanh form of gelu on the
 * gate, times up, f32 arithmetic in the reference's order, one rounding to f16. ---- */
uint16_t orc_gelu_mul_f16(float g, float u) {
    const float x3 = g * g * g;
    const float a = (0.5f * g * (1.0f + tanhf(0.7978846f * (g + 0.044715f * x3)))) * u;
    return orc_f32_to_f16(a);
}

void orc_moe_act_gelu_f16(const uint16_t* c13, size_t ns, size_t n_ff, uint16_t* act) {
    for (size_t r = 0; r < ns; r++)
        for (size_t c = 0; c < n_ff; c++) {
            const float g = orc_half_to_f32(c13[r * 2 * n_ff + c]);
            const float u = orc_half_to_f32(c13[r * 2 * n_ff + n_ff + c]);
            act[r * n_ff + c] = orc_gelu_mul_f16(g, u);
        }
}

/* ---- w4a16_moe_topk_sum_f16 (assets/moe.cu:1662-1674): out[r][c] = sum over the token's top_k slots of
 * f16 c2[(r*top_k + kk)][c], added in slot order in f32. ---- */
void orc_moe_topk_sum_f16(const uint16_t* c2, size_t t, size_t h, size_t top_k, float* out) {
    for (size_t r = 0; r < t; r++)
        for (size_t c = 0; c < h; c++) {
            float acc = 0.0f;
            for (size_t kk = 0; kk < top_k; kk++) acc = acc + orc_half_to_f32(c2[(r * top_k + kk) * h + c]);
            out[r * h + c] = acc;
        }
}

/* ---- w4a16_moe_align2 + w4a16_moe_align_marlin (assets/moe.cu:860-908, 1599-1633): slots sorted by expert,
 * stable in slot order; each expert's run padded to a multiple of `block` with the sentinel ns; expert_ids holds
 * the expert of every block; returns the padded total (num_post). ---- */
size_t orc_moe_align(const int32_t* idx, size_t ns, size_t n_exp, size_t block, int32_t* sorted_ids,
                     int32_t* expert_ids) {
    size_t* cnt = (size_t*)calloc(n_exp, sizeof(size_t));
    size_t* base = (size_t*)calloc(n_exp, sizeof(size_t));
    for (size_t j = 0; j < ns; j++) cnt[idx[j]]++;
    size_t pos = 0;
    for (size_t e = 0; e < n_exp; e++) {
        base[e] = pos;
        const size_t padded = (cnt[e] + block - 1) / block * block;
        for (size_t p = 0; p < padded; p++) sorted_ids[pos + p] = (int32_t)ns;
        for (size_t b = 0; b < padded / block; b++) expert_ids[pos / block + b] = (int32_t)e;
        pos += padded;
    }
    memset(cnt, 0, n_exp * sizeof(size_t));
    for (size_t j = 0; j < ns; j++) {
        const size_t e = (size_t)idx[j];
        sorted_ids[base[e] + cnt[e]++] = (int32_t)j;
    }
    free(cnt);
    free(base);
    return pos;
}

/* Array form of orc_f32_to_f16 (same routine, element by element). */
void orc_f32_to_f16_array(const float* v, size_t n, uint16_t* out) {
    for (size_t i = 0; i < n; i++) out[i] = orc_f32_to_f16(v[i]);
}

/* ---- RMS rescale emitting f16: the normalisation of norm_resid (crates/backend-gpu/src/rawcuda/assets/norm.cu:4-48)
 * without residual and weight.  out[r][c] = f16(v[r*ld + c] * inv), inv = f32(1 / sqrt(ss / ncols + 1e-6)).
 * Order of the sum of squares (the contract the device kernel shares): 1024 partials, partial i adds the exact f64
 * squares of columns i, i+1024, ... in order; partials folded pairwise at strides 512, 256, ..., 1. ---- */
void orc_rms_rescale_f16(const float* v, size_t ld, size_t ncols, size_t t, uint16_t* out) {
    for (size_t r = 0; r < t; r++) {
        const float* row = v + r * ld;
        double red[1024];
        for (size_t i = 0; i < 1024; i++) {
            double ss = 0.0;
            for (size_t c = i; c < ncols; c += 1024) {
                const double d = (double)row[c];
                ss = ss + d * d;
            }
            red[i] = ss;
        }
        for (size_t st = 512; st > 0; st >>= 1)
            for (size_t i = 0; i < st; i++) red[i] = red[i] + red[i + st];
        const float inv = (float)(1.0 / sqrt(red[0] / (double)ncols + 1e-6));
        for (size_t c = 0; c < ncols; c++) out[r * ncols + c] = orc_f32_to_f16(row[c] * inv);
    }
}

/* ---- norm_resid / norm_resid_g (crates/backend-gpu/src/rawcuda/assets/norm.cu:4-48, 97-148), f32 throughout.
 * Thread tid of 1024 adds the squares of its columns tid, tid+1024, ... with one fused multiply-add each: the file is
 * compiled with nvcc's default -fmad=true (scripts/build_cuda_kernels.sh:67 "build norm", unlike the kernels built
 * with -fmad=false), which contracts ss += v*v.  Partials are folded at strides 512..1; divide and square root are
 * IEEE (nvcc defaults -prec-div=true -prec-sqrt=true).  x is updated in place to x + ab.  xn32 / xn16 may be NULL. ---- */
void orc_norm_resid(float* x, const float* nw, const float* ab, float* xn, float* xn32, uint16_t* xn16, size_t t,
                    size_t w_off, size_t hidden) {
    for (size_t r = 0; r < t; r++) {
        float* xr = x + r * hidden;
        const float* ar = ab + r * hidden;
        float red[1024];
        for (size_t tid = 0; tid < 1024; tid++) {
            float ss = 0.0f;
            for (size_t c = tid; c < hidden; c += 1024) {
                const float v = xr[c] + ar[c];
                ss = fmaf(v, v, ss);
            }
            red[tid] = ss;
        }
        for (size_t st = 512; st > 0; st >>= 1)
            for (size_t i = 0; i < st; i++) red[i] = red[i] + red[i + st];
        const float inv = 1.0f / sqrtf(red[0] / (float)hidden + 1e-6f);
        for (size_t c = 0; c < hidden; c++) {
            const float v = xr[c] + ar[c];
            volatile float y0 = v * inv; /* two roundings */
            const float y = y0 * nw[w_off + c];
            xn[r * hidden + c] = y;
            if (xn32 || xn16) {
                const uint16_t h = orc_f32_to_f16(y);
                if (xn32) xn32[r * hidden + c] = orc_half_to_f32(h);
                if (xn16) xn16[r * hidden + c] = h;
            }
            xr[c] = v;
        }
    }
}

/* ---- ew (assets/ew.cu:9-32) on rows gu f32 [t][2*n_ff] = (gate | up): out[r][c] = f16((g / (1 + exp(-g))) * u) in
 * f32 arithmetic. ---- */
void orc_silu_mul_f16_rows(const float* gu, size_t n_ff, size_t t, uint16_t* out) {
    for (size_t r = 0; r < t; r++)
        for (size_t c = 0; c < n_ff; c++)
            out[r * n_ff + c] = orc_silu_mul_f16(gu[r * 2 * n_ff + c], gu[r * 2 * n_ff + n_ff + c]);
}

/* ---- ew_gelu (assets/ew.cu:34-57) on the same rows: the tanh form of gelu on the gate, times up. ---- */
void orc_gelu_mul_f16_rows(const float* gu, size_t n_ff, size_t t, uint16_t* out) {
    for (size_t r = 0; r < t; r++)
        for (size_t c = 0; c < n_ff; c++)
            out[r * n_ff + c] = orc_gelu_mul_f16(gu[r * 2 * n_ff + c], gu[r * 2 * n_ff + n_ff + c]);
}
