/*
 * rmi_qwen3.c — Qwen3Session::generate_inner (src/models/qwen3.rs:581-1158)
 * restated for the end-to-end configuration: all 2-D weights Q8_0, F16 KV
 * cache, NeoX RoPE, q/k RMS norm, greedy sampling, no EOS.  TEST
 * INFRASTRUCTURE ONLY (see rmi_oracle.h).
 *
 * The elementwise ops follow the x86-64, non-parity-trace build:
 *   rms_norm            src/ops/norm.rs:3-19   (f64 sum of f32 squares)
 *   rope_neox           src/ops/rope.rs:21-37  (powf/cosf/sinf of the host libm)
 *   softmax             src/ops/attention.rs:28-38
 *   dot_f16             src/ops/dot.rs:99-119  (f64 sum of f32 products)
 *   silu_mul_inplace    src/ops/activation/mod.rs:137-151
 *   embedding_lookup    src/ops/embedding.rs:12-22
 *   greedy_token        src/models/qwen3.rs:172-191
 * Pins (tests/test_oracle_qwen3.py): rms_norm, rms_norm_inplace and rope_neox by the reference's own bit
 * vectors (src/ops/matmul_tests.rs:127-198); silu_mul_inplace by the scalar-order bit vector of
 * tests/quantized_inference.rs:21-29 and, for operand order, the fixture of src/ops/matmul_tests.rs:361-372;
 * greedy_token by src/models/qwen3.rs:1519-1522; softmax, dot_f16, the attention block and embedding_lookup_q8_0
 * (no reference vector exists for the x86-64 branch) by an independent numpy statement with every rounding
 * point enumerated; the loop's wiring by a second composition of the pinned pieces written from qwen3.rs.
 * expf/cosf/sinf/powf come from this host's libm, as Rust's f32::exp/cos/sin/powf do on the same platform.
 *
 * Built with -mf16c (hardware f16 conversions, as the reference with
 * target-cpu=native, src/ops/float.rs:177-207).
 */
#include "rmi_oracle.h"

#include <immintrin.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

static inline float h2f(uint16_t h) { return _mm_cvtss_f32(_mm_cvtph_ps(_mm_set1_epi16((short)h))); }
static inline uint16_t f2h(float v) { return (uint16_t)_mm_extract_epi16(_mm_cvtps_ph(_mm_set_ss(v), 0), 0); }

static double now_s(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

int rmi_ref_cpu_matmul(const void *weight, const uint8_t *input_q8, const float *input_scales, float *output,
                       uint32_t n_in, uint32_t n_out, uint32_t ith, uint32_t nth) {
    const rmi_ref_cpu_weight *w = (const rmi_ref_cpu_weight *)weight;
    (void)ith;
    (void)nth; /* the pool splits rows itself: one pool.compute per matmul */
    rmi_ref_pool_matmul_q8_0(w->pool, w->blocks, input_q8, input_scales, output, n_in, n_out, 1);
    return 0;
}

static void rms_norm(const float *input, const float *weight, float *output, size_t n, float eps) {
    double sum_sq = 0.0;
    for (size_t i = 0; i < n; i++) {
        float sq = input[i] * input[i];
        sum_sq += (double)sq;
    }
    float mean_sq = (float)(sum_sq / (double)n);
    float scale = 1.0f / sqrtf(mean_sq + eps);
    for (size_t i = 0; i < n; i++) {
        float t = input[i] * scale;
        output[i] = t * weight[i];
    }
}

static void rope_neox(float *x, size_t pos, size_t head_dim, float freq_base) {
    size_t half = head_dim / 2;
    float theta_scale = powf(freq_base, -2.0f / (float)head_dim);
    float theta = (float)pos;
    for (size_t i = 0; i < half; i++) {
        float cos_a = cosf(theta), sin_a = sinf(theta);
        float x0 = x[i], x1 = x[i + half];
        float a = x1 * -sin_a;
        float b = x1 * cos_a;
        x[i] = fmaf(x0, cos_a, a);
        x[i + half] = fmaf(x0, sin_a, b);
        theta *= theta_scale;
    }
}

static void softmax(float *x, size_t n) {
    float max_val = -INFINITY;
    for (size_t i = 0; i < n; i++) max_val = fmaxf(max_val, x[i]);
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++) {
        x[i] = expf(x[i] - max_val);
        sum += x[i];
    }
    if (sum > 0.0f)
        for (size_t i = 0; i < n; i++) x[i] /= sum;
}

static float dot_f16(const uint16_t *a, const uint16_t *b, size_t n) {
    double sum = 0.0;
    for (size_t i = 0; i < n; i++) {
        float p = h2f(a[i]) * h2f(b[i]);
        sum += (double)p;
    }
    return (float)sum;
}

/* src/ops/activation/mod.rs:137-151 (the scalar loop; x86-64 has no vector variant) */
static void silu_mul_inplace(const float *gate, float *up, size_t n) {
    for (size_t i = 0; i < n; i++) {
        float g = gate[i];
        float s = g / (1.0f + expf(-g));
        up[i] *= s;
    }
}

/* src/ops/embedding.rs:12-22 */
static void embedding_lookup_q8_0(const uint8_t *weight, uint32_t token_id, size_t n_embd, float *out) {
    size_t bpr = n_embd / 32;
    const uint8_t *row = weight + (size_t)token_id * bpr * 34;
    for (size_t b = 0; b < bpr; b++) {
        uint16_t dh;
        memcpy(&dh, row + b * 34, 2);
        float d = h2f(dh);
        for (int jx = 0; jx < 32; jx++) out[b * 32 + jx] = d * (float)(int8_t)row[b * 34 + 2 + jx];
    }
}

/* greedy_token (src/models/qwen3.rs:172-191): the first strict maximum; returns 0 when the logits are empty or
 * one of them is not finite (the reference's Err).  `second` is the largest of the others (not in the
 * reference: the decode tests compare it). */
static int greedy_top2(const float *logits, size_t n, uint32_t *best_id, float *best_out, float *second_out) {
    if (n == 0) return 0;
    uint32_t id = 0;
    float best = logits[0], second = -INFINITY;
    int finite = isfinite(best);
    for (size_t i = 1; i < n && finite; i++) {
        float l = logits[i];
        if (!isfinite(l)) finite = 0;
        if (l > best) {
            second = best;
            best = l;
            id = (uint32_t)i;
        } else if (l > second) {
            second = l;
        }
    }
    *best_id = id;
    *best_out = best;
    *second_out = second;
    return finite;
}

typedef struct {
    const rmi_ref_qwen3_model *m;
    const float *q;
    float *attn_out;
    const uint16_t *k_cache, *v_cache;
    float *scores;       /* [nth][score_stride] */
    size_t score_stride; /* floats per thread; holds weights f16 + values f16 too */
    size_t layer_base, kv_stride, step;
} attn_job;

static void attention_heads(void *argp, int ith, int nth) {
    attn_job *j = (attn_job *)argp;
    const rmi_ref_qwen3_model *m = j->m;
    size_t hk = m->head_dim_k, hv = m->head_dim_v, step = j->step;
    size_t group = m->n_head / m->n_head_kv;
    float kq_scale = 1.0f / sqrtf((float)hk);
    size_t head_start = (size_t)ith * m->n_head / (size_t)nth, head_end = ((size_t)ith + 1) * m->n_head / (size_t)nth;
    size_t n_padded = (step + 1 + 255) / 256 * 256;
    float *scores = j->scores + (size_t)ith * j->score_stride;
    /* two f16 scratch rows behind the scores: softmax weights and gathered values */
    uint16_t *weights16 = (uint16_t *)(scores + n_padded);
    uint16_t *values16 = weights16 + n_padded;
    uint16_t query[1024];
    for (size_t head = head_start; head < head_end; head++) {
        size_t kv_head = head / group;
        for (size_t d = 0; d < hk; d++) query[d] = f2h(j->q[head * hk + d]);
        for (size_t t = 0; t < n_padded; t++) scores[t] = -INFINITY;
        for (size_t t = 0; t <= step; t++) {
            const uint16_t *key = j->k_cache + j->layer_base + t * j->kv_stride + kv_head * hk;
            scores[t] = dot_f16(query, key, hk) * kq_scale;
        }
        softmax(scores, n_padded);
        for (size_t t = 0; t < n_padded; t++) weights16[t] = f2h(scores[t]);
        for (size_t t = step + 1; t < n_padded; t++) values16[t] = 0;
        float *out = j->attn_out + head * hv;
        for (size_t d = 0; d < hv; d++) {
            for (size_t t = 0; t <= step; t++)
                values16[t] = j->v_cache[j->layer_base + t * j->kv_stride + kv_head * hv + d];
            out[d] = dot_f16(values16, weights16, n_padded);
        }
    }
}

/* ---- the elementwise pieces, exported for per-kernel parity tests ---- */
void rmi_ref_rms_norm(const float *input, const float *weight, float *output, size_t n, float eps) {
    rms_norm(input, weight, output, n, eps);
}
void rmi_ref_rope_neox(float *x, size_t pos, size_t head_dim, float freq_base) { rope_neox(x, pos, head_dim, freq_base); }
void rmi_ref_rope_angles(size_t pos, size_t head_dim, float freq_base, float *cos_out, float *sin_out) {
    float theta_scale = powf(freq_base, -2.0f / (float)head_dim), theta = (float)pos;
    for (size_t i = 0; i < head_dim / 2; i++) {
        cos_out[i] = cosf(theta);
        sin_out[i] = sinf(theta);
        theta *= theta_scale;
    }
}
void rmi_ref_softmax(float *x, size_t n) { softmax(x, n); }
float rmi_ref_dot_f16(const uint16_t *a, const uint16_t *b, size_t n) { return dot_f16(a, b, n); }
void rmi_ref_embedding_lookup_q8_0(const uint8_t *weight, uint32_t token_id, size_t n_embd, float *out) {
    embedding_lookup_q8_0(weight, token_id, n_embd, out);
}
int rmi_ref_greedy_token(const float *logits, size_t n, uint32_t *token_id) {
    float best, second;
    return greedy_top2(logits, n, token_id, &best, &second) ? 0 : -1;
}
/* silu_mul_inplace(&gate_out, &mut up_out): up_out[i] *= gate_out[i] / (1 + exp(-gate_out[i])) */
void rmi_ref_silu_mul(const float *gate_out, float *up_out, size_t n) { silu_mul_inplace(gate_out, up_out, n); }
/* attention of one token over keys 0..step of an F16 cache laid out [t][kv_stride] (qwen3.rs:876-933) */
void rmi_ref_attention_f16(const float *q, const uint16_t *k_cache, const uint16_t *v_cache, size_t step,
                           size_t kv_stride, size_t n_head, size_t n_head_kv, size_t hk, size_t hv, float *attn_out) {
    rmi_ref_qwen3_model m;
    memset(&m, 0, sizeof m);
    m.n_head = (uint32_t)n_head;
    m.n_head_kv = (uint32_t)n_head_kv;
    m.head_dim_k = (uint32_t)hk;
    m.head_dim_v = (uint32_t)hv;
    size_t n_padded = (step + 1 + 255) / 256 * 256, score_stride = n_padded * 2 + 64;
    float *scores = (float *)calloc(score_stride, 4);
    attn_job job = {&m, q, attn_out, k_cache, v_cache, scores, score_stride, 0, kv_stride, step};
    attention_heads(&job, 0, 1);
    free(scores);
}

static uint64_t fnv1a(const void *data, size_t n) {
    const uint8_t *p = (const uint8_t *)data;
    uint64_t h = 1469598103934665603ull;
    for (size_t i = 0; i < n; i++) {
        h ^= p[i];
        h *= 1099511628211ull;
    }
    return h;
}

int rmi_ref_qwen3_generate(const rmi_ref_qwen3_model *m, rmi_ref_matmul_fn matmul, rmi_ref_pool *pool,
                           const uint32_t *prompt, uint32_t n_prompt, uint32_t max_new, uint32_t *generated,
                           uint64_t *step_hash, uint32_t *step_argmax, float *step_top2,
                           const uint32_t *dump_steps, uint32_t n_dump, float *dump_logits,
                           double *seconds_total, double *seconds_matmul) {
    if (n_prompt == 0 || (size_t)n_prompt + max_new > m->n_ctx || m->head_dim_k > 1024) return -1;
    size_t capacity = (size_t)n_prompt + max_new;
    size_t n_embd = m->n_embd, n_ff = m->n_ff, hk = m->head_dim_k, hv = m->head_dim_v;
    size_t n_embd_q = m->n_head * hk, n_embd_k = m->n_head_kv * hk, n_embd_v = m->n_head_kv * hv, n_attn = m->n_head * hv;
    size_t kv_stride = n_embd_k > n_embd_v ? n_embd_k : n_embd_v;
    size_t max_n_in = n_embd_q;
    if (n_attn > max_n_in) max_n_in = n_attn;
    if (n_ff > max_n_in) max_n_in = n_ff;
    if (n_embd > max_n_in) max_n_in = n_embd;
    int nth = rmi_ref_pool_threads(pool);
    size_t n_padded_max = (capacity + 255) / 256 * 256;
    size_t score_stride = n_padded_max * 2 + 64; /* f32 scores + two f16 rows */

    uint16_t *k_cache = (uint16_t *)calloc(m->n_layer * capacity * kv_stride, 2);
    uint16_t *v_cache = (uint16_t *)calloc(m->n_layer * capacity * kv_stride, 2);
    float *x = (float *)calloc(n_embd, 4), *normed = (float *)calloc(n_embd, 4);
    float *q = (float *)calloc(n_embd_q, 4), *k = (float *)calloc(n_embd_k, 4), *v = (float *)calloc(n_embd_v, 4);
    float *attn_out = (float *)calloc(n_attn, 4), *attn_proj = (float *)calloc(n_embd, 4);
    float *down = (float *)calloc(n_embd, 4), *gate_buf = (float *)calloc(n_ff, 4), *up_buf = (float *)calloc(n_ff, 4);
    uint8_t *q8 = (uint8_t *)calloc(max_n_in, 1);
    float *sc = (float *)calloc(max_n_in / 32 + 1, 4);
    float *logits = (float *)calloc(m->vocab, 4);
    float *scores = (float *)calloc((size_t)nth * score_stride, 4);
    int rc = 0;
    uint32_t n_generated = 0;
    double t_mm = 0.0, t_start = now_s();
    size_t steps = capacity - 1;
    int qv = m->quant_variant;

#define MATMUL(w, out, nin, nout)                                        \
    do {                                                                 \
        double _t = now_s();                                             \
        if (matmul((w), q8, sc, (out), (uint32_t)(nin), (uint32_t)(nout), 0, 1) != 0) { \
            rc = -1;                                                     \
            goto done;                                                   \
        }                                                                \
        t_mm += now_s() - _t;                                            \
    } while (0)

    for (size_t step = 0; step < steps; step++) {
        size_t position = step; /* text prompt: positions 0..n-1, then last+1+i */
        uint32_t token = step < n_prompt ? prompt[step] : generated[n_generated - 1];
        embedding_lookup_q8_0(m->token_embd, token, n_embd, x);
        for (size_t layer = 0; layer < m->n_layer; layer++) {
            rms_norm(x, m->attn_norm[layer], normed, n_embd, m->eps);
            rmi_ref_quantize_q8_0(normed, n_embd, q8, sc, qv);
            MATMUL(m->wq[layer], q, n_embd, n_embd_q);
            MATMUL(m->wk[layer], k, n_embd, n_embd_k);
            MATMUL(m->wv[layer], v, n_embd, n_embd_v);
            if (m->has_qk_norm) {
                for (size_t h = 0; h < m->n_head; h++) rms_norm(q + h * hk, m->q_norm[layer], q + h * hk, hk, m->eps);
                for (size_t h = 0; h < m->n_head_kv; h++) rms_norm(k + h * hk, m->k_norm[layer], k + h * hk, hk, m->eps);
            }
            for (size_t h = 0; h < m->n_head; h++) rope_neox(q + h * hk, position, hk, m->freq_base);
            for (size_t h = 0; h < m->n_head_kv; h++) rope_neox(k + h * hk, position, hk, m->freq_base);
            size_t layer_base = layer * capacity * kv_stride;
            size_t cache_row = layer_base + step * kv_stride;
            for (size_t i = 0; i < n_embd_k; i++) k_cache[cache_row + i] = f2h(k[i]);
            for (size_t i = 0; i < n_embd_v; i++) v_cache[cache_row + i] = f2h(v[i]);

            attn_job job = {m, q, attn_out, k_cache, v_cache, scores, score_stride, layer_base, kv_stride, step};
            rmi_ref_pool_run(pool, attention_heads, &job);

            rmi_ref_quantize_q8_0(attn_out, n_attn, q8, sc, qv);
            MATMUL(m->wo[layer], attn_proj, n_attn, n_embd);
            for (size_t i = 0; i < n_embd; i++) x[i] += attn_proj[i];
            rms_norm(x, m->ffn_norm[layer], normed, n_embd, m->eps);
            rmi_ref_quantize_q8_0(normed, n_embd, q8, sc, qv);
            /* w_gate's output lands in up_buf and w_up's in gate_buf (qwen3.rs:996-1015) */
            MATMUL(m->w_gate[layer], up_buf, n_embd, n_ff);
            MATMUL(m->w_up[layer], gate_buf, n_embd, n_ff);
            silu_mul_inplace(up_buf, gate_buf, n_ff); /* silu_mul_inplace(&up_buf, &mut gate_buf) */
            rmi_ref_quantize_q8_0(gate_buf, n_ff, q8, sc, qv);
            MATMUL(m->w_down[layer], down, n_ff, n_embd);
            for (size_t i = 0; i < n_embd; i++) x[i] += down[i];
        }
        rms_norm(x, m->output_norm, normed, n_embd, m->eps);
        rmi_ref_quantize_q8_0(normed, n_embd, q8, sc, qv);
        MATMUL(m->output, logits, n_embd, m->vocab);

        uint32_t best_id = 0;
        float best = 0.0f, second = 0.0f;
        int finite = greedy_top2(logits, m->vocab, &best_id, &best, &second);
        if (step_hash) step_hash[step] = fnv1a(logits, (size_t)m->vocab * 4);
        if (step_argmax) step_argmax[step] = best_id;
        if (step_top2) {
            step_top2[2 * step] = best;
            step_top2[2 * step + 1] = second;
        }
        for (uint32_t d = 0; d < n_dump; d++)
            if (dump_steps[d] == step) memcpy(dump_logits + (size_t)d * m->vocab, logits, (size_t)m->vocab * 4);
        if (step + 1 < n_prompt) continue;
        if (!finite) {
            rc = -1;
            goto done;
        }
        if (n_generated >= max_new) break;
        generated[n_generated++] = best_id;
    }
done:
    if (seconds_total) *seconds_total = now_s() - t_start;
    if (seconds_matmul) *seconds_matmul = t_mm;
    free(k_cache); free(v_cache); free(x); free(normed); free(q); free(k); free(v); free(attn_out); free(attn_proj);
    free(down); free(gate_buf); free(up_buf); free(q8); free(sc); free(logits); free(scores);
    return rc < 0 ? rc : (int)n_generated;
}
