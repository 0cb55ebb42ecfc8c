/*
 * rmi_oracle_avx2.c — the reference's x86-64 production kernels restated with
 * the same intrinsics in the same order, plus a persistent-thread row
 * partition to time them.  TEST INFRASTRUCTURE ONLY (see rmi_oracle.h): this
 * is the CPU baseline timed beside the GPU kernels and the cross-check of the
 * portable order emulation in rmi_oracle.c; no shipped code path calls it.
 *
 * Built with -mavx2 -mfma -mf16c; callers must test rmi_ref_have_avx2() first.
 */
#include "rmi_oracle.h"

#include <immintrin.h>
#include <pthread.h>
#include <stdatomic.h>
#include <stdlib.h>
#include <string.h>

#define Q8_0_BLOCK 34
#define QK_K 256
#define Q4K_BLOCK 144

int rmi_ref_have_avx2(void) {
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma") &&
           __builtin_cpu_supports("f16c");
}

static inline float f16_load(const uint8_t *p) {
    uint16_t h;
    memcpy(&h, p, 2);
    return _mm_cvtss_f32(_mm_cvtph_ps(_mm_set1_epi16((short)h)));
}

/* src/ops/dot.rs:447-456 */
static inline float hsum_ps(__m256 v) {
    __m128 hi = _mm256_extractf128_ps(v, 1);
    __m128 lo = _mm256_castps256_ps128(v);
    __m128 s128 = _mm_add_ps(hi, lo);
    __m128 shuf = _mm_movehdup_ps(s128);
    __m128 s2 = _mm_add_ps(s128, shuf);
    __m128 s3 = _mm_movehl_ps(shuf, s2);
    return _mm_cvtss_f32(_mm_add_ss(s2, s3));
}

/* src/ops/quant/q8_0.rs:176-230 */
void rmi_ref_x86_quantize_q8_0(const float *input, size_t n, uint8_t *q8,
                               float *scales) {
    const __m256 sign_mask = _mm256_set1_ps(-0.0f);
    const __m256 max_i8 = _mm256_set1_ps(127.0f);
    const __m256 min_i8 = _mm256_set1_ps(-128.0f);
    size_t blocks = n / 32;
    for (size_t b = 0; b < blocks; b++) {
        const float *ptr = input + b * 32;
        __m256 v0 = _mm256_loadu_ps(ptr), v1 = _mm256_loadu_ps(ptr + 8);
        __m256 v2 = _mm256_loadu_ps(ptr + 16), v3 = _mm256_loadu_ps(ptr + 24);
        __m256 m01 = _mm256_max_ps(_mm256_andnot_ps(sign_mask, v0), _mm256_andnot_ps(sign_mask, v1));
        __m256 m23 = _mm256_max_ps(_mm256_andnot_ps(sign_mask, v2), _mm256_andnot_ps(sign_mask, v3));
        __m256 m0123 = _mm256_max_ps(m01, m23);
        __m128 m128 = _mm_max_ps(_mm256_extractf128_ps(m0123, 1), _mm256_castps256_ps128(m0123));
        __m128 shuf = _mm_movehdup_ps(m128);
        __m128 m2 = _mm_max_ps(m128, shuf);
        __m128 m3 = _mm_movehl_ps(shuf, m2);
        float amax = _mm_cvtss_f32(_mm_max_ss(m2, m3));
        float d = amax == 0.0f ? 0.0f : amax / 127.0f;
        float id = amax == 0.0f ? 0.0f : 127.0f / amax;
        scales[b] = _mm_cvtss_f32(_mm_cvtph_ps(_mm_cvtps_ph(_mm_set_ss(d), 0)));
        __m256 id_v = _mm256_set1_ps(id);
#define RMI_Q(v) \
    _mm256_cvtps_epi32(_mm256_min_ps(_mm256_max_ps(_mm256_round_ps(_mm256_mul_ps(v, id_v), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC), min_i8), max_i8))
        __m256i i0 = RMI_Q(v0), i1 = RMI_Q(v1), i2 = RMI_Q(v2), i3 = RMI_Q(v3);
#undef RMI_Q
        __m256i packed = _mm256_packs_epi16(_mm256_packs_epi32(i0, i1), _mm256_packs_epi32(i2, i3));
        __m256i fixed = _mm256_permutevar8x32_epi32(packed, _mm256_setr_epi32(0, 4, 1, 5, 2, 6, 3, 7));
        _mm256_storeu_si256((__m256i *)(q8 + b * 32), fixed);
    }
}

/* src/ops/kernel/q8_0/avx2.rs:53-174 — 4-row tiles, then single-row tail */
void rmi_ref_x86_matmul_q8_0_range(const uint8_t *weight,
                                   const uint8_t *input_q8,
                                   const float *input_scales, float *output,
                                   size_t n_in, size_t row_start,
                                   size_t row_end) {
    size_t blocks = n_in / 32, stride = blocks * Q8_0_BLOCK;
    const __m256i ones = _mm256_set1_epi16(1);
    size_t n_rows = row_end - row_start, full4 = n_rows / 4;
    for (size_t tile = 0; tile < full4; tile++) {
        const uint8_t *r[4];
        for (int t = 0; t < 4; t++) r[t] = weight + (row_start + tile * 4 + t) * stride;
        __m256 cv[4] = {_mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps()};
        for (size_t b = 0; b < blocks; b++) {
            __m256i qy = _mm256_loadu_si256((const __m256i *)(input_q8 + b * 32));
            float bd = input_scales[b];
            uint16_t dbits[4];
            for (int t = 0; t < 4; t++) memcpy(&dbits[t], r[t] + b * Q8_0_BLOCK, 2);
            __m128 da = _mm_mul_ps(
                _mm_cvtph_ps(_mm_set_epi16(0, 0, 0, 0, (short)dbits[3], (short)dbits[2], (short)dbits[1], (short)dbits[0])),
                _mm_set1_ps(bd));
            __m256 s[4];
            s[0] = _mm256_broadcastss_ps(da);
            s[1] = _mm256_broadcastss_ps(_mm_shuffle_ps(da, da, 0x55));
            s[2] = _mm256_broadcastss_ps(_mm_shuffle_ps(da, da, 0xAA));
            s[3] = _mm256_broadcastss_ps(_mm_shuffle_ps(da, da, 0xFF));
            for (int t = 0; t < 4; t++) {
                __m256i av = _mm256_loadu_si256((const __m256i *)(r[t] + b * Q8_0_BLOCK + 2));
                __m256i ax = _mm256_sign_epi8(av, av);
                __m256i sy = _mm256_sign_epi8(qy, av);
                cv[t] = _mm256_fmadd_ps(
                    s[t], _mm256_cvtepi32_ps(_mm256_madd_epi16(ones, _mm256_maddubs_epi16(ax, sy))), cv[t]);
            }
        }
        for (int t = 0; t < 4; t++) output[tile * 4 + t] = hsum_ps(cv[t]);
    }
    for (size_t j = row_start + full4 * 4; j < row_end; j++) {
        const uint8_t *row = weight + j * stride;
        __m256 acc = _mm256_setzero_ps();
        for (size_t b = 0; b < blocks; b++) {
            float d = f16_load(row + b * Q8_0_BLOCK) * input_scales[b];
            __m256i qx = _mm256_loadu_si256((const __m256i *)(row + b * Q8_0_BLOCK + 2));
            __m256i qy = _mm256_loadu_si256((const __m256i *)(input_q8 + b * 32));
            __m256i ax = _mm256_sign_epi8(qx, qx);
            __m256i sy = _mm256_sign_epi8(qy, qx);
            acc = _mm256_fmadd_ps(_mm256_set1_ps(d),
                                  _mm256_cvtepi32_ps(_mm256_madd_epi16(ones, _mm256_maddubs_epi16(ax, sy))), acc);
        }
        output[j - row_start] = hsum_ps(acc);
    }
}

/* src/ops/quant/mod.rs:140-200 */
void rmi_ref_x86_quantize_row_q8_k(const float *x, size_t n, float *d,
                                   int8_t *qs, int16_t *bsums) {
    size_t nb = n / QK_K;
    for (size_t i = 0; i < nb; i++) {
        const float *block = x + i * QK_K;
        int8_t *q = qs + i * QK_K;
        float amax = 0.0f, max_val = 0.0f;
        for (int j = 0; j < QK_K; j++) {
            float ax = block[j] < 0 ? -block[j] : block[j];
            if (ax > amax) {
                amax = ax;
                max_val = block[j];
            }
        }
        if (amax == 0.0f) {
            d[i] = 0.0f;
            memset(q, 0, QK_K);
            memset(bsums + i * 16, 0, 32);
            continue;
        }
        float iscale = -127.0f / max_val;
        __m256 iscale_vec = _mm256_set1_ps(iscale);
        __m256i ni8 = _mm256_set1_epi32(-127), pi8 = _mm256_set1_epi32(127);
        for (int j = 0; j < QK_K; j += 8) {
            __m256 scaled = _mm256_mul_ps(_mm256_loadu_ps(block + j), iscale_vec);
            __m256i i32s = _mm256_cvtps_epi32(_mm256_round_ps(scaled, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
            __m256i clamped = _mm256_min_epi32(_mm256_max_epi32(i32s, ni8), pi8);
            int32_t arr[8];
            _mm256_storeu_si256((__m256i *)arr, clamped);
            for (int k = 0; k < 8; k++) q[j + k] = (int8_t)arr[k];
        }
        for (int g = 0; g < 16; g++) {
            int32_t sum = 0;
            for (int k = 0; k < 16; k++) sum += q[g * 16 + k];
            bsums[i * 16 + g] = (int16_t)sum;
        }
        d[i] = 1.0f / iscale;
    }
}

/* src/ops/quant/mod.rs:701-799 */
float rmi_ref_x86_vec_dot_q4k_q8k(const uint8_t *q4k, size_t nb, const float *d8,
                                  const int8_t *qs, const int16_t *bsums) {
    const uint32_t kmask1 = 0x3f3f3f3fu, kmask2 = 0x0f0f0f0fu, kmask3 = 0x03030303u;
    const __m256i m4 = _mm256_set1_epi8(0xF);
    __m256 acc = _mm256_setzero_ps();
    __m128 acc_m = _mm_setzero_ps();
    for (size_t i = 0; i < nb; i++) {
        const uint8_t *blk = q4k + i * Q4K_BLOCK;
        float d = f16_load(blk) * d8[i];
        float dmin = -f16_load(blk + 2) * d8[i];
        uint32_t utmp[4];
        memcpy(utmp, blk + 4, 12);
        utmp[3] = ((utmp[2] >> 4) & kmask2) | (((utmp[1] >> 6) & kmask3) << 4);
        uint32_t uaux = utmp[1] & kmask1;
        utmp[1] = (utmp[2] & kmask2) | (((utmp[0] >> 6) & kmask3) << 4);
        utmp[2] = uaux;
        utmp[0] &= kmask1;
        __m256i mins_and_scales =
            _mm256_cvtepu8_epi16(_mm_set_epi32((int)utmp[3], (int)utmp[2], (int)utmp[1], (int)utmp[0]));
        __m256i q8sums = _mm256_loadu_si256((const __m256i *)(bsums + i * 16));
        __m128i q8s = _mm_hadd_epi16(_mm256_extracti128_si256(q8sums, 0), _mm256_extracti128_si256(q8sums, 1));
        __m128i prod = _mm_madd_epi16(_mm256_extracti128_si256(mins_and_scales, 1), q8s);
        acc_m = _mm_fmadd_ps(_mm_set1_ps(dmin), _mm_cvtepi32_ps(prod), acc_m);
        __m128i sc128 = _mm256_extracti128_si256(mins_and_scales, 0);
        __m256i scales256 = _mm256_set_m128i(sc128, sc128);
        __m256i sumi = _mm256_setzero_si256();
        const uint8_t *q4 = blk + 16;
        const int8_t *q8 = qs + i * QK_K;
        for (int j = 0; j < 4; j++) {
            __m256i shuf_l = _mm256_set1_epi16((short)(((4 * j + 1) << 8) | (4 * j)));
            __m256i shuf_h = _mm256_set1_epi16((short)(((4 * j + 3) << 8) | (4 * j + 2)));
            __m256i scale_l = _mm256_shuffle_epi8(scales256, shuf_l);
            __m256i scale_h = _mm256_shuffle_epi8(scales256, shuf_h);
            __m256i q4bits = _mm256_loadu_si256((const __m256i *)q4);
            q4 += 32;
            __m256i q4l = _mm256_and_si256(q4bits, m4);
            __m256i q4h = _mm256_and_si256(_mm256_srli_epi16(q4bits, 4), m4);
            __m256i q8l = _mm256_loadu_si256((const __m256i *)q8);
            q8 += 32;
            __m256i p16l = _mm256_madd_epi16(scale_l, _mm256_maddubs_epi16(q4l, q8l));
            __m256i q8h = _mm256_loadu_si256((const __m256i *)q8);
            q8 += 32;
            __m256i p16h = _mm256_madd_epi16(scale_h, _mm256_maddubs_epi16(q4h, q8h));
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(p16l, p16h));
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    acc_m = _mm_add_ps(acc_m, _mm_movehl_ps(acc_m, acc_m));
    acc_m = _mm_add_ss(acc_m, _mm_movehdup_ps(acc_m));
    return hsum_ps(acc) + _mm_cvtss_f32(acc_m);
}

/* ------------------------------------------------- persistent thread pool */

enum { JOB_NONE = 0, JOB_Q8_0 = 1, JOB_Q4K = 2, JOB_EXIT = 3, JOB_FN = 4 };

struct rmi_ref_pool {
    int n_threads;
    pthread_t *threads;
    atomic_int epoch;   /* bumped by the caller to publish a job        */
    atomic_int done;    /* workers that finished the current epoch      */
    int job;
    const uint8_t *weight;
    const uint8_t *x_q8;
    const float *x_scales;
    const float *d8;
    const int8_t *qs;
    const int16_t *bsums;
    float *output;
    size_t n_in, n_out, n_tokens;
    void (*fn)(void *, int, int);
    void *fn_arg;
};

typedef struct {
    rmi_ref_pool *pool;
    int ith;
} worker_arg;

static void run_slice(rmi_ref_pool *p, int ith) {
    if (p->job == JOB_FN) {
        p->fn(p->fn_arg, ith, p->n_threads);
        return;
    }
    size_t nth = (size_t)p->n_threads;
    size_t per = (p->n_out + nth - 1) / nth;
    size_t start = (size_t)ith * per;
    size_t end = start + per < p->n_out ? start + per : p->n_out;
    if (start >= end) return;
    if (p->job == JOB_Q8_0) {
        size_t nb = p->n_in / 32;
        for (size_t t = 0; t < p->n_tokens; t++)
            rmi_ref_x86_matmul_q8_0_range(p->weight, p->x_q8 + t * p->n_in, p->x_scales + t * nb,
                                          p->output + t * p->n_out + start, p->n_in, start, end);
    } else if (p->job == JOB_Q4K) {
        size_t nb = p->n_in / QK_K;
        for (size_t r = start; r < end; r++)
            p->output[r] = rmi_ref_x86_vec_dot_q4k_q8k(p->weight + r * nb * Q4K_BLOCK, nb, p->d8, p->qs, p->bsums);
    }
}

static void *worker_main(void *argp) {
    worker_arg *arg = (worker_arg *)argp;
    rmi_ref_pool *p = arg->pool;
    int ith = arg->ith;
    free(arg);
    int seen = 0;
    for (;;) {
        int e;
        while ((e = atomic_load_explicit(&p->epoch, memory_order_acquire)) == seen) _mm_pause();
        seen = e;
        if (p->job == JOB_EXIT) break;
        run_slice(p, ith);
        atomic_fetch_add_explicit(&p->done, 1, memory_order_release);
    }
    return NULL;
}

rmi_ref_pool *rmi_ref_pool_create(int n_threads) {
    if (n_threads < 1) n_threads = 1;
    rmi_ref_pool *p = (rmi_ref_pool *)calloc(1, sizeof(*p));
    p->n_threads = n_threads;
    atomic_init(&p->epoch, 0);
    atomic_init(&p->done, 0);
    p->threads = (pthread_t *)calloc((size_t)n_threads, sizeof(pthread_t));
    for (int i = 1; i < n_threads; i++) {
        worker_arg *arg = (worker_arg *)malloc(sizeof(*arg));
        arg->pool = p;
        arg->ith = i;
        pthread_create(&p->threads[i], NULL, worker_main, arg);
    }
    return p;
}

static void pool_run(rmi_ref_pool *p) {
    atomic_store_explicit(&p->done, 0, memory_order_relaxed);
    atomic_fetch_add_explicit(&p->epoch, 1, memory_order_release);
    run_slice(p, 0);
    while (atomic_load_explicit(&p->done, memory_order_acquire) != p->n_threads - 1) _mm_pause();
}

void rmi_ref_pool_destroy(rmi_ref_pool *p) {
    if (!p) return;
    p->job = JOB_EXIT;
    atomic_fetch_add_explicit(&p->epoch, 1, memory_order_release);
    for (int i = 1; i < p->n_threads; i++) pthread_join(p->threads[i], NULL);
    free(p->threads);
    free(p);
}

int rmi_ref_pool_threads(const rmi_ref_pool *p) { return p->n_threads; }

void rmi_ref_pool_matmul_q8_0(rmi_ref_pool *p, const uint8_t *weight,
                              const uint8_t *input_q8,
                              const float *input_scales, float *output,
                              size_t n_in, size_t n_out, size_t n_tokens) {
    p->job = JOB_Q8_0;
    p->weight = weight;
    p->x_q8 = input_q8;
    p->x_scales = input_scales;
    p->output = output;
    p->n_in = n_in;
    p->n_out = n_out;
    p->n_tokens = n_tokens;
    pool_run(p);
}

void rmi_ref_pool_matmul_q4k_q8k(rmi_ref_pool *p, const uint8_t *weight,
                                 const float *d, const int8_t *qs,
                                 const int16_t *bsums, float *output,
                                 size_t n_in, size_t n_out) {
    p->job = JOB_Q4K;
    p->weight = weight;
    p->d8 = d;
    p->qs = qs;
    p->bsums = bsums;
    p->output = output;
    p->n_in = n_in;
    p->n_out = n_out;
    p->n_tokens = 1;
    pool_run(p);
}

void rmi_ref_pool_run(rmi_ref_pool *p, void (*fn)(void *arg, int ith, int nth), void *arg) {
    p->job = JOB_FN;
    p->fn = fn;
    p->fn_arg = arg;
    pool_run(p);
}
