/*
 * rmi_q6_k.c — the reference's Q6_K paths restated.  TEST INFRASTRUCTURE ONLY
 * (see rmi_oracle.h).
 *
 * Q6_K super-block, 210 bytes, 256 elements (src/ops/quant/mod.rs:10, 530-569):
 *   [0..128)   ql: low 4 bits      [128..192) qh: high 2 bits
 *   [192..208) 16 int8 scales (one per 16 elements)      [208..210) f16 d
 * element 128j + 32t + l (j<2, t<4, l<32):
 *   low  = t<2 ? ql[64j + 32t + l] & 15 : ql[64j + 32(t-2) + l] >> 4
 *   high = (qh[32j + l] >> 2t) & 3,   q = (low | high<<4) - 32
 *   scale index 8j + 2t + l/16
 */
#include "rmi_oracle.h"

#include <immintrin.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define QK_K 256
#define Q6K_BLOCK 210

static inline float load_f16(const uint8_t *p) {
    return rmi_ref_f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
}

/* unsigned 6-bit value (0..63) of element e of a super-block */
static inline int q6k_elem_u(const uint8_t *blk, int e) {
    int j = e >> 7, t = (e >> 5) & 3, l = e & 31;
    uint8_t lo = blk[64 * j + 32 * (t & 1) + l];
    int low = t < 2 ? (lo & 0xF) : (lo >> 4);
    int high = (blk[128 + 32 * j + l] >> (2 * t)) & 3;
    return low | (high << 4);
}

/* src/ops/quant/mod.rs:530-569: d * sc * q, left to right ((d*sc)*q) */
void rmi_ref_dequantize_row_q6_k(const uint8_t *blocks, float *output, size_t n) {
    size_t nb = n / QK_K;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t *blk = blocks + bi * Q6K_BLOCK;
        float d = load_f16(blk + 208);
        float *out = output + bi * QK_K;
        for (int j128 = 0; j128 < 2; j128++) {
            for (int l = 0; l < 32; l++) {
                int ql_idx = j128 * 64 + l, qh_idx = j128 * 32 + l;
                int q1 = ((blk[ql_idx] & 0xF) | ((blk[128 + qh_idx] & 3) << 4)) - 32;
                int q2 = ((blk[ql_idx + 32] & 0xF) | (((blk[128 + qh_idx] >> 2) & 3) << 4)) - 32;
                int q3 = ((blk[ql_idx] >> 4) | (((blk[128 + qh_idx] >> 4) & 3) << 4)) - 32;
                int q4 = ((blk[ql_idx + 32] >> 4) | (((blk[128 + qh_idx] >> 6) & 3) << 4)) - 32;
                int is = l / 16;
                const int8_t *sc = (const int8_t *)(blk + 192 + j128 * 8 + is);
                float t;
                t = d * (float)sc[0];
                out[j128 * 128 + l] = t * (float)q1;
                t = d * (float)sc[2];
                out[j128 * 128 + l + 32] = t * (float)q2;
                t = d * (float)sc[4];
                out[j128 * 128 + l + 64] = t * (float)q3;
                t = d * (float)sc[6];
                out[j128 * 128 + l + 96] = t * (float)q4;
            }
        }
    }
}

/* src/ops/quant/mod.rs:640-692 */
static float vec_dot_q6k_q8k_scalar(const uint8_t *w, size_t nb, const float *d8, const int8_t *qs) {
    float sums[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    float sumf = 0.0f;
    for (size_t i = 0; i < nb; i++) {
        const uint8_t *blk = w + i * Q6K_BLOCK;
        int32_t aux32[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int sb = 0; sb < 16; sb++) {
            int32_t scale = (int8_t)blk[192 + sb];
            for (int k = 0; k < 16; k++) {
                int e = 16 * sb + k;
                aux32[k & 7] += scale * (int32_t)qs[i * QK_K + e] * (q6k_elem_u(blk, e) - 32);
            }
        }
        float d = load_f16(blk + 208) * d8[i];
        for (int l = 0; l < 8; l++) {
            float t = d * (float)aux32[l];
            sums[l] = sums[l] + t;
        }
    }
    for (int l = 0; l < 8; l++) sumf = sumf + sums[l];
    return sumf;
}

/* The eight int32 lanes of src/ops/quant/mod.rs:996-1055 for one super-block:
 * lane m sums, over the eight 32-element groups g, scale[2g + (m>=4)] times the
 * products of the unsigned quants 4m..4m+3 of the group, minus
 * 32 * (bsums[2m]*scale[2m] + bsums[2m+1]*scale[2m+1]).  maddubs pairs stay below
 * i16 saturation (2*63*127), madd_epi16 and the adds are exact in i32. */
static void q6k_lanes(const uint8_t *blk, const int8_t *q8, const int16_t *bs, int32_t lanes[8]) {
    const int8_t *sc = (const int8_t *)(blk + 192);
    for (int m = 0; m < 8; m++) {
        int32_t s = 0;
        for (int g = 0; g < 8; g++) {
            int32_t scale = sc[2 * g + (m >= 4)];
            int32_t dot = 0;
            for (int k = 0; k < 4; k++) {
                int e = 32 * g + 4 * m + k;
                dot += (int32_t)q6k_elem_u(blk, e) * (int32_t)q8[e];
            }
            s += scale * dot;
        }
        int32_t off = (int32_t)bs[2 * m] * sc[2 * m] + (int32_t)bs[2 * m + 1] * sc[2 * m + 1];
        lanes[m] = s - (int32_t)((uint32_t)off << 5);
    }
}

static inline float hsum8(const float a[8]) {
    float s0 = a[4] + a[0], s1 = a[5] + a[1], s2 = a[6] + a[2], s3 = a[7] + a[3];
    return (s0 + s1) + (s2 + s3);
}

/* src/ops/quant/mod.rs:964-1062 in plain C */
static float vec_dot_q6k_q8k_avx2_order(const uint8_t *w, size_t nb, const float *d8, const int8_t *qs,
                                        const int16_t *bsums) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (size_t i = 0; i < nb; i++) {
        const uint8_t *blk = w + i * Q6K_BLOCK;
        float d = load_f16(blk + 208) * d8[i];
        int32_t lanes[8];
        q6k_lanes(blk, qs + i * QK_K, bsums + i * 16, lanes);
        for (int m = 0; m < 8; m++) acc[m] = fmaf(d, (float)lanes[m], acc[m]);
    }
    return hsum8(acc);
}

float rmi_ref_vec_dot_q6k_q8k(const uint8_t *row, size_t nb, const float *d, const int8_t *qs, const int16_t *bsums,
                              int variant) {
    if (variant == RMI_REF_AVX2) return vec_dot_q6k_q8k_avx2_order(row, nb, d, qs, bsums);
    return vec_dot_q6k_q8k_scalar(row, nb, d, qs);
}

void rmi_ref_q6k_q8k_block_ints(const uint8_t *row, size_t nb, const int8_t *qs, int32_t *isum) {
    for (size_t i = 0; i < nb; i++) {
        const uint8_t *blk = row + i * Q6K_BLOCK;
        int32_t s = 0;
        for (int e = 0; e < QK_K; e++)
            s += (int32_t)(int8_t)blk[192 + e / 16] * (int32_t)qs[i * QK_K + e] * (q6k_elem_u(blk, e) - 32);
        isum[i] = s;
    }
}

void rmi_ref_q6k_q8k_lane_ints(const uint8_t *row, size_t nb, const int8_t *qs, const int16_t *bsums,
                               int32_t *lanes) {
    for (size_t i = 0; i < nb; i++) q6k_lanes(row + i * Q6K_BLOCK, qs + i * QK_K, bsums + i * 16, lanes + 8 * i);
}

static void row_partition(size_t n_out, size_t ith, size_t nth, size_t *start, size_t *end) {
    if (nth == 0) nth = 1;
    size_t per = (n_out + nth - 1) / nth;
    *start = ith * per;
    *end = *start + per < n_out ? *start + per : n_out;
}

/* src/ops/kernel/q6_k.rs:44-80 */
void rmi_ref_q6k_forward_prepared(const uint8_t *weight, const float *d, const int8_t *qs, const int16_t *bsums,
                                  float *output, size_t n_in, size_t n_out, size_t ith, size_t nth, int variant) {
    size_t start, end;
    row_partition(n_out, ith, nth, &start, &end);
    size_t nb = n_in / QK_K;
    for (size_t r = start; r < end; r++)
        output[r] = rmi_ref_vec_dot_q6k_q8k(weight + r * nb * Q6K_BLOCK, nb, d, qs, bsums, variant);
}

/* src/ops/kernel/q6_k.rs:83-119: x = q8*scale per element, dequantised row,
 * products summed left to right (Iterator::sum; its start value, +0.0 or -0.0
 * depending on the toolchain, only decides the sign of an all-zero result). */
void rmi_ref_q6k_forward_prequantized(const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
                                      float *output, size_t n_in, size_t n_out, size_t ith, size_t nth) {
    size_t start, end;
    row_partition(n_out, ith, nth, &start, &end);
    if (start >= end) return;
    float *x = (float *)malloc(n_in * sizeof(float));
    float *row = (float *)malloc(n_in * sizeof(float));
    for (size_t i = 0; i < n_in; i++) x[i] = (float)(int8_t)input_q8[i] * input_scales[i / 32];
    size_t row_bytes = n_in / QK_K * Q6K_BLOCK;
    for (size_t r = start; r < end; r++) {
        rmi_ref_dequantize_row_q6_k(weight + r * row_bytes, row, n_in);
        float sum = 0.0f;
        for (size_t k = 0; k < n_in; k++) {
            float t = row[k] * x[k];
            sum = sum + t;
        }
        output[r] = sum;
    }
    free(x);
    free(row);
}

/* ---- the AVX2 kernel with the reference's own intrinsics
 * (src/ops/quant/mod.rs:964-1062) ---- */
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

float rmi_ref_x86_vec_dot_q6k_q8k(const uint8_t *q6k, size_t nb, const float *d8, const int8_t *qs,
                                  const int16_t *bsums) {
    const __m256i m3 = _mm256_set1_epi8(3), m15 = _mm256_set1_epi8(15);
    uint8_t shuf[8][16];
    for (int i = 0; i < 8; i++)
        for (int j = 0; j < 8; j++) {
            shuf[i][j] = (uint8_t)(2 * i);
            shuf[i][8 + j] = (uint8_t)(2 * i + 1);
        }
    __m256 acc = _mm256_setzero_ps();
    for (size_t i = 0; i < nb; i++) {
        const uint8_t *blk = q6k + i * Q6K_BLOCK;
        uint16_t hb;
        memcpy(&hb, blk + 208, 2);
        float d = _mm_cvtss_f32(_mm_cvtph_ps(_mm_set1_epi16((short)hb))) * d8[i];
        __m256i q8sums = _mm256_loadu_si256((const __m256i *)(bsums + i * 16));
        __m128i scales = _mm_loadu_si128((const __m128i *)(blk + 192));
        __m256i scales_16 = _mm256_cvtepi8_epi16(scales);
        __m256i q8sclsub = _mm256_slli_epi32(_mm256_madd_epi16(q8sums, scales_16), 5);
        __m256i sumi = _mm256_setzero_si256();
        const uint8_t *ql = blk, *qh = blk + 128;
        const int8_t *q8 = qs + i * QK_K;
        int is = 0;
        for (int j = 0; j < 2; j++) {
            __m256i q4bits1 = _mm256_loadu_si256((const __m256i *)ql);
            __m256i q4bits2 = _mm256_loadu_si256((const __m256i *)(ql + 32));
            __m256i q4bitsH = _mm256_loadu_si256((const __m256i *)qh);
            ql += 64;
            qh += 32;
            __m256i q4h_0 = _mm256_slli_epi16(_mm256_and_si256(q4bitsH, m3), 4);
            __m256i q4h_1 = _mm256_slli_epi16(_mm256_and_si256(q4bitsH, _mm256_set1_epi8(12)), 2);
            __m256i q4h_2 = _mm256_and_si256(q4bitsH, _mm256_set1_epi8(48));
            __m256i q4h_3 = _mm256_srli_epi16(_mm256_and_si256(q4bitsH, _mm256_set1_epi8((char)-64)), 2);
            __m256i q4_0 = _mm256_or_si256(_mm256_and_si256(q4bits1, m15), q4h_0);
            __m256i q4_1 = _mm256_or_si256(_mm256_and_si256(q4bits2, m15), q4h_1);
            __m256i q4_2 = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(q4bits1, 4), m15), q4h_2);
            __m256i q4_3 = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(q4bits2, 4), m15), q4h_3);
            __m256i q8_0 = _mm256_loadu_si256((const __m256i *)q8);
            __m256i q8_1 = _mm256_loadu_si256((const __m256i *)(q8 + 32));
            __m256i q8_2 = _mm256_loadu_si256((const __m256i *)(q8 + 64));
            __m256i q8_3 = _mm256_loadu_si256((const __m256i *)(q8 + 96));
            q8 += 128;
            __m256i p16_0 = _mm256_maddubs_epi16(q4_0, q8_0);
            __m256i p16_1 = _mm256_maddubs_epi16(q4_1, q8_1);
            __m256i p16_2 = _mm256_maddubs_epi16(q4_2, q8_2);
            __m256i p16_3 = _mm256_maddubs_epi16(q4_3, q8_3);
            __m128i scale_0 = _mm_shuffle_epi8(scales, _mm_loadu_si128((const __m128i *)shuf[is]));
            __m128i scale_1 = _mm_shuffle_epi8(scales, _mm_loadu_si128((const __m128i *)shuf[is + 1]));
            __m128i scale_2 = _mm_shuffle_epi8(scales, _mm_loadu_si128((const __m128i *)shuf[is + 2]));
            __m128i scale_3 = _mm_shuffle_epi8(scales, _mm_loadu_si128((const __m128i *)shuf[is + 3]));
            is += 4;
            p16_0 = _mm256_madd_epi16(_mm256_cvtepi8_epi16(scale_0), p16_0);
            p16_1 = _mm256_madd_epi16(_mm256_cvtepi8_epi16(scale_1), p16_1);
            p16_2 = _mm256_madd_epi16(_mm256_cvtepi8_epi16(scale_2), p16_2);
            p16_3 = _mm256_madd_epi16(_mm256_cvtepi8_epi16(scale_3), p16_3);
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(p16_0, p16_1));
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(p16_2, p16_3));
        }
        sumi = _mm256_sub_epi32(sumi, q8sclsub);
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    return hsum_ps(acc);
}

/* rows [ith*ceil(n_out/nth), ...) with the intrinsics kernel: one slice of the timed CPU baseline */
void rmi_ref_x86_q6k_forward_prepared(const uint8_t *weight, const float *d, const int8_t *qs, const int16_t *bsums,
                                      float *output, size_t n_in, size_t n_out, size_t ith, size_t nth) {
    size_t start, end;
    row_partition(n_out, ith, nth, &start, &end);
    size_t nb = n_in / QK_K;
    for (size_t r = start; r < end; r++)
        output[r] = rmi_ref_x86_vec_dot_q6k_q8k(weight + r * nb * Q6K_BLOCK, nb, d, qs, bsums);
}

/* y = W x over the persistent pool: rows split as (ith, nth), the AVX2 kernel per row */
typedef struct {
    const uint8_t *weight;
    const float *d;
    const int8_t *qs;
    const int16_t *bsums;
    float *output;
    size_t n_in, n_out;
} q6k_job;

static void q6k_slice(void *arg, int ith, int nth) {
    const q6k_job *j = (const q6k_job *)arg;
    rmi_ref_x86_q6k_forward_prepared(j->weight, j->d, j->qs, j->bsums, j->output, j->n_in, j->n_out, (size_t)ith,
                                     (size_t)nth);
}

void rmi_ref_pool_matmul_q6k_q8k(rmi_ref_pool *pool, const uint8_t *weight, const float *d, const int8_t *qs,
                                 const int16_t *bsums, float *output, size_t n_in, size_t n_out) {
    q6k_job job = {weight, d, qs, bsums, output, n_in, n_out};
    rmi_ref_pool_run(pool, q6k_slice, &job);
}
