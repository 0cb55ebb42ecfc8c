/*
 * rmi_q4_0.c — the reference's Q4_0 x Q8_0 matmul restated.  TEST INFRASTRUCTURE ONLY
 * (see rmi_oracle.h).
 *
 * Q4_0 block, 18 bytes, 32 elements (src/ops/kernel/q4_0/scalar.rs:24-25, 38-47):
 *   [0..2) f16 d, [2..18) 16 bytes; element l (l < 16) = low nibble of byte l, element 16 + l = high nibble,
 *   value = nibble - 8.
 * Per row one f32 accumulator, block after block: sum += (float(dot) * d) * scale (two roundings, then the
 * add); the AVX2 kernel (avx2.rs:24-105) is written to give the same bits as the scalar one.
 */
#include "rmi_oracle.h"

#include <immintrin.h>
#include <string.h>

#define Q40_BLOCK 18

static inline float load_f16(const uint8_t *p) {
    return rmi_ref_f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
}

static int32_t q4_0_block_dot(const uint8_t *blk, const uint8_t *q8) {
    int32_t dot = 0;
    for (int l = 0; l < 16; l++) {
        int32_t x0 = (int32_t)(blk[2 + l] & 0x0F) - 8, x1 = (int32_t)(blk[2 + l] >> 4) - 8;
        dot += x0 * (int32_t)(int8_t)q8[l] + x1 * (int32_t)(int8_t)q8[16 + l];
    }
    return dot;
}

/* src/ops/kernel/q4_0/scalar.rs:13-52 */
void rmi_ref_matmul_q4_0_scalar_range(const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
                                      float *output, size_t n_in, size_t n_out, size_t ith, size_t nth) {
    size_t nb = n_in / 32, stride = nb * Q40_BLOCK;
    if (nth == 0) nth = 1;
    size_t per = (n_out + nth - 1) / nth, start = ith * per, end = start + per < n_out ? start + per : n_out;
    for (size_t r = start; r < end; r++) {
        float sum = 0.0f;
        for (size_t b = 0; b < nb; b++) {
            const uint8_t *blk = weight + r * stride + b * Q40_BLOCK;
            float d = load_f16(blk);
            int32_t dot = q4_0_block_dot(blk, input_q8 + 32 * b);
            float t = (float)dot * d;
            t = t * input_scales[b];
            sum = sum + t;
        }
        output[r] = sum;
    }
}

/* dots[r * nb + b] = sum over the block of (nibble - 8) * q8 */
void rmi_ref_block_dots_q4_0(const uint8_t *weight, const uint8_t *input_q8, int32_t *dots, size_t n_in, size_t n_out) {
    size_t nb = n_in / 32;
    for (size_t r = 0; r < n_out; r++)
        for (size_t b = 0; b < nb; b++)
            dots[r * nb + b] = q4_0_block_dot(weight + (r * nb + b) * Q40_BLOCK, input_q8 + 32 * b);
}

/* ---- the AVX2 kernel with the reference's own intrinsics (src/ops/kernel/q4_0/avx2.rs:24-190) ---- */
static inline int32_t hsum_epi32(__m256i v) {
    __m128i hi128 = _mm256_extracti128_si256(v, 1), lo128 = _mm256_castsi256_si128(v);
    __m128i sum128 = _mm_add_epi32(hi128, lo128);
    __m128i t = _mm_add_epi32(sum128, _mm_srli_si128(sum128, 8));
    __m128i r = _mm_add_epi32(t, _mm_srli_si128(t, 4));
    return _mm_cvtsi128_si32(r);
}

static inline float x86_block_dot(__m128i q4_bytes, __m256i q8_input) {
    const __m128i low_mask = _mm_set1_epi8(0x0F);
    const __m256i ones = _mm256_set1_epi16(1);
    __m128i lo = _mm_and_si128(q4_bytes, low_mask);
    __m128i hi = _mm_and_si128(_mm_srli_epi16(q4_bytes, 4), low_mask);
    __m256i q4_unpacked = _mm256_set_m128i(hi, lo);
    __m256i prod16 = _mm256_maddubs_epi16(q4_unpacked, q8_input);
    __m256i prod32 = _mm256_madd_epi16(ones, prod16);
    __m256i y_lo16 = _mm256_cvtepi8_epi16(_mm256_castsi256_si128(q8_input));
    __m256i y_hi16 = _mm256_cvtepi8_epi16(_mm256_extracti128_si256(q8_input, 1));
    __m256i y_sum32 = _mm256_add_epi32(_mm256_madd_epi16(ones, y_lo16), _mm256_madd_epi16(ones, y_hi16));
    int32_t corrected = hsum_epi32(prod32) - 8 * hsum_epi32(y_sum32);
    return (float)corrected;
}

void rmi_ref_x86_matmul_q4_0_range(const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
                                   float *output, size_t n_in, size_t row_start, size_t row_end) {
    size_t nb = n_in / 32, stride = nb * Q40_BLOCK;
    for (size_t row = row_start, i = 0; row < row_end; row++, i++) {
        float acc = 0.0f;
        for (size_t b = 0; b < nb; b++) {  /* the reference's two-block unroll adds block by block as well */
            const uint8_t *blk = weight + row * stride + b * Q40_BLOCK;
            uint16_t hb;
            memcpy(&hb, blk, 2);
            float d = _mm_cvtss_f32(_mm_cvtph_ps(_mm_set1_epi16((short)hb)));
            float dc = x86_block_dot(_mm_loadu_si128((const __m128i *)(blk + 2)),
                                     _mm256_loadu_si256((const __m256i *)(input_q8 + 32 * b)));
            float t = dc * d;
            t = t * input_scales[b];
            acc = acc + t;
        }
        output[i] = acc;
    }
}

/* y = W x over the persistent pool: rows split as (ith, nth) (q4_0/mod.rs:46-51), the AVX2 kernel per slice */
typedef struct {
    const uint8_t *weight, *q8;
    const float *scales;
    float *output;
    size_t n_in, n_out;
} q40_job;

static void q40_slice(void *arg, int ith, int nth) {
    const q40_job *j = (const q40_job *)arg;
    size_t per = (j->n_out + (size_t)nth - 1) / (size_t)nth, start = (size_t)ith * per;
    size_t end = start + per < j->n_out ? start + per : j->n_out;
    if (start < end) rmi_ref_x86_matmul_q4_0_range(j->weight, j->q8, j->scales, j->output + start, j->n_in, start, end);
}

void rmi_ref_pool_matmul_q4_0(rmi_ref_pool *pool, const uint8_t *weight, const uint8_t *input_q8,
                              const float *input_scales, float *output, size_t n_in, size_t n_out) {
    q40_job job = {weight, input_q8, input_scales, output, n_in, n_out};
    rmi_ref_pool_run(pool, q40_slice, &job);
}
