/*
 * rmi_oracle.c — portable C restatement of the reference CPU kernels for the
 * quantized matrix products.  TEST INFRASTRUCTURE ONLY (see rmi_oracle.h).
 *
 * Must be compiled with -ffp-contract=off: every `a*b+c` below is two
 * roundings unless it is spelled fmaf(), exactly as in the Rust source, where
 * only explicit mul_add / _mm*_fmadd_ps calls fuse.
 *
 * Parity status of each function (what pins it without running the reference):
 *   f16 conversions ............ numpy.float16 on all 65536 patterns + random f32
 *   quantize_q8_0 .............. reference KATs (scale bits 0x3c010000, q=[127,4];
 *                                scalar [127,.5,-.5]->[127,1,-1]; ties-even 34.5->34)
 *   matmul_q8_0 scalar/avx2/neon closed-form KATs (32.0, 16.0, partition slices,
 *                                31.998047), NEON-order bit pin 0x3d1cc57d, brute
 *                                force int dots, f64 dequantised dot, intrinsics twin
 *   quantize_row_q8_k .......... reference KAT [-127,0,2,2,0], sum(bsums)==sum(qs)
 *   get_scale_min_k4 / kmask ... the reference's two formulations against each other
 *   vec_dot_q4k_q8k ............ dequant-path closed form 256.0, f64 dequantised dot,
 *                                intrinsics twin; exact f32 bits on random data are
 *                                "parity unpinned" (no golden vector exists upstream)
 *   matmul_q8_0_f32 (legacy) ... f64 dequantised dot only: "parity unpinned" at bit level
 */
#include "rmi_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define QK8_0 32
#define Q8_0_BLOCK 34
#define QK_K 256
#define Q4K_BLOCK 144

/* ------------------------------------------------------------------ f16 */

static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

float rmi_ref_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        int e = -1;
        do {
            e++;
            man <<= 1;
        } while (!(man & 0x400u));
        man &= 0x3ffu;
        return bits_f32(sign | ((uint32_t)(112 - e) << 23) | (man << 13));
    }
    if (exp == 31) {
        uint32_t quiet = man ? 0x00400000u : 0u;
        return bits_f32(sign | 0x7f800000u | quiet | (man << 13));
    }
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t rmi_ref_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) {
        if (x > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((x >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    uint32_t exp = x >> 23;
    if (exp >= 143u) return (uint16_t)(sign | 0x7c00u);
    if (exp >= 113u) {
        uint32_t man = x & 0x7fffffu;
        uint32_t h = ((exp - 112u) << 10) | (man >> 13);
        uint32_t rem = man & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    if (exp >= 102u) {
        uint32_t man = (x & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126u - exp;
        uint32_t h = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    return sign;
}

static inline float load_f16(const uint8_t *p) {
    return rmi_ref_f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
}

/* Rust `f32 as i8` after clamp: saturating, NaN -> 0. */
static inline int8_t f32_as_i8(float v) {
    if (v != v) return 0;
    if (v <= -128.0f) return -128;
    if (v >= 127.0f) return 127;
    return (int8_t)v;
}

/* _mm_max_ps(a,b): a > b ? a : b (b when unordered). */
static inline float sse_max(float a, float b) { return a > b ? a : b; }
static inline float sse_min(float a, float b) { return a < b ? a : b; }

/* ------------------------------------------------ Q8_0 activation quantizer */

static void quantize_q8_0_scalar(const float *input, size_t n, uint8_t *q8,
                                 float *scales) {
    size_t blocks = n / QK8_0;
    for (size_t b = 0; b < blocks; b++) {
        const float *v = input + b * QK8_0;
        float amax = 0.0f;
        for (int k = 0; k < QK8_0; k++) amax = fmaxf(amax, fabsf(v[k]));
        float scale = amax == 0.0f ? 0.0f : amax / 127.0f;
        float inverse = scale == 0.0f ? 0.0f : 1.0f / scale;
        scales[b] = rmi_ref_f16_to_f32(rmi_ref_f32_to_f16(scale));
        for (int k = 0; k < QK8_0; k++) {
            float r = roundf(v[k] * inverse); /* half away from zero */
            if (r < -128.0f) r = -128.0f;
            if (r > 127.0f) r = 127.0f;
            q8[b * QK8_0 + k] = (uint8_t)f32_as_i8(r);
        }
    }
}

static void quantize_q8_0_avx2(const float *input, size_t n, uint8_t *q8,
                               float *scales) {
    size_t blocks = n / QK8_0;
    for (size_t b = 0; b < blocks; b++) {
        const float *v = input + b * QK8_0;
        float m[8];
        for (int i = 0; i < 8; i++) {
            float m01 = sse_max(fabsf(v[i]), fabsf(v[8 + i]));
            float m23 = sse_max(fabsf(v[16 + i]), fabsf(v[24 + i]));
            m[i] = sse_max(m01, m23);
        }
        float m128[4];
        for (int i = 0; i < 4; i++) m128[i] = sse_max(m[4 + i], m[i]);
        float m2_0 = sse_max(m128[0], m128[1]);
        float m2_2 = sse_max(m128[2], m128[3]);
        float amax = sse_max(m2_0, m2_2);
        float d = amax == 0.0f ? 0.0f : amax / 127.0f;
        float id = amax == 0.0f ? 0.0f : 127.0f / amax;
        scales[b] = rmi_ref_f16_to_f32(rmi_ref_f32_to_f16(d));
        for (int k = 0; k < QK8_0; k++) {
            float r = nearbyintf(v[k] * id); /* ties to even */
            float c = sse_min(sse_max(r, -128.0f), 127.0f);
            q8[b * QK8_0 + k] = (uint8_t)(int8_t)(int32_t)c;
        }
    }
}

/* vmaxq_f32 / vmaxvq_f32 hand a NaN on, vcvtnq_s32_f32 turns one into 0 */
static void quantize_q8_0_neon(const float *input, size_t n, uint8_t *q8,
                               float *scales) {
    size_t blocks = n / QK8_0;
    for (size_t b = 0; b < blocks; b++) {
        const float *v = input + b * QK8_0;
        float amax = 0.0f;
        for (int k = 0; k < QK8_0; k++) amax = (isnan(v[k]) || isnan(amax)) ? NAN : fmaxf(amax, fabsf(v[k]));
        float scale = amax / 127.0f;
        float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
        scales[b] = rmi_ref_f16_to_f32(rmi_ref_f32_to_f16(scale));
        for (int k = 0; k < QK8_0; k++) {
            float t = v[k] * inv;
            int32_t i = 0;
            if (!isnan(t)) {
                float c = fminf(fmaxf(t, -127.0f), 127.0f);
                i = (int32_t)nearbyintf(c);
                if (i < -127) i = -127;
                if (i > 127) i = 127;
            }
            q8[b * QK8_0 + k] = (uint8_t)(int8_t)i;
        }
    }
}

void rmi_ref_quantize_q8_0(const float *input, size_t n, uint8_t *q8,
                           float *scales, int variant) {
    if (variant == RMI_REF_AVX2)
        quantize_q8_0_avx2(input, n, q8, scales);
    else if (variant == RMI_REF_NEON)
        quantize_q8_0_neon(input, n, q8, scales);
    else
        quantize_q8_0_scalar(input, n, q8, scales);
}

/* ------------------------------------------------------------- Q8_0 GEMV */

static inline int32_t block_dot_i8(const uint8_t *w, const uint8_t *x) {
    int32_t dot = 0;
    for (int k = 0; k < QK8_0; k++) dot += (int32_t)(int8_t)w[k] * (int32_t)(int8_t)x[k];
    return dot;
}

static inline int16_t sat16(int32_t v) {
    return (int16_t)(v > 32767 ? 32767 : (v < -32768 ? -32768 : v));
}

/* The eight int32 lanes of
 *   _mm256_madd_epi16(ones, _mm256_maddubs_epi16(sign(w,w), sign(x,w)))
 * (avx2.rs:128-147): lane L = sum of products k=4L..4L+3, built from two
 * i16-saturating pair sums, with the |w|*sign(w)x operand trick. */
static inline void avx2_lane_dots(const uint8_t *w, const uint8_t *x, int32_t p[8]) {
    int16_t pair[16];
    for (int i = 0; i < 16; i++) {
        int32_t acc = 0;
        for (int t = 0; t < 2; t++) {
            int8_t wv = (int8_t)w[2 * i + t];
            int8_t xv = (int8_t)x[2 * i + t];
            uint8_t ax = (uint8_t)(wv < 0 ? (int8_t)(-wv) : wv); /* -128 stays 0x80 */
            int8_t sy = wv < 0 ? (int8_t)(-xv) : (wv == 0 ? 0 : xv);
            acc += (int32_t)ax * (int32_t)sy;
        }
        pair[i] = sat16(acc);
    }
    for (int L = 0; L < 8; L++) p[L] = (int32_t)pair[2 * L] + (int32_t)pair[2 * L + 1];
}

/* hsum_ps, src/ops/dot.rs:447-456 */
static inline float hsum8(const float a[8]) {
    float s0 = a[4] + a[0], s1 = a[5] + a[1], s2 = a[6] + a[2], s3 = a[7] + a[3];
    return (s0 + s1) + (s2 + s3);
}

static float row_dot_scalar(const uint8_t *row, const uint8_t *q8, const float *xs,
                            size_t blocks) {
    float sum = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *blk = row + b * Q8_0_BLOCK;
        float wd = load_f16(blk);
        int32_t dot = block_dot_i8(blk + 2, q8 + b * QK8_0);
        float t = wd * xs[b];
        t = t * (float)dot;
        sum = sum + t;
    }
    return sum;
}

static float row_dot_avx2(const uint8_t *row, const uint8_t *q8, const float *xs,
                          size_t blocks) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *blk = row + b * Q8_0_BLOCK;
        float s = load_f16(blk) * xs[b];
        int32_t p[8];
        avx2_lane_dots(blk + 2, q8 + b * QK8_0, p);
        for (int L = 0; L < 8; L++) acc[L] = fmaf(s, (float)p[L], acc[L]);
    }
    return hsum8(acc);
}

static float row_dot_neon(const uint8_t *row, const uint8_t *q8, const float *xs,
                          size_t blocks) {
    float sum = 0.0f;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t *blk = row + b * Q8_0_BLOCK;
        float wd = load_f16(blk);
        int32_t dot = block_dot_i8(blk + 2, q8 + b * QK8_0);
        sum = fmaf((float)dot, wd * xs[b], sum);
    }
    return sum;
}

void rmi_ref_matmul_q8_0_quantized_range(const uint8_t *weight,
                                         const uint8_t *input_q8,
                                         const float *input_scales,
                                         float *output, size_t n_in,
                                         size_t row_start, size_t row_end,
                                         int variant) {
    size_t blocks = n_in / QK8_0;
    size_t stride = blocks * Q8_0_BLOCK;
    for (size_t r = row_start; r < row_end; r++) {
        const uint8_t *row = weight + r * stride;
        float y;
        if (variant == RMI_REF_AVX2)
            y = row_dot_avx2(row, input_q8, input_scales, blocks);
        else if (variant == RMI_REF_NEON)
            y = row_dot_neon(row, input_q8, input_scales, blocks);
        else
            y = row_dot_scalar(row, input_q8, input_scales, blocks);
        output[r - row_start] = y;
    }
}

/* Not a function of the reference: the aarch64 kernel's chain (neon.rs:49-73) cut into runs of quads_per_part whole
 * quads (4 blocks), each run summed in block order from zero, the runs' sums added in run order.  It is what the
 * device's split-K GEMM promises to compute; one run is row_dot_neon itself, and tests hold every split to the
 * reference orders within the reference's own tolerance. */
void rmi_ref_matmul_q8_0_neon_split(const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
                                    float *output, size_t n_in, size_t n_out, size_t quads_per_part) {
    size_t blocks = n_in / QK8_0, quads = (blocks + 3) / 4;
    size_t per = quads_per_part ? quads_per_part : 1;
    size_t k_parts = (quads + per - 1) / per;
    if (k_parts == 0) k_parts = 1;
    for (size_t r = 0; r < n_out; r++) {
        const uint8_t *row = weight + r * blocks * Q8_0_BLOCK;
        float total = 0.0f;
        for (size_t p = 0; p < k_parts; p++) {
            size_t b0 = p * per * 4, b1 = (p + 1) * per * 4;
            if (b1 > blocks) b1 = blocks;
            float sum = 0.0f;
            for (size_t b = b0; b < b1; b++) {
                const uint8_t *blk = row + b * Q8_0_BLOCK;
                sum = fmaf((float)block_dot_i8(blk + 2, input_q8 + b * QK8_0), load_f16(blk) * input_scales[b], sum);
            }
            total = p == 0 ? sum : total + sum;
        }
        output[r] = total;
    }
}

/* Not a function of the reference either: the chain cut into n_groups interleaved chains, group g taking the quads
 * g, g + n_groups, g + 2 n_groups, ... in order from zero, the groups' sums added in group order (the device's tiled
 * GEMM with groups of waves; n_groups = 1 is row_dot_neon). */
void rmi_ref_matmul_q8_0_neon_interleaved(const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
                                          float *output, size_t n_in, size_t n_out, size_t n_groups) {
    size_t blocks = n_in / QK8_0;
    if (n_groups == 0) n_groups = 1;
    for (size_t r = 0; r < n_out; r++) {
        const uint8_t *row = weight + r * blocks * Q8_0_BLOCK;
        float total = 0.0f;
        for (size_t g = 0; g < n_groups; g++) {
            float sum = 0.0f;
            for (size_t b = 0; b < blocks; b++) {
                if ((b / 4) % n_groups != g) continue;
                const uint8_t *blk = row + b * Q8_0_BLOCK;
                sum = fmaf((float)block_dot_i8(blk + 2, input_q8 + b * QK8_0), load_f16(blk) * input_scales[b], sum);
            }
            total = g == 0 ? sum : total + sum;
        }
        output[r] = total;
    }
}

void rmi_ref_matmul_q8_0_quantized_parallel_rows(
    const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
    float *output, size_t n_in, size_t n_out, size_t ith, size_t nth,
    int variant) {
    if (nth <= 1 || n_out == 0) {
        rmi_ref_matmul_q8_0_quantized_range(weight, input_q8, input_scales, output,
                                            n_in, 0, n_out, variant);
        return;
    }
    size_t per_thread = (n_out + nth - 1) / nth;
    size_t my_start = ith * per_thread;
    size_t my_end = my_start + per_thread < n_out ? my_start + per_thread : n_out;
    if (my_start >= my_end) return;
    rmi_ref_matmul_q8_0_quantized_range(weight, input_q8, input_scales,
                                        output + my_start, n_in, my_start, my_end,
                                        variant);
}

void rmi_ref_block_dots_q8_0(const uint8_t *weight, const uint8_t *input_q8,
                             int32_t *dots, size_t n_in, size_t n_out) {
    size_t blocks = n_in / QK8_0;
    for (size_t r = 0; r < n_out; r++)
        for (size_t b = 0; b < blocks; b++)
            dots[r * blocks + b] = block_dot_i8(
                weight + (r * blocks + b) * Q8_0_BLOCK + 2, input_q8 + b * QK8_0);
}

void rmi_ref_matmul_q8_0_f32(const uint8_t *weight, const float *input,
                             float *output, size_t n_in, size_t n_out,
                             int variant) {
    size_t blocks = n_in / QK8_0;
    size_t stride = blocks * Q8_0_BLOCK;
    for (size_t r = 0; r < n_out; r++) {
        const uint8_t *row = weight + r * stride;
        if (variant == RMI_REF_AVX2) {
            float acc0[8] = {0}, acc1[8] = {0};
            for (size_t b = 0; b < blocks; b++) {
                const uint8_t *blk = row + b * Q8_0_BLOCK;
                float d = load_f16(blk);
                const float *inp = input + b * QK8_0;
                for (int g = 0; g < 4; g++) {
                    float *acc = (g & 1) ? acc1 : acc0;
                    for (int i = 0; i < 8; i++) {
                        float wq = d * (float)(int8_t)blk[2 + g * 8 + i];
                        acc[i] = fmaf(wq, inp[g * 8 + i], acc[i]);
                    }
                }
            }
            float s[8];
            for (int i = 0; i < 8; i++) s[i] = acc0[i] + acc1[i];
            output[r] = hsum8(s);
        } else {
            float sum = 0.0f;
            for (size_t b = 0; b < blocks; b++) {
                const uint8_t *blk = row + b * Q8_0_BLOCK;
                float d = load_f16(blk);
                float local = 0.0f;
                for (int k = 0; k < QK8_0; k++) {
                    float t = (float)(int8_t)blk[2 + k] * input[b * QK8_0 + k];
                    local = local + t;
                }
                float t = d * local;
                sum = sum + t;
            }
            output[r] = sum;
        }
    }
}

void rmi_ref_q8_0_forward_batched(const uint8_t *weight, const float *input,
                                  float *output, size_t n_in, size_t n_out,
                                  size_t n_tokens, int variant) {
    size_t nb = (n_in + 31) / 32;
    uint8_t *q8 = (uint8_t *)malloc(n_in ? n_in : 1);
    float *sc = (float *)malloc((nb ? nb : 1) * sizeof(float));
    for (size_t t = 0; t < n_tokens; t++) {
        rmi_ref_quantize_q8_0(input + t * n_in, n_in, q8, sc, variant);
        rmi_ref_matmul_q8_0_quantized_range(weight, q8, sc, output + t * n_out, n_in,
                                            0, n_out, variant);
    }
    free(q8);
    free(sc);
}

size_t rmi_ref_fuse_vstack(const uint8_t *a, size_t a_len, size_t a_rows,
                           const uint8_t *b, size_t b_len, size_t b_rows,
                           uint8_t *fused) {
    size_t row_bytes_a = a_len / (a_rows ? a_rows : 1);
    size_t row_bytes_b = b_len / (b_rows ? b_rows : 1);
    if (row_bytes_a != row_bytes_b) return 0;
    memcpy(fused, a, a_len);
    memcpy(fused + a_len, b, b_len);
    return a_rows + b_rows;
}

/* ---------------------------------------------------------------- Q8_K */

static inline int32_t nearest_int_magic(float value) {
    float t = value + 12582912.0f;
    return (int32_t)(f32_bits(t) & 0x007fffffu) - 0x00400000;
}

void rmi_ref_quantize_row_q8_k(const float *x, size_t n, float *d, int8_t *qs,
                               int16_t *bsums, int variant) {
    size_t nb = n / QK_K;
    for (size_t i = 0; i < nb; i++) {
        const float *block = x + i * QK_K;
        int8_t *q = qs + i * QK_K;
        float amax = 0.0f, max_val = 0.0f;
        for (int j = 0; j < QK_K; j++) {
            float ax = fabsf(block[j]);
            if (ax > amax) {
                amax = ax;
                max_val = block[j];
            }
        }
        if (amax == 0.0f) {
            d[i] = 0.0f;
            memset(q, 0, QK_K);
            memset(bsums + i * 16, 0, 16 * sizeof(int16_t));
            continue;
        }
        float iscale = -127.0f / max_val;
        for (int j = 0; j < QK_K; j++) {
            if (variant == RMI_REF_AVX2) {
                int32_t v = (int32_t)nearbyintf(block[j] * iscale);
                if (v < -127) v = -127;
                if (v > 127) v = 127;
                q[j] = (int8_t)v;
            } else {
                int32_t v = nearest_int_magic(iscale * block[j]);
                if (v > 127) v = 127;
                q[j] = (int8_t)v;
            }
        }
        for (int g = 0; g < 16; g++) {
            int32_t sum = 0;
            for (int k = 0; k < 16; k++) sum += q[g * 16 + k];
            bsums[i * 16 + g] = (int16_t)sum;
        }
        d[i] = 1.0f / iscale;
    }
}

/* ---------------------------------------------------------------- Q4_K */

void rmi_ref_get_scale_min_k4(int j, const uint8_t *s, uint8_t *sc, uint8_t *mn) {
    if (j < 4) {
        *sc = s[j] & 63;
        *mn = s[j + 4] & 63;
    } else {
        *sc = (uint8_t)((s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4));
        *mn = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}

void rmi_ref_unpack_scales_kmask(const uint8_t *s, uint8_t *out16) {
    uint32_t utmp[4];
    utmp[0] = (uint32_t)s[0] | ((uint32_t)s[1] << 8) | ((uint32_t)s[2] << 16) | ((uint32_t)s[3] << 24);
    utmp[1] = (uint32_t)s[4] | ((uint32_t)s[5] << 8) | ((uint32_t)s[6] << 16) | ((uint32_t)s[7] << 24);
    utmp[2] = (uint32_t)s[8] | ((uint32_t)s[9] << 8) | ((uint32_t)s[10] << 16) | ((uint32_t)s[11] << 24);
    const uint32_t kmask1 = 0x3f3f3f3fu, kmask2 = 0x0f0f0f0fu, kmask3 = 0x03030303u;
    utmp[3] = ((utmp[2] >> 4) & kmask2) | (((utmp[1] >> 6) & kmask3) << 4);
    uint32_t uaux = utmp[1] & kmask1;
    utmp[1] = (utmp[2] & kmask2) | (((utmp[0] >> 6) & kmask3) << 4);
    utmp[2] = uaux;
    utmp[0] &= kmask1;
    for (int k = 0; k < 4; k++)
        for (int t = 0; t < 4; t++) out16[k * 4 + t] = (uint8_t)(utmp[k] >> (8 * t));
}

/* element e (0..255) of a Q4_K super-block's 4-bit quants, mod.rs:226-235 */
static inline int32_t q4k_elem(const uint8_t *qs128, int e) {
    int g = e >> 6, r = e & 63;
    uint8_t byte = qs128[g * 32 + (r & 31)];
    return r < 32 ? (byte & 0xF) : (byte >> 4);
}

static float vec_dot_q4k_q8k_scalar(const uint8_t *w, size_t nb, const float *d8,
                                    const int8_t *qs, const int16_t *bsums) {
    float sums[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    float sumf = 0.0f;
    for (size_t i = 0; i < nb; i++) {
        const uint8_t *blk = w + i * Q4K_BLOCK;
        float d = load_f16(blk), dmin = load_f16(blk + 2);
        uint8_t sm[16];
        rmi_ref_unpack_scales_kmask(blk + 4, sm);
        const int8_t *q8 = qs + i * QK_K;
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) sumi += (int32_t)bsums[i * 16 + j] * (int32_t)sm[8 + j / 2];
        int32_t aux32[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        int idx = 0;
        for (int j = 0; j < 8; j++) {
            int32_t scale = sm[j];
            for (int t = 0; t < 4; t++)
                for (int l = 0; l < 8; l++, idx++)
                    aux32[l] += scale * (int32_t)q8[idx] * q4k_elem(blk + 16, idx);
        }
        float dd = d * d8[i];
        for (int l = 0; l < 8; l++) {
            float t = dd * (float)aux32[l];
            sums[l] = sums[l] + t;
        }
        float dmin_val = dmin * d8[i];
        float t = dmin_val * (float)sumi;
        sumf = sumf - t;
    }
    for (int l = 0; l < 8; l++) sumf = sumf + sums[l];
    return sumf;
}

static float vec_dot_q4k_q8k_avx2(const uint8_t *w, size_t nb, const float *d8,
                                  const int8_t *qs, const int16_t *bsums) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    float acc_m[4] = {0, 0, 0, 0};
    for (size_t i = 0; i < nb; i++) {
        const uint8_t *blk = w + i * Q4K_BLOCK;
        float d = load_f16(blk) * d8[i];
        float dmin = -load_f16(blk + 2) * d8[i];
        uint8_t sm[16];
        rmi_ref_unpack_scales_kmask(blk + 4, sm);
        const int16_t *bs = bsums + i * 16;
        /* _mm_hadd_epi16 wraps in i16 */
        int16_t q8s[8];
        for (int j = 0; j < 8; j++) q8s[j] = (int16_t)(bs[2 * j] + bs[2 * j + 1]);
        for (int t = 0; t < 4; t++) {
            int32_t prod = (int32_t)sm[8 + 2 * t] * q8s[2 * t] + (int32_t)sm[8 + 2 * t + 1] * q8s[2 * t + 1];
            acc_m[t] = fmaf(dmin, (float)prod, acc_m[t]);
        }
        const int8_t *q8 = qs + i * QK_K;
        int32_t sumi[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int j = 0; j < 4; j++) {
            const uint8_t *q4 = blk + 16 + j * 32;
            for (int T = 0; T < 8; T++) {
                int32_t lo = 0, hi = 0;
                for (int p = 0; p < 2; p++) {
                    /* maddubs: u8*i8 pair sum saturating to i16 */
                    int k = 4 * T + 2 * p;
                    int32_t l2 = (int32_t)(q4[k] & 0xF) * q8[64 * j + k] +
                                 (int32_t)(q4[k + 1] & 0xF) * q8[64 * j + k + 1];
                    int32_t h2 = (int32_t)(q4[k] >> 4) * q8[64 * j + 32 + k] +
                                 (int32_t)(q4[k + 1] >> 4) * q8[64 * j + 32 + k + 1];
                    lo += (int32_t)sm[2 * j] * sat16(l2);
                    hi += (int32_t)sm[2 * j + 1] * sat16(h2);
                }
                sumi[T] += lo + hi;
            }
        }
        for (int T = 0; T < 8; T++) acc[T] = fmaf(d, (float)sumi[T], acc[T]);
    }
    float min_val = (acc_m[0] + acc_m[2]) + (acc_m[1] + acc_m[3]);
    float main_val = hsum8(acc);
    return main_val + min_val;
}

float rmi_ref_vec_dot_q4k_q8k(const uint8_t *q4k_row, size_t n_blocks,
                              const float *d, const int8_t *qs,
                              const int16_t *bsums, int variant) {
    if (variant == RMI_REF_AVX2) return vec_dot_q4k_q8k_avx2(q4k_row, n_blocks, d, qs, bsums);
    return vec_dot_q4k_q8k_scalar(q4k_row, n_blocks, d, qs, bsums);
}

void rmi_ref_q4k_q8k_block_ints(const uint8_t *w, size_t nb, const int8_t *qs,
                                const int16_t *bsums, int32_t *isum,
                                int32_t *msum) {
    for (size_t i = 0; i < nb; i++) {
        const uint8_t *blk = w + i * Q4K_BLOCK;
        int32_t si = 0, smn = 0;
        for (int j = 0; j < 8; j++) {
            uint8_t sc, mn;
            rmi_ref_get_scale_min_k4(j, blk + 4, &sc, &mn);
            int32_t dot = 0;
            for (int k = 0; k < 32; k++)
                dot += (int32_t)qs[i * QK_K + 32 * j + k] * q4k_elem(blk + 16, 32 * j + k);
            si += (int32_t)sc * dot;
            smn += (int32_t)mn * ((int32_t)bsums[i * 16 + 2 * j] + (int32_t)bsums[i * 16 + 2 * j + 1]);
        }
        isum[i] = si;
        msum[i] = smn;
    }
}

/* the same integers for every row of a weight against one token: ints[n_out][nb][2] = {isum, msum} */
void rmi_ref_q4k_q8k_block_ints_matrix(const uint8_t *w, size_t n_out, size_t nb, const int8_t *qs,
                                       const int16_t *bsums, int32_t *ints) {
    for (size_t r = 0; r < n_out; r++) {
        int32_t isum[nb], msum[nb];
        rmi_ref_q4k_q8k_block_ints(w + r * nb * Q4K_BLOCK, nb, qs, bsums, isum, msum);
        for (size_t i = 0; i < nb; i++) {
            ints[(r * nb + i) * 2] = isum[i];
            ints[(r * nb + i) * 2 + 1] = msum[i];
        }
    }
}

void rmi_ref_dequantize_row_q4_k(const uint8_t *blocks, float *output, size_t n) {
    size_t nb = n / QK_K;
    for (size_t bi = 0; bi < nb; bi++) {
        const uint8_t *blk = blocks + bi * Q4K_BLOCK;
        float d = load_f16(blk), dmin = load_f16(blk + 2);
        float *out = output + bi * QK_K;
        for (int g = 0; g < 4; g++) {
            uint8_t sc1, m1, sc2, m2;
            rmi_ref_get_scale_min_k4(2 * g, blk + 4, &sc1, &m1);
            rmi_ref_get_scale_min_k4(2 * g + 1, blk + 4, &sc2, &m2);
            float d1 = d * (float)sc1, m1e = dmin * (float)m1;
            float d2 = d * (float)sc2, m2e = dmin * (float)m2;
            for (int l = 0; l < 32; l++) {
                uint8_t ql = blk[16 + g * 32 + l];
                float a = d1 * (float)(ql & 0xF);
                float b = d2 * (float)(ql >> 4);
                out[64 * g + l] = a - m1e;
                out[64 * g + 32 + l] = b - m2e;
            }
        }
    }
}

static void row_partition(size_t n_out, size_t ith, size_t nth, size_t *start,
                          size_t *end) {
    if (nth == 0) nth = 1;
    size_t per = (n_out + nth - 1) / nth;
    *start = ith * per;
    *end = *start + per < n_out ? *start + per : n_out;
}

void rmi_ref_q4k_forward_prepared(const uint8_t *weight, const float *d,
                                  const int8_t *qs, const int16_t *bsums,
                                  float *output, size_t n_in, size_t n_out,
                                  size_t ith, size_t nth, int variant) {
    size_t start, end;
    row_partition(n_out, ith, nth, &start, &end);
    size_t nb = n_in / QK_K;
    for (size_t r = start; r < end; r++)
        output[r] = rmi_ref_vec_dot_q4k_q8k(weight + r * nb * Q4K_BLOCK, nb, d, qs, bsums, variant);
}

void rmi_ref_q4k_forward_prequantized(const uint8_t *weight,
                                      const uint8_t *input_q8,
                                      const float *input_scales,
                                      float *output, size_t n_in,
                                      size_t n_out, size_t ith, size_t nth) {
    size_t start, end;
    row_partition(n_out, ith, nth, &start, &end);
    if (start >= end) return;
    float *x = (float *)malloc(n_in * sizeof(float));
    float *row = (float *)malloc(n_in * sizeof(float));
    for (size_t i = 0; i < n_in; i++) x[i] = (float)(int8_t)input_q8[i] * input_scales[i / 32];
    size_t row_bytes = n_in / QK_K * Q4K_BLOCK;
    for (size_t r = start; r < end; r++) {
        rmi_ref_dequantize_row_q4_k(weight + r * row_bytes, row, n_in);
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

void rmi_ref_quantized_linear_forward(const uint8_t *weight,
                                      const float *input, float *output,
                                      size_t in_features,
                                      size_t out_features) {
    float *row = (float *)malloc(in_features * sizeof(float));
    size_t row_bytes = in_features / QK_K * Q4K_BLOCK;
    for (size_t i = 0; i < out_features; i++) {
        rmi_ref_dequantize_row_q4_k(weight + i * row_bytes, row, in_features);
        float sum = 0.0f;
        for (size_t j = 0; j < in_features; j++) {
            float t = row[j] * input[j];
            sum = sum + t;
        }
        output[i] = sum;
    }
    free(row);
}

/* ---- expf of the platform libm, restated (glibc >= 2.27, the FMA build that
 * hosts with AVX2 select): x*32/ln2 = k + r in f64, 2^(k/32) from a table, a
 * cubic in r; the reduction and the three polynomial steps are fused
 * multiply-adds.  The reference's f32::exp (softmax, SiLU) resolves to that
 * function; the GPU kernels carry the same formula.  rmi_ref_expf_mismatches
 * compares it with this host's expf. ---- */
static const uint64_t k_exp2f_tab[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull,
};

float rmi_ref_expf_restated(float x) {
    uint32_t ux, abstop;
    memcpy(&ux, &x, 4);
    abstop = (ux >> 20) & 0x7ff;
    if (abstop >= (0x42b00000u >> 20)) { /* |x| >= 88 or NaN */
        if (ux == 0xff800000u) return 0.0f;
        if (abstop >= (0x7f800000u >> 20)) return x + x;
        if (x > 0x1.62e42ep6f) return INFINITY;
        if (x < -0x1.9fe368p6f) return 0.0f;
    }
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32, shift = 0x1.8p+52;
    const double c0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32, c1 = 0x1.ebfce50fac4f3p-3 / 32 / 32,
                 c2 = 0x1.62e42ff0c52d6p-1 / 32;
    double xd = (double)x, z = inv_ln2_n * xd, kd = z + shift, r, s, p, r2, y;
    uint64_t ki, t;
    memcpy(&ki, &kd, 8);
    kd -= shift;
    r = fma(inv_ln2_n, xd, -kd);
    t = k_exp2f_tab[ki & 31] + (ki << 47);
    memcpy(&s, &t, 8);
    p = fma(c0, r, c1);
    r2 = r * r;
    y = fma(c2, r, 1.0);
    y = fma(p, r2, y);
    y = y * s;
    return (float)y;
}

/* inputs with bit patterns first, first+stride, ... (count of them): how many differ from the host's expf */
uint64_t rmi_ref_expf_mismatches(uint32_t first, uint32_t stride, uint64_t count) {
    uint64_t bad = 0;
    uint32_t b = first;
    for (uint64_t i = 0; i < count; i++, b += stride) {
        float x, a, m;
        uint32_t ua, um;
        memcpy(&x, &b, 4);
        a = expf(x);
        m = rmi_ref_expf_restated(x);
        memcpy(&ua, &a, 4);
        memcpy(&um, &m, 4);
        if (ua != um && !(a != a && m != m)) bad++;
    }
    return bad;
}

/* y[i] = exp(x[i]): which = 0 the host's expf, 1 the restatement */
void rmi_ref_expf_array(const float *x, float *y, size_t n, int which) {
    for (size_t i = 0; i < n; i++) y[i] = which ? rmi_ref_expf_restated(x[i]) : expf(x[i]);
}
