/*
 * rmi_oracle.h — CPU restatement of rust-model-inference's quantized matrix
 * products.  TEST INFRASTRUCTURE ONLY: this library is the checker that the
 * HIP kernels are compared against and the CPU baseline that is timed beside
 * them.  Nothing in the shipped GPU path links, loads or calls it.
 *
 * Every function follows one reference function in arithmetic order; the
 * reference file:line is cited at each declaration (paths are relative to the
 * reference repository root).  Three f32 accumulation orders exist in the
 * reference for the same Q8_0 GEMV (scalar, AVX2, NEON); each is restated
 * separately because they differ in the last bits.
 *
 * Pinned by reference-held known-answer vectors (see tests/test_oracle_*.py);
 * functions for which no reference vector exists are cross-pinned against an
 * independent formulation (brute-force integer dots, f64 dequantised dots,
 * numpy.float16, the intrinsics twin in rmi_oracle_avx2.c).
 */
#ifndef RMI_ORACLE_H
#define RMI_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    RMI_REF_SCALAR = 0, /* portable scalar kernels                        */
    RMI_REF_AVX2 = 1,   /* x86-64 production kernels (AVX2+FMA order)     */
    RMI_REF_NEON = 2    /* aarch64 production kernels (fused sequential)  */
};

/* src/ops/float.rs:177-207 — IEEE binary16 <-> binary32, round-to-nearest-even */
float rmi_ref_f16_to_f32(uint16_t bits);
uint16_t rmi_ref_f32_to_f16(float v);

/* expf of the platform libm restated (the formula the GPU kernels use), and a check against the host's expf */
float rmi_ref_expf_restated(float x);
uint64_t rmi_ref_expf_mismatches(uint32_t first, uint32_t stride, uint64_t count);
void rmi_ref_expf_array(const float *x, float *y, size_t n, int which);

/* src/ops/quant/q8_0.rs:49-71 (scalar), :176-230 (AVX2), :75-164 (NEON).
 * q8[n] int8 bit patterns, scales[n/32] f32 holding f16-rounded values. */
void rmi_ref_quantize_q8_0(const float *input, size_t n, uint8_t *q8,
                           float *scales, int variant);

/* src/ops/kernel/q8_0/scalar.rs:31-58, avx2.rs:53-174, neon.rs:49-73.
 * output[0] is row_start (the pre-sliced convention of dispatch.rs:36). */
void rmi_ref_matmul_q8_0_quantized_range(const uint8_t *weight,
                                         const uint8_t *input_q8,
                                         const float *input_scales,
                                         float *output, size_t n_in,
                                         size_t row_start, size_t row_end,
                                         int variant);

/* src/ops/kernel/q8_0/parallel.rs:102-139 — full-length output, writes only
 * rows [ith*ceil(n_out/nth), ...). */
void rmi_ref_matmul_q8_0_quantized_parallel_rows(
    const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
    float *output, size_t n_in, size_t n_out, size_t ith, size_t nth,
    int variant);

/* The "per-block int32 dot" of scalar.rs:49-53: dots[row*n_in/32 + block]. */
/* the aarch64 chain cut into runs of quads_per_part whole quads (128 elements each), runs summed in order (the
 * device's split-K GEMM; not a function of the reference) */
void rmi_ref_matmul_q8_0_neon_split(const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
                                    float *output, size_t n_in, size_t n_out, size_t quads_per_part);
/* the aarch64 chain as n_groups interleaved chains of quads, the groups' sums added in order (the device's tiled
 * GEMM with groups of waves; not a function of the reference) */
void rmi_ref_matmul_q8_0_neon_interleaved(const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
                                          float *output, size_t n_in, size_t n_out, size_t n_groups);
void rmi_ref_block_dots_q8_0(const uint8_t *weight, const uint8_t *input_q8,
                             int32_t *dots, size_t n_in, size_t n_out);

/* src/ops/kernel/q8_0/scalar.rs:3-29 (variant SCALAR) and avx2.rs:180-217
 * (variant AVX2): the f32-activation `matmul_q8_0` of parallel.rs:317-341. */
void rmi_ref_matmul_q8_0_f32(const uint8_t *weight, const float *input,
                             float *output, size_t n_in, size_t n_out,
                             int variant);

/* src/ops/kernel/trait_.rs:59-109 — Kernel::forward / forward_batched for a
 * Q8_0 weight: quantize each token row, one GEMV per token, token-major out. */
void rmi_ref_q8_0_forward_batched(const uint8_t *weight, const float *input,
                                  float *output, size_t n_in, size_t n_out,
                                  size_t n_tokens, int variant);

/* src/ops/quant/fuse.rs:25-64 — byte concat of two row-stacked weights.
 * Returns fused row count, or 0 when the per-row byte lengths differ
 * (the reference's `None`).  `fused` must hold a_len+b_len bytes. */
size_t rmi_ref_fuse_vstack(const uint8_t *a, size_t a_len, size_t a_rows,
                           const uint8_t *b, size_t b_len, size_t b_rows,
                           uint8_t *fused);

/* src/ops/quant/mod.rs:75-122 (scalar), :140-200 (AVX2).  SoA output:
 * d[n/256], qs[n], bsums[n/16]. */
void rmi_ref_quantize_row_q8_k(const float *x, size_t n, float *d, int8_t *qs,
                               int16_t *bsums, int variant);

/* src/ops/quant/mod.rs:25-33 */
void rmi_ref_get_scale_min_k4(int j, const uint8_t *scales12, uint8_t *sc,
                              uint8_t *mn);
/* the kmask unpack of src/ops/quant/mod.rs:237-258: out[0..8)=scales,
 * out[8..16)=mins */
void rmi_ref_unpack_scales_kmask(const uint8_t *scales12, uint8_t *out16);

/* src/ops/quant/mod.rs:210-289 (scalar) and :701-799 (AVX2). */
float rmi_ref_vec_dot_q4k_q8k(const uint8_t *q4k_row, size_t n_blocks,
                              const float *d, const int8_t *qs,
                              const int16_t *bsums, int variant);

/* Exact integers per super-block of the same dot: isum[b] = sum_l aux32[l]
 * (scale-weighted q4*q8 products), msum[b] = sum_j bsums[j]*mins[j/2]. */
void rmi_ref_q4k_q8k_block_ints(const uint8_t *q4k_row, size_t n_blocks,
                                const int8_t *qs, const int16_t *bsums,
                                int32_t *isum, int32_t *msum);
void rmi_ref_q4k_q8k_block_ints_matrix(const uint8_t *q4k_weight, size_t n_out, size_t n_blocks, const int8_t *qs,
                                       const int16_t *bsums, int32_t *ints);

/* src/ops/quant/mod.rs:456-490, 492-508 */
void rmi_ref_dequantize_row_q4_k(const uint8_t *blocks, float *output,
                                 size_t n);

/* src/ops/kernel/q4_k.rs:56-93 — Q4_KKernel::forward_prepared over a Q8_K
 * activation; rows [ith*ceil(n_out/nth), ...) of the full output. */
void rmi_ref_q4k_forward_prepared(const uint8_t *weight, const float *d,
                                  const int8_t *qs, const int16_t *bsums,
                                  float *output, size_t n_in, size_t n_out,
                                  size_t ith, size_t nth, int variant);

/* src/ops/kernel/q4_k.rs:20-54 — Q4_KKernel::forward_prequantized: rebuild
 * f32 x from (q8, scales), dequantise each row, sequential f32 dot. */
void rmi_ref_q4k_forward_prequantized(const uint8_t *weight,
                                      const uint8_t *input_q8,
                                      const float *input_scales,
                                      float *output, size_t n_in,
                                      size_t n_out, size_t ith, size_t nth);

/* src/core/model.rs:65-85 — QuantizedLinear::forward_dequant: whole-weight
 * Q4_K dequant, then sequential f32 GEMV with the raw f32 input. */
void rmi_ref_quantized_linear_forward(const uint8_t *weight,
                                      const float *input, float *output,
                                      size_t in_features,
                                      size_t out_features);

/* ---- rmi_q4_0.c: Q4_0 x Q8_0 ----
 * Pinned by the closed forms of the reference's own tests (src/ops/kernel/q4_0/avx2.rs:243-330: all-zero,
 * all-max and all-min inputs against nibbles 0 and 15), integer dots by brute force, f64 dequantised dots, and
 * the intrinsics twin, which the reference requires to equal the scalar kernel bit for bit. */
/* src/ops/kernel/q4_0/scalar.rs:13-52 */
void rmi_ref_matmul_q4_0_scalar_range(const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
                                      float *output, size_t n_in, size_t n_out, size_t ith, size_t nth);
void rmi_ref_block_dots_q4_0(const uint8_t *weight, const uint8_t *input_q8, int32_t *dots, size_t n_in, size_t n_out);
/* src/ops/kernel/q4_0/avx2.rs:24-105, output pre-sliced (index 0 = row_start) */
void rmi_ref_x86_matmul_q4_0_range(const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
                                   float *output, size_t n_in, size_t row_start, size_t row_end);

/* ---- rmi_q6_k.c: Q6_K x Q8_K ----
 * Pinned by: the uniform-block value 256.0 (tests/quantized_inference.rs:252-263),
 * the element layout cross-checked between dequantize_row_q6_k and the aux8
 * unpack of the dot (two formulations inside the reference), brute-force
 * integer sums, and the intrinsics twin below (same instructions as the
 * reference's AVX2 kernel).  The exact f32 bits of the AVX2 kernel on random
 * data have no golden vector in the reference: parity unpinned beyond that. */
/* src/ops/quant/mod.rs:530-569 */
void rmi_ref_dequantize_row_q6_k(const uint8_t *blocks, float *output, size_t n);
/* src/ops/quant/mod.rs:640-692 (scalar) and :964-1062 (AVX2 order) */
float rmi_ref_vec_dot_q6k_q8k(const uint8_t *q6k_row, size_t n_blocks, const float *d, const int8_t *qs,
                              const int16_t *bsums, int variant);
/* isum[b] = sum over the super-block of scale * q8 * (q6 - 32) */
void rmi_ref_q6k_q8k_block_ints(const uint8_t *q6k_row, size_t n_blocks, const int8_t *qs, int32_t *isum);
/* the eight int32 lanes the AVX2 kernel converts to f32, per super-block: lanes[b*8 + m] */
void rmi_ref_q6k_q8k_lane_ints(const uint8_t *q6k_row, size_t n_blocks, const int8_t *qs, const int16_t *bsums,
                               int32_t *lanes);
/* src/ops/kernel/q6_k.rs:44-80 */
void rmi_ref_q6k_forward_prepared(const uint8_t *weight, const float *d, const int8_t *qs, const int16_t *bsums,
                                  float *output, size_t n_in, size_t n_out, size_t ith, size_t nth, int variant);
/* src/ops/kernel/q6_k.rs:83-119 */
void rmi_ref_q6k_forward_prequantized(const uint8_t *weight, const uint8_t *input_q8, const float *input_scales,
                                      float *output, size_t n_in, size_t n_out, size_t ith, size_t nth);
/* the reference's intrinsics, src/ops/quant/mod.rs:964-1062 */
float rmi_ref_x86_vec_dot_q6k_q8k(const uint8_t *q6k_row, size_t n_blocks, const float *d, const int8_t *qs,
                                  const int16_t *bsums);
void rmi_ref_x86_q6k_forward_prepared(const uint8_t *weight, const float *d, const int8_t *qs, const int16_t *bsums,
                                      float *output, size_t n_in, size_t n_out, size_t ith, size_t nth);

/* ---- rmi_oracle_avx2.c: the same AVX2 kernels written with the same
 * intrinsics the reference uses; bit-identical to the RMI_REF_AVX2 variants
 * above on any AVX2+FMA host.  Used to cross-check the order emulation and
 * as the timed CPU baseline. ---- */
int rmi_ref_have_avx2(void);
void rmi_ref_x86_quantize_q8_0(const float *input, size_t n, uint8_t *q8,
                               float *scales);
void rmi_ref_x86_matmul_q8_0_range(const uint8_t *weight,
                                   const uint8_t *input_q8,
                                   const float *input_scales, float *output,
                                   size_t n_in, size_t row_start,
                                   size_t row_end);
float rmi_ref_x86_vec_dot_q4k_q8k(const uint8_t *q4k_row, size_t n_blocks,
                                  const float *d, const int8_t *qs,
                                  const int16_t *bsums);
void rmi_ref_x86_quantize_row_q8_k(const float *x, size_t n, float *d,
                                   int8_t *qs, int16_t *bsums);

/* Threaded baseline: the (ith,nth) row partition of parallel.rs:124-138 over
 * persistent threads with a spin barrier per matmul (the shape of
 * ComputePool::compute, src/core/thread_pool.rs:119-161). */
typedef struct rmi_ref_pool rmi_ref_pool;
rmi_ref_pool *rmi_ref_pool_create(int n_threads);
void rmi_ref_pool_destroy(rmi_ref_pool *pool);
int rmi_ref_pool_threads(const rmi_ref_pool *pool);
/* y[t] = W x[t] for t < n_tokens, AVX2 kernels, rows split over the pool. */
void rmi_ref_pool_matmul_q8_0(rmi_ref_pool *pool, const uint8_t *weight,
                              const uint8_t *input_q8,
                              const float *input_scales, float *output,
                              size_t n_in, size_t n_out, size_t n_tokens);
void rmi_ref_pool_matmul_q4k_q8k(rmi_ref_pool *pool, const uint8_t *weight,
                                 const float *d, const int8_t *qs,
                                 const int16_t *bsums, float *output,
                                 size_t n_in, size_t n_out);

/* generic job on the pool: fn(arg, ith, nth) on every thread, then a barrier */
void rmi_ref_pool_matmul_q4_0(rmi_ref_pool *pool, const uint8_t *weight, const uint8_t *input_q8,
                              const float *input_scales, float *output, size_t n_in, size_t n_out);
void rmi_ref_pool_matmul_q6k_q8k(rmi_ref_pool *pool, const uint8_t *weight, const float *d, const int8_t *qs,
                                 const int16_t *bsums, float *output, size_t n_in, size_t n_out);
void rmi_ref_pool_run(rmi_ref_pool *pool, void (*fn)(void *arg, int ith, int nth), void *arg);

/* ---- rmi_qwen3.c: Qwen3Session::generate_inner (src/models/qwen3.rs:581-1158)
 * restated for an all-Q8_0 model with F16 KV cache, NeoX RoPE, greedy sampling.
 * Every quantized matmul goes through `matmul`, whose signature is that of
 * Kernel::forward_prequantized with the weight as an opaque first argument, so
 * the same loop runs on the restated CPU kernels or on any back end that is
 * handed in from outside. ---- */
typedef int (*rmi_ref_matmul_fn)(const void *weight, const uint8_t *input_q8, const float *input_scales,
                                 float *output, uint32_t n_in, uint32_t n_out, uint32_t ith, uint32_t nth);

typedef struct {
    uint32_t n_embd, n_layer, n_head, n_head_kv, head_dim_k, head_dim_v, n_ff, vocab, n_ctx;
    float eps, freq_base;
    int32_t has_qk_norm;
    int32_t quant_variant;        /* RMI_REF_SCALAR / RMI_REF_AVX2 activation quantizer */
    const uint8_t *token_embd;    /* raw Q8_0 rows, for embedding_lookup_q8_0 */
    const float *output_norm;
    const void *output;           /* matmul weight of the (tied) lm_head */
    const float *const *attn_norm, *const *ffn_norm, *const *q_norm, *const *k_norm; /* [n_layer] */
    const void *const *wq, *const *wk, *const *wv, *const *wo, *const *w_gate, *const *w_up, *const *w_down;
} rmi_ref_qwen3_model;

/* the elementwise pieces of the loop, for per-kernel parity tests */
void rmi_ref_rms_norm(const float *input, const float *weight, float *output, size_t n, float eps);
void rmi_ref_rope_neox(float *x, size_t pos, size_t head_dim, float freq_base);
void rmi_ref_rope_angles(size_t pos, size_t head_dim, float freq_base, float *cos_out, float *sin_out);
void rmi_ref_silu_mul(const float *gate_out, float *up_out, size_t n);
/* src/ops/attention.rs:28-38 (the x86-64, non-parity-trace branch: f32 sum, one division per element) */
void rmi_ref_softmax(float *x, size_t n);
/* src/ops/dot.rs:99-119 (f64 sum of f32 products) */
float rmi_ref_dot_f16(const uint16_t *a, const uint16_t *b, size_t n);
/* src/ops/embedding.rs:12-22 */
void rmi_ref_embedding_lookup_q8_0(const uint8_t *weight, uint32_t token_id, size_t n_embd, float *out);
/* src/models/qwen3.rs:172-191: 0 and the first strict maximum, or -1 for empty or non-finite logits */
int rmi_ref_greedy_token(const float *logits, size_t n, uint32_t *token_id);
void rmi_ref_attention_f16(const float *q, const uint16_t *k_cache, const uint16_t *v_cache, size_t step,
                           size_t kv_stride, size_t n_head, size_t n_head_kv, size_t hk, size_t hv, float *attn_out);

/* weight argument for rmi_ref_cpu_matmul */
typedef struct {
    const uint8_t *blocks;
    rmi_ref_pool *pool;
} rmi_ref_cpu_weight;
int rmi_ref_cpu_matmul(const void *weight, const uint8_t *input_q8, const float *input_scales, float *output,
                       uint32_t n_in, uint32_t n_out, uint32_t ith, uint32_t nth);

/* Runs n_prompt + max_new - 1 decoder steps (one token per step, prompt
 * included).  Per step: FNV-1a hash of the logits' bytes, argmax, the two
 * largest logits; full logits of the steps listed in dump_steps.  Returns the
 * number of generated tokens, or -1 on error (non-finite logits, capacity). */
int rmi_ref_qwen3_generate(const rmi_ref_qwen3_model *model, rmi_ref_matmul_fn matmul, rmi_ref_pool *pool,
                           const uint32_t *prompt, uint32_t n_prompt, uint32_t max_new, uint32_t *generated,
                           uint64_t *step_hash, uint32_t *step_argmax, float *step_top2,
                           const uint32_t *dump_steps, uint32_t n_dump, float *dump_logits,
                           double *seconds_total, double *seconds_matmul);

#ifdef __cplusplus
}
#endif
#endif /* RMI_ORACLE_H */
