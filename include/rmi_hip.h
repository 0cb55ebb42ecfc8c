/*
 * rmi_hip.h — C ABI of the MI355X (gfx950) back end for rust-model-inference's
 * quantized-weight matrix products.
 *
 * This is what the crate's `hip` op back end binds over FFI.  Every entry
 * point names the reference interface it stands in for (paths relative to the
 * reference repository).  Conventions:
 *   - plain pointers and sizes only; weights live behind opaque handles;
 *   - functions returning int give 0 on success and a negative RMI_HIP_E_*
 *     code on failure, never abort or throw; rmi_hip_last_error() returns the
 *     message of the calling thread's last failure;
 *   - "host" entry points take caller-owned host slices that are valid only
 *     for the call (the `&[u8]` / `&mut [f32]` of the Kernel trait);
 *     "_dev" entry points take device pointers and a hipStream_t (as void*),
 *     enqueue work and return without synchronising;
 *   - re-entrant: the Kernel trait is Send + Sync and is called concurrently
 *     by all pool threads; every host thread gets its own stream and staging.
 *
 * f32 results of the Q8_0 GEMV and the Q4_K x Q8_K GEMV reproduce the
 * accumulation order of the reference's x86-64 production kernels
 * (avx2.rs:71-173, quant/mod.rs:701-799) bit for bit; the MFMA GEMM
 * reproduces the fused sequential order of neon.rs:49-73.
 */
#ifndef RMI_HIP_H
#define RMI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RMI_HIP_OK 0
#define RMI_HIP_E_INVALID (-1)   /* bad argument / shape mismatch            */
#define RMI_HIP_E_RUNTIME (-2)   /* HIP runtime error (message has details)  */
#define RMI_HIP_E_NOT_INIT (-3)  /* rmi_hip_init has not succeeded           */
#define RMI_HIP_E_NO_DEVICE (-4) /* no gfx950 device visible                 */

#define RMI_HIP_DTYPE_Q4_0 2
#define RMI_HIP_DTYPE_Q8_0 8
#define RMI_HIP_DTYPE_Q4_K 12
#define RMI_HIP_DTYPE_Q6_K 14

/* Activation rounding of quantize_q8_0_into: the reference picks it per host
 * architecture (src/ops/quant/q8_0.rs:3-24). */
#define RMI_HIP_ROUND_HALF_AWAY 0 /* scalar path, :49-71: 1/d, round()        */
#define RMI_HIP_ROUND_TIES_EVEN 1 /* AVX2 path, :176-230: 127/amax, rint()    */
#define RMI_HIP_ROUND_NEON 2      /* NEON path, :75-164: 1/d, nearest-even, clamped to [-127, 127] */

typedef struct rmi_hip_weight rmi_hip_weight;

/* ---- context: replaces the lazy OnceLock GPU context of src/ops/float.rs:44-58.
 * A failing init is the "fall back to CPU" signal of float.rs:51-57. */
int rmi_hip_init(int device);
void rmi_hip_shutdown(void);
const char *rmi_hip_last_error(void);
/* Diagnostic, no counterpart in the reference: how many per-thread contexts (a stream plus staging buffers) the
 * library holds.  A thread that exits hands its context to the next new thread, so this is the largest number
 * of threads that were inside the library at once, not the number of threads ever seen. */
size_t rmi_hip_thread_context_count(void);
/* name/arch of the bound device, compute units, bytes of HBM */
int rmi_hip_device_info(char *name, size_t name_len, int *compute_units, size_t *hbm_bytes);

/* ---- weights: replace the borrowed `&[u8]` of QuantizedTensor::from_bytes /
 * Q8Kernel::new / Q4_KKernel::new (src/ops/kernel/quantized_tensor.rs:120-138,
 * q8_0/mod.rs:21-31, q4_k.rs:13-17).  The bytes are copied to HBM and repacked
 * once; the host slice may be dropped afterwards.  NULL on failure. */
rmi_hip_weight *rmi_hip_upload_q8_0(const uint8_t *blocks, size_t nbytes, uint32_t n_in, uint32_t n_out);
rmi_hip_weight *rmi_hip_upload_q4_k(const uint8_t *blocks, size_t nbytes, uint32_t n_in, uint32_t n_out);
/* Q4_0Kernel::new (src/ops/kernel/q4_0/mod.rs:26-28): rows of 18-byte blocks. */
rmi_hip_weight *rmi_hip_upload_q4_0(const uint8_t *blocks, size_t nbytes, uint32_t n_in, uint32_t n_out);
/* Q6_KKernel::new (src/ops/kernel/q6_k.rs:15-18): rows of 210-byte super-blocks. */
rmi_hip_weight *rmi_hip_upload_q6_k(const uint8_t *blocks, size_t nbytes, uint32_t n_in, uint32_t n_out);
/* QTensorOwned::fuse_vstack (src/ops/kernel/qtensor_owned.rs:138-164) and
 * fuse_vstack_q8_0 / _q4_k (src/ops/quant/fuse.rs:25-64): rows of a then rows
 * of b.  NULL (the reference's None) when dtype or n_in differ. */
rmi_hip_weight *rmi_hip_fuse_vstack(const rmi_hip_weight *a, const rmi_hip_weight *b);
void rmi_hip_free_weight(rmi_hip_weight *w);
uint32_t rmi_hip_weight_n_in(const rmi_hip_weight *w);
uint32_t rmi_hip_weight_n_out(const rmi_hip_weight *w);
int rmi_hip_weight_dtype(const rmi_hip_weight *w);
/* bytes this weight occupies in HBM after repacking */
size_t rmi_hip_weight_device_bytes(const rmi_hip_weight *w);
/* device address of that repacked tile stream (read-only for callers; valid until rmi_hip_free_weight) */
const void *rmi_hip_weight_device_data(const rmi_hip_weight *w);

/* ---- Q8_0, host slices ---------------------------------------------------*/

/* Kernel::forward_prequantized for Q8Kernel (src/ops/kernel/q8_0/mod.rs:33-55)
 * = matmul_q8_0_quantized_parallel_rows (q8_0/parallel.rs:102-139): `output`
 * is the FULL n_out-long slice; only rows of partition (ith, nth) are written.
 * Activation quants of -128: the integer dot is exact (the scalar kernel, scalar.rs:49-53).  The reference's
 * AVX2 kernel negates the activation byte where the weight is negative, which wraps -(-128), and saturates pair
 * sums to i16 (avx2.rs:128-147): it is wrong wherever a -128 activation quant meets a negative weight, and
 * this library does not follow it there.  No quantizer of the reference emits -128 from finite input. */
int rmi_hip_q8_0_forward_prequantized(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                      float *output, uint32_t n_in, uint32_t n_out, uint32_t ith, uint32_t nth);
/* matmul_q8_0_quantized_range (q8_0/dispatch.rs:27-108), the slot the Vulkan
 * hook occupies (:36-52): `output` is PRE-SLICED, output[0] = row_start. */
int rmi_hip_matmul_q8_0_quantized_range(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                        float *output, uint32_t n_in, uint32_t row_start, uint32_t row_end);
/* n_tokens prequantized activations in one call: input_q8[n_tokens][n_in],
 * input_scales[n_tokens][n_in/32], output[n_tokens][n_out] token-major
 * (the layout of Kernel::forward_batched, trait_.rs:78-109). */
int rmi_hip_matmul_q8_0_quantized_batch(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                        float *output, uint32_t n_in, uint32_t n_out, uint32_t n_tokens);
/* How rmi_hip_q8_0_forward_batched and rmi_hip_q4_k_forward_batched multiply a batch (process-wide; a caller that
 * implements Kernel::forward_batched, src/ops/kernel/trait_.rs:78-109, on those two entry points chooses once at
 * start-up instead of at every call site):
 *   X86_ORDER (default)  every token through the GEMV in the x86-64 kernels' accumulation order: the bits of an
 *                        x86-64 host for any token count, and the whole weight is read once per 8 tokens;
 *   AARCH64_ORDER        Q8_0: the aarch64 kernel's order on the matrix cores (what the *_neon entry computes), bit
 *                        for bit an aarch64 host; Q4_K: as FAST (its CPU kernels have one order);
 *   FAST                 the fastest kernel per product, every output within 1e-4 + 1e-4 |ref| of the CPU kernels
 *                        and built from exact integer block dots: up to 8 tokens the GEMV, then the small-batch
 *                        kernel and rmi_hip_gemm_q8_0_fast_dev / the Q4_K GEMM. */
#define RMI_HIP_BATCHED_X86_ORDER 0
#define RMI_HIP_BATCHED_AARCH64_ORDER 1
#define RMI_HIP_BATCHED_FAST 2
int rmi_hip_set_forward_batched_mode(int mode);
int rmi_hip_get_forward_batched_mode(void);
/* Kernel::forward / forward_batched with f32 input (trait_.rs:59-109):
 * quantize each token row on the device (rounding as given), then the GEMV in
 * the x86-64 kernel's order for every token, eight tokens a launch.  As in the
 * reference, a token's result does not depend on the batch it arrives in:
 * forward_batched(x)[t] == forward(x[t]) bit for bit. */
int rmi_hip_q8_0_forward_batched(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                 uint32_t n_out, uint32_t n_tokens, int rounding);
/* The same call on the matrix cores, in the aarch64 kernel's accumulation order (neon.rs:49-73) for every
 * token count: the small-batch kernel up to 16 tokens (32 for very tall matrices), the tiled int8-MFMA GEMM
 * beyond.  Batch-independent in the same sense; with RMI_HIP_ROUND_NEON it is what an aarch64 host computes
 * end to end.  Differs from the call above in the last bits only (within 1e-4 + 1e-4 |ref|); prefill-sized
 * batches run one to two orders of magnitude faster here. */
int rmi_hip_q8_0_forward_batched_neon(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                      uint32_t n_out, uint32_t n_tokens, int rounding);
/* quantize_q8_0_into (src/ops/quant/q8_0.rs:3-24) run on the device. */
int rmi_hip_quantize_q8_0(const float *input, uint32_t n, uint8_t *q8, float *scales, int rounding);
/* The per-block int32 dots of scalar.rs:49-53, dots[n_out][n_in/32], computed
 * from the repacked HBM copy (debug / parity entry point). */
int rmi_hip_block_dots_q8_0(const rmi_hip_weight *w, const uint8_t *input_q8, int32_t *dots);
/* ops::matmul_q8_0 (q8_0/parallel.rs:317-341): f32 activations used as they
 * are, no activation quantisation. */
int rmi_hip_matmul_q8_0_f32(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in, uint32_t n_out);
/* matmul_q8_0_fallback_range (src/ops/kernel/q8_0/scalar.rs:3-29), the same product on hosts without AVX2: per
 * row one f32 chain, local += float(q)*x over the 32 elements of a block in order, sum += d*local block after
 * block.  output has row_end - row_start entries.  Differs from the AVX2 order in the last bits only. */
int rmi_hip_matmul_q8_0_fallback_range(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                       uint32_t row_start, uint32_t row_end);

/* ---- Q4_K, host slices ---------------------------------------------------*/

/* Q4_KKernel::forward_prepared (src/ops/kernel/q4_k.rs:56-93) with the Q8_K
 * activation passed as three arrays (BlockQ8K has no repr(C),
 * src/ops/quant/mod.rs:35-40): d[n_in/256], qs[n_in], bsums[n_in/16]. */
int rmi_hip_q4_k_forward_prepared(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                                  const int16_t *q8k_bsums, float *output, uint32_t n_in, uint32_t n_out, uint32_t ith,
                                  uint32_t nth);
/* Same with f32 input: quantize_row_q8_k on the device (quant/mod.rs:140-200),
 * the `q8_k == None` branch of q4_k.rs:77-84; n_tokens rows, token-major out, every token through the GEMV in
 * the x86-64 kernel's order (forward_batched(x)[t] == forward(x[t]) bit for bit, trait_.rs:78-109). */
int rmi_hip_q4_k_forward_batched(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                 uint32_t n_out, uint32_t n_tokens);
/* The same call with prefill-sized batches (16 tokens and more) on the int8 matrix cores: exact integers, the
 * f32 sum of an output as one chain over the super-blocks instead of the AVX2 kernel's 8 + 4 lane chains, so
 * results agree with the call above within 1e-4 + 1e-4 |ref|, not bit for bit. */
int rmi_hip_q4_k_forward_batched_mfma(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                      uint32_t n_out, uint32_t n_tokens);
/* quantize_row_q8_k (quant/mod.rs:42-59) run on the device. */
int rmi_hip_quantize_row_q8_k(const float *input, uint32_t n, float *d, int8_t *qs, int16_t *bsums);
/* Q4_KKernel::forward_prequantized (q4_k.rs:20-54): dequantise-and-dot with
 * the Q8_0 activation turned back into f32. */
int rmi_hip_q4_k_forward_prequantized(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                      float *output, uint32_t n_in, uint32_t n_out, uint32_t ith, uint32_t nth);
/* QuantizedLinear::forward / forward_dequant (src/core/model.rs:65-91): f32
 * input, Q4_K weight dequantised in registers, no scratch needed. */
int rmi_hip_quantized_linear_forward(const rmi_hip_weight *w, const float *input, float *output, uint32_t in_features,
                                     uint32_t out_features);
/* The same on device pointers (x f32[in_features], y f32[out_features]); does not synchronise. */
int rmi_hip_quantized_linear_forward_dev(const rmi_hip_weight *w, const float *x, float *y, void *stream);
/* Exact integers of the Q4_K x Q8_K dot per super-block (parity entry point):
 * isum/msum[n_out][n_in/256] as in vec_dot_q4k_q8k_scalar, quant/mod.rs:260-284. */
int rmi_hip_block_ints_q4_k(const rmi_hip_weight *w, const int8_t *q8k_qs, const int16_t *q8k_bsums, int32_t *isum,
                            int32_t *msum);

/* ---- Q4_0, host slices ---------------------------------------------------*/

/* Q4_0Kernel::forward_prequantized (src/ops/kernel/q4_0/mod.rs:33-84): rows
 * [ith*ceil(n_out/nth), ...) of the full output; the scalar kernel's arithmetic
 * (q4_0/scalar.rs:13-52), which the AVX2 one (q4_0/avx2.rs:24-105) equals bit for bit. */
int rmi_hip_q4_0_forward_prequantized(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                      float *output, uint32_t n_in, uint32_t n_out, uint32_t ith, uint32_t nth);
/* Kernel::forward / forward_batched on a Q4_0 kernel (src/ops/kernel/trait_.rs:59-109): quantize_q8_0_into on
 * the device, then the product; n_tokens rows, token-major out. */
int rmi_hip_q4_0_forward_batched(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                 uint32_t n_out, uint32_t n_tokens, int rounding);
/* Exact per-block integers (parity entry point): dots[n_out][n_in/32] = sum of (nibble - 8) * q8
 * (q4_0/scalar.rs:40-47). */
int rmi_hip_block_dots_q4_0(const rmi_hip_weight *w, const uint8_t *input_q8, int32_t *dots);

/* ---- Q6_K, host slices ---------------------------------------------------*/

/* Q6_KKernel::forward_prepared (src/ops/kernel/q6_k.rs:44-80): vec_dot_q6k_q8k
 * (src/ops/quant/mod.rs:938-944, AVX2 kernel :964-1062) per row, Q8_K activation
 * as three arrays. */
int rmi_hip_q6_k_forward_prepared(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                                  const int16_t *q8k_bsums, float *output, uint32_t n_in, uint32_t n_out, uint32_t ith,
                                  uint32_t nth);
/* Same with f32 input (the `q8_k == None` branch, q6_k.rs:63-69): quantize_row_q8_k
 * on the device; n_tokens rows, token-major out (Kernel::forward_batched,
 * src/ops/kernel/trait_.rs:78-109). */
int rmi_hip_q6_k_forward_batched(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                 uint32_t n_out, uint32_t n_tokens);
/* Q6_KKernel::forward_prequantized = matmul_q6_k_scalar_range (q6_k.rs:83-119):
 * dequantise-and-dot with the Q8_0 activation turned back into f32. */
int rmi_hip_q6_k_forward_prequantized(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                      float *output, uint32_t n_in, uint32_t n_out, uint32_t ith, uint32_t nth);
/* Exact integers of the Q6_K x Q8_K dot (parity entry point): lanes[n_out][n_in/256][8],
 * the eight int32 the AVX2 kernel converts to f32 per super-block (quant/mod.rs:1053-1055);
 * their sum is the scalar kernel's sum of aux32 (:676-688). */
int rmi_hip_block_lanes_q6_k(const rmi_hip_weight *w, const int8_t *q8k_qs, const int16_t *q8k_bsums,
                             int32_t *lanes);

/* ---- device-resident entry points (activations stay in HBM) ---------------
 * Device pointers: activation quants (x_q8, q8k_qs) 16-byte aligned; scales, d, bsums and outputs 4-byte
 * aligned (what rmi_hip_malloc returns is aligned for all of them).  Anything else is RMI_HIP_E_INVALID. */

void *rmi_hip_malloc(size_t nbytes);
void rmi_hip_free(void *dptr);
int rmi_hip_memcpy_h2d(void *dst, const void *src, size_t nbytes);
int rmi_hip_memcpy_d2h(void *dst, const void *src, size_t nbytes);
int rmi_hip_synchronize(void);

/* Kernel::forward / forward_batched of a Q8_0 weight on device pointers WITHOUT any allocation: x f32
 * [n_tokens][n_in] is quantized (rounding as given) and multiplied as rmi_hip_q8_0_forward_batched does, bit for
 * bit, into y[t * y_stride + row].  No counterpart in the reference: it exists for callers that cannot allocate
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The quantized
 * activation lives in a fixed 288 KiB array inside the library's code object, one copy per GPU, held until the
 * process ends: n_tokens * n_in may not exceed RMI_HIP_NOALLOC_MAX_ELEMS (RMI_HIP_E_INVALID beyond), and calls
 * that overlap on one GPU (two streams, two threads) race on it -- order them on one stream.  The calling
 * thread's current device must be the one given to rmi_hip_init.  Calls no hipMalloc / hipFree, creates no
 * stream, does not synchronise. */
#define RMI_HIP_NOALLOC_MAX_ELEMS 262144
int rmi_hip_q8_0_forward_noalloc_dev(const rmi_hip_weight *w, const float *x, float *y, uint32_t n_tokens,
                                     uint32_t y_stride, int rounding, void *stream);

/* Plain device-to-device streaming copy kernel (nbytes a multiple of 16).  No
 * counterpart in the reference: it is the known-size kernel against which
 * hardware HBM-traffic counters are calibrated when profiling. */
int rmi_hip_copy_dev(void *dst, const void *src, size_t nbytes, void *stream);

/* y[t][row] for rows [row_start,row_end) of n_tokens (1..8) activations.
 * y has row stride 1 and token stride y_stride floats; y[t][0] is row 0. */
int rmi_hip_gemv_q8_0_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                          uint32_t n_tokens, uint32_t y_stride, uint32_t row_start, uint32_t row_end, void *stream);
int rmi_hip_quantize_q8_0_dev(const float *x, int8_t *q8, float *scales, uint32_t n_tokens, uint32_t n_in,
                              int rounding, void *stream);
/* The same product for a small batch, 1..64 tokens whose activations fit the kernel's LDS staging
 * (n_in * 1.14 bytes a token, 159 KiB in all), in the accumulation order of the reference's NEON kernel:
 * sum = fma(float(dot_b), f32(w.d_b) * x_scale_b, sum) block after block (matmul_q8_0_vs_q8_0_neon,
 * src/ops/kernel/q8_0/neon.rs:49-73), bit for bit, through int8 MFMA with the weights streamed once.  The
 * AVX2-order call above converts eight partial sums per block and is bound by the vector ALU from four tokens
 * on; this one stays bound by HBM.  Results of the two orders differ in the last bits only. */
int rmi_hip_gemv_q8_0_neon_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                               uint32_t n_tokens, uint32_t y_stride, uint32_t row_start, uint32_t row_end, void *stream);
/* Y[t][:] = W . Q8_0(X[t][:]) for n_tokens >= 1 through int8 MFMA. */
int rmi_hip_gemm_q8_0_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                          uint32_t n_tokens, uint32_t y_stride, void *stream);
/* The same product for few tokens, for callers that ask for the reference's tolerance rather than one host's bits
 * (Kernel::forward_batched, src/ops/kernel/trait_.rs:78-109: every token is an independent GEMV; outputs within
 * 1e-4 + 1e-4 |ref| of either CPU kernel).  rmi_hip_gemm_q8_0_dev keeps the aarch64 kernel's single f32 chain per
 * output, which leaves most of the chip idle below a few hundred tokens; here a workgroup is one 32 x 32 tile whose
 * waves split the blocks of a row into runs of rmi_hip_gemm_q8_0_ksplit_quads_per_part(n_in) quads (128 elements
 * each): every per-block int32 dot is exact, every run is added from zero in block order, the runs' sums are added
 * in run order.  Deterministic, the same for a token whatever batch it arrives in, not bit-identical to the single
 * chain.  No workspace, no allocation, no synchronisation. */
int rmi_hip_gemm_q8_0_ksplit_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                                 uint32_t n_tokens, uint32_t y_stride, void *stream);
uint32_t rmi_hip_gemm_q8_0_ksplit_quads_per_part(uint32_t n_in);
/* The prefill product for callers that ask for the reference's tolerance rather than one host's bits: the library
 * takes what it expects to be fastest for this product, the k-split kernel above (few tokens, long rows), the tiled
 * kernel of rmi_hip_gemm_q8_0_dev, or that kernel with two or four groups of waves per tile, group g of G taking the
 * quads g, g + G, ... of a row (a chain per group, the groups' sums added in group order), which puts every compute
 * unit to work on a product of a few hundred tokens.  Every output is built from exact integer block dots, deterministic,
 * and within 1e-4 + 1e-4 |ref| of the CPU kernels; which chain a token's result follows depends on the token count
 * of the call.  rmi_hip_gemm_q8_0_fast_plan says which one a call would take: RMI_HIP_GEMM_PLAN_* and, in *param,
 * the quads per run (k-split) or the number of interleaved groups (tiled). */
#define RMI_HIP_GEMM_PLAN_TILED_SINGLE_CHAIN 0
#define RMI_HIP_GEMM_PLAN_TILED_GROUPS 1
#define RMI_HIP_GEMM_PLAN_KSPLIT 2
int rmi_hip_gemm_q8_0_fast_plan(const rmi_hip_weight *w, uint32_t n_tokens, uint32_t *param);
int rmi_hip_gemm_q8_0_fast_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                               uint32_t n_tokens, uint32_t y_stride, void *stream);
int rmi_hip_gemv_q4_k_q8k_dev(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                              const int16_t *q8k_bsums, float *y, uint32_t n_tokens, uint32_t y_stride,
                              uint32_t row_start, uint32_t row_end, void *stream);
/* Y[t][:] = vec_dot_q4k_q8k(W, Q8_K(X[t][:])) for many tokens through int8 MFMA (Kernel::forward_batched,
 * src/ops/kernel/trait_.rs:78-109, on Q4_KKernel::forward_prepared, src/ops/kernel/q4_k.rs:56-93): exact
 * integers, the f32 sums within rounding of the CPU kernels. */
int rmi_hip_gemm_q4_k_q8k_dev(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                              const int16_t *q8k_bsums, float *y, uint32_t n_tokens, uint32_t y_stride, void *stream);
/* The integers of rmi_hip_gemm_q4_k_q8k_dev as they leave the matrix cores, per token, row and super-block:
 * ints[((t * n_out + n) * (n_in / 256) + sb) * 2 + 0] = sum_j scale_j * dot_j (the sum of the eight lane integers
 * of src/ops/quant/mod.rs:701-799), + 1 = sum_j min_j * bsum_j.  Same kernel, same tile width as the product takes
 * for this problem; writes no y (debug / parity entry point). */
int rmi_hip_gemm_block_ints_q4_k_dev(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                                     const int16_t *q8k_bsums, int32_t *ints, uint32_t n_tokens, void *stream);
/* Q4_0 weights, Q8_0 activations on the device (src/ops/kernel/q4_0/scalar.rs:13-52). */
int rmi_hip_gemv_q4_0_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                          uint32_t n_tokens, uint32_t y_stride, uint32_t row_start, uint32_t row_end, void *stream);
/* y[t*y_stride + r] = vec_dot_q6k_q8k(row r, Q8_K token t) for rows [row_start,row_end), 1..n tokens
 * (Q6_KKernel::forward_prepared, src/ops/kernel/q6_k.rs:44-80). */
int rmi_hip_gemv_q6_k_q8k_dev(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                              const int16_t *q8k_bsums, float *y, uint32_t n_tokens, uint32_t y_stride,
                              uint32_t row_start, uint32_t row_end, void *stream);
int rmi_hip_quantize_row_q8_k_dev(const float *x, float *d, int8_t *qs, int16_t *bsums, uint32_t n_tokens,
                                  uint32_t n_in, void *stream);

/* A fixed list of independent Q8_0 GEMVs (a token-step's projection set, or
 * the q/k/v and gate/up pairs that share an input) run as ONE launch.  The
 * reference issues them one after another inside one pool.compute closure
 * (src/models/qwen3.rs:738-774, 991-1019).  The weights are all Q8_0 or all
 * Q4_0 (src/ops/kernel/q4_0/mod.rs:33-84 per problem); both take Q8_0
 * activations. */
typedef struct rmi_hip_gemv_group rmi_hip_gemv_group;
rmi_hip_gemv_group *rmi_hip_gemv_group_create(uint32_t n_problems, const rmi_hip_weight *const *weights,
                                              const int8_t *const *x_q8, const float *const *x_scales,
                                              float *const *y, uint32_t n_tokens);
/* The same list (Q8_0 weights only) for 1..64 tokens through rmi_hip_gemv_q8_0_neon_dev's kernel. */
rmi_hip_gemv_group *rmi_hip_gemv_group_create_neon(uint32_t n_problems, const rmi_hip_weight *const *weights,
                                                   const int8_t *const *x_q8, const float *const *x_scales,
                                                   float *const *y, uint32_t n_tokens);
/* The same for Q4_K weights with Q8_K activations (three arrays per problem). */
rmi_hip_gemv_group *rmi_hip_gemv_group_create_q4_k(uint32_t n_problems, const rmi_hip_weight *const *weights,
                                                   const float *const *q8k_d, const int8_t *const *q8k_qs,
                                                   const int16_t *const *q8k_bsums, float *const *y,
                                                   uint32_t n_tokens);
/* And for Q6_K weights (src/ops/kernel/q6_k.rs:44-80 per problem). */
rmi_hip_gemv_group *rmi_hip_gemv_group_create_q6_k(uint32_t n_problems, const rmi_hip_weight *const *weights,
                                                   const float *const *q8k_d, const int8_t *const *q8k_qs,
                                                   const int16_t *const *q8k_bsums, float *const *y,
                                                   uint32_t n_tokens);
void rmi_hip_gemv_group_destroy(rmi_hip_gemv_group *g);
int rmi_hip_gemv_group_run_dev(const rmi_hip_gemv_group *g, void *stream);
/* Launch shape of a group, for profiling tools: workgroups per launch and waves per workgroup. */
int rmi_hip_gemv_group_shape(const rmi_hip_gemv_group *g, uint32_t *n_workgroups, uint32_t *waves_per_workgroup);

/* ---------------------------------------------------------------------------
 * Device-resident decode: Qwen3Session::generate_inner (src/models/qwen3.rs:581-1158)
 * with every tensor in HBM between two token ids.  Embedding lookup
 * (src/ops/embedding.rs:12-22), RMS norms (src/ops/norm.rs:3-19), the
 * activation quantizer, NeoX RoPE (src/ops/rope.rs:21-37), attention over the
 * F16 KV cache (qwen3.rs:876-933), SiLU (src/ops/activation/mod.rs:137-151) and
 * greedy_token (qwen3.rs:172-191) run as kernels around the Q8_0 GEMVs.  All
 * 2-D weights are Q8_0 blocks as in the GGUF file (dims [n_in, n_out],
 * qwen3.rs:1297-1311); `output` NULL ties the head to token_embd (qwen3.rs:283-287).
 * ------------------------------------------------------------------------- */
typedef struct rmi_hip_qwen3 rmi_hip_qwen3;

/* y[i] = exp(x[i]) as the decode kernels compute it: the bits of the platform libm's expf, which the
 * reference's f32::exp resolves to (softmax src/ops/attention.rs:28-38, SiLU src/ops/activation/mod.rs:137-151).
 * Device pointers; for parity tests of that function. */
int rmi_hip_expf_dev(const float *x, float *y, size_t n, void *stream);

typedef struct {
    uint32_t n_embd, n_layer, n_head, n_head_kv, head_dim_k, head_dim_v, n_ff, vocab;
    uint32_t capacity; /* positions the KV cache holds (prompt + generated); about 12 900 at most: one head's
                        * scores and weights of all positions stay in a workgroup's LDS */
    float eps, freq_base;
    int32_t has_qk_norm;
    int32_t rounding; /* RMI_HIP_ROUND_* of the activation quantizer */
} rmi_hip_qwen3_config;

typedef struct {
    const uint8_t *token_embd; /* Q8_0 [vocab][n_embd] */
    const uint8_t *output;     /* Q8_0 [vocab][n_embd] or NULL */
    const float *output_norm;  /* [n_embd] */
    /* per layer, [n_layer] pointers each */
    const float *const *attn_norm, *const *ffn_norm, *const *q_norm, *const *k_norm;
    const uint8_t *const *wq, *const *wk, *const *wv, *const *wo, *const *w_gate, *const *w_up, *const *w_down;
} rmi_hip_qwen3_weights;

/* The kernels of one step, on device pointers (what a host that keeps its own loop would call between
 * the GEMVs).  None synchronises.
 * x += residual (when not NULL), then rms_norm(x, weight) (src/ops/norm.rs:3-19) quantized as
 * quantize_q8_0_into does (src/ops/quant/q8_0.rs); x keeps the sum.  n % 32 == 0. */
int rmi_hip_rms_norm_quantize_q8_0_dev(float *x, const float *residual, const float *weight, uint32_t n, float eps,
                                       int8_t *q8, float *scales, int rounding, void *stream);
/* The same three steps and the Q8_0 product that follows them in one launch: y = W . Q8_0(rms_norm(x_in +
 * residual) * norm_weight), x_out = x_in + residual (src/models/qwen3.rs:719-774 and :1016-1019: norm,
 * quantize_q8_0_into, then the q/k/v or the gate/up matmul).  One token; n_in a multiple of 256 up to 2048 and
 * at most 32768 rows, else RMI_HIP_E_INVALID (use the separate calls).  x_out must not alias x_in. */
int rmi_hip_rms_norm_gemv_q8_0_dev(const rmi_hip_weight *w, const float *x_in, const float *residual,
                                   const float *norm_weight, float eps, int rounding, float *x_out, float *y,
                                   void *stream);
/* The attention block's first half in one launch (src/models/qwen3.rs:719-874), head dimension 128: norm as
 * above, the q, k and v products of the stacked weight [W_q ; W_k ; W_v], then what
 * rmi_hip_qk_norm_rope_f16_dev does to the three vectors.  n_in a multiple of 256 up to 1024. */
int rmi_hip_rms_norm_qkv_rope_q8_0_dev(const rmi_hip_weight *w_qkv, const float *x_in, const float *residual,
                                       const float *norm_weight, float eps, int rounding, float *x_out,
                                       const float *q_norm, const float *k_norm, const float *cos_row,
                                       const float *sin_row, uint16_t *q16, uint16_t *k_row, uint16_t *v_row,
                                       uint32_t n_head, uint32_t n_head_kv, void *stream);
/* The FFN's first half in one launch (src/models/qwen3.rs:1016-1027): norm as above, the gate and up products
 * of the stacked weight [W_gate ; W_up] (rmi_hip_fuse_vstack), then h = up * silu(gate) quantized to Q8_0
 * (h_q8[n_ff], h_scales[n_ff/32]).  n_in a multiple of 256 up to 2048, n_ff a multiple of 32. */
int rmi_hip_rms_norm_ffn_gate_up_q8_0_dev(const rmi_hip_weight *w_gate_up, const float *x_in, const float *residual,
                                          const float *norm_weight, float eps, int rounding, float *x_out,
                                          int8_t *h_q8, float *h_scales, void *stream);
/* gate_up = [W_gate x ; W_up x] (2*n_ff): (W_up x) * silu(W_gate x), src/ops/activation/mod.rs:137-151
 * as called at src/models/qwen3.rs:1016-1027, quantized to Q8_0. */
int rmi_hip_silu_mul_quantize_q8_0_dev(const float *gate_up, uint32_t n_ff, int8_t *q8, float *scales, int rounding,
                                       void *stream);
/* qkv = [q ; k ; v] of one token: per-head RMS norm of q and k (NULL weights = none), rope_neox with the
 * cos/sin of the position (head_dim_k/2 each, src/ops/rope.rs:21-37), rounding to f16: q to q16, k and v to
 * their cache rows (src/models/qwen3.rs:826-875). */
int rmi_hip_qk_norm_rope_f16_dev(const float *qkv, const float *q_norm, const float *k_norm, const float *cos_row,
                                 const float *sin_row, uint16_t *q16, uint16_t *k_row, uint16_t *v_row, uint32_t n_head,
                                 uint32_t n_head_kv, uint32_t head_dim_k, uint32_t head_dim_v, float eps, void *stream);
/* Attention of one token over keys 0..n_keys-1 of an F16 cache [t][kv_stride] (src/models/qwen3.rs:876-933,
 * dot_f16 src/ops/dot.rs:99-119, softmax src/ops/attention.rs:28-38); the output leaves quantized to Q8_0.
 * Head dimension 128 and 1280 keys or more: a head's keys are spread over up to 16 workgroups in two launches
 * (scores; then weights and p.v, the parts meeting in the workgroup that arrives last).  The softmax sum is still
 * the reference's sequential f32 sum; results have the same bits as the one-workgroup-per-head kernel.  The
 * hand-over uses a scratch region of the calling host thread: calls of one host thread that overlap on different
 * streams would share it, and the thread synchronises its launches before it exits (the region goes back to the
 * library with the thread).  rmi_hip_attention_reserve(n_head, max_keys) makes the region ahead of time (it
 * synchronises the device, allocates and clears; no counterpart in the reference), after which no call of this
 * thread with at most that many heads and keys allocates or synchronises; without it the first call that needs
 * the region synchronises `stream` and allocates it.  Up to 16 384 keys (head dimension 128); otherwise what one
 * workgroup holds in LDS (12 bytes a key of 159 KiB). */
int rmi_hip_attention_reserve(uint32_t n_head, uint32_t max_keys);
int rmi_hip_attention_f16_quantize_q8_0_dev(const uint16_t *q16, const uint16_t *k_cache, const uint16_t *v_cache,
                                            uint32_t n_keys, uint32_t kv_stride, uint32_t n_head, uint32_t n_head_kv,
                                            uint32_t head_dim_k, uint32_t head_dim_v, int8_t *q8, float *scales,
                                            int rounding, void *stream);

/* The two calls above in one launch, for head dimension 128 and contexts of up to 3392 keys: qkv is the f32
 * [q ; k ; v] of the new token (position n_keys - 1); every head's workgroup norms and rotates its q and its
 * key/value head's k, rounds them and v to f16, uses them from on-chip memory and writes k and v to row
 * n_keys - 1 of the caches; keys 0..n_keys-2 are read from the caches (src/models/qwen3.rs:776-933).  Same bits
 * as the two calls.  It lets the q/k/v product in front be a plain GEMV over the whole chip. */
int rmi_hip_qkv_attention_f16_quantize_q8_0_dev(const float *qkv, const float *q_norm, const float *k_norm,
                                                const float *cos_row, const float *sin_row, uint16_t *k_cache,
                                                uint16_t *v_cache, uint32_t n_keys, uint32_t kv_stride, uint32_t n_head,
                                                uint32_t n_head_kv, float eps, int8_t *q8, float *scales, int rounding,
                                                void *stream);

/* Uploads and repacks the weights (host slices may be dropped afterwards), allocates the KV cache. */
rmi_hip_qwen3 *rmi_hip_qwen3_create(const rmi_hip_qwen3_config *cfg, const rmi_hip_qwen3_weights *weights);
void rmi_hip_qwen3_destroy(rmi_hip_qwen3 *s);
/* Token ids that end generation (the tokenizer's EOS id and "im_end", src/models/qwen3.rs:1123-1130); none by
 * default.  At most 16. */
int rmi_hip_qwen3_set_stop_ids(rmi_hip_qwen3 *s, const uint32_t *ids, uint32_t n_ids);
/* Prompt positions are known in advance, so rmi_hip_qwen3_generate takes them 128 to a pass while it can (head
 * dimension 128, contexts short of the split attention's 1280 keys): every product is one launch for all of them
 * (eight tokens to a workgroup, the x86-64 order's bits for each), the other kernels run once per position inside
 * one launch; each position's logits, argmax and cache rows are what the step-by-step run gives, bit for bit.
 * enabled = 1 (the default): 128 positions a pass; 0: every position its own step; n > 1: n positions a pass (at
 * most 128).  Measured on the 512-token prompt of a Qwen3-0.6B model: 0.73 ms a position step by step, 0.07 ms in
 * passes of 128. */
int rmi_hip_qwen3_set_prompt_passes(rmi_hip_qwen3 *s, int enabled);
/* Runs up to n_prompt + max_new - 1 steps, one token per step, positions 0.. (the prompt is fed token by
 * token as generate_inner does), greedy sampling (temperature 0, sample_token's argmax branch).  With stop
 * ids set the run ends at the first sampled stop id, which is not part of the result, as in generate_inner
 * (checked by the host every 32 generated steps, so up to 31 further steps may have run); without, all steps
 * are enqueued at once and synchronised once at the end.  Per step run the argmax and the two largest
 * logits; full logits of the steps listed in dump_steps.
 * Returns the number of generated tokens or a negative code (non-finite logits are an error). */
int rmi_hip_qwen3_generate(rmi_hip_qwen3 *s, const uint32_t *prompt, uint32_t n_prompt, uint32_t max_new,
                           uint32_t *generated, uint32_t *step_argmax, float *step_top2, const uint32_t *dump_steps,
                           uint32_t n_dump, float *dump_logits, double *seconds);

/* ------------------------------------------------------------------ GGUF file -> HBM
 * The reference maps the file and hands slices of the mapping to its layers (GGUFLoader::from_file,
 * src/core/loader.rs:211-320; TensorSource::tensor_data, :363-372).  Here the same mapping feeds the uploads:
 * tensor bytes go from the page cache through two pinned staging chunks to the device, where the repack kernel
 * writes the tile stream; no whole-tensor copy on the host, no intermediate device copy of a whole tensor.
 * Parsing accepts what from_mmap accepts (versions 2 and 3, every metadata and tensor type it knows) and
 * rejects what it rejects (truncation, unknown tags, nested arrays, a tensor past the end of the file), with
 * the reference's message in rmi_hip_last_error().  open/close and the metadata and tensor queries need no
 * device and no rmi_hip_init. */
typedef struct rmi_hip_gguf rmi_hip_gguf;
rmi_hip_gguf *rmi_hip_gguf_open(const char *path); /* NULL on error */
void rmi_hip_gguf_close(rmi_hip_gguf *g);          /* weights and sessions made from it stay valid */
uint32_t rmi_hip_gguf_version(const rmi_hip_gguf *g);
uint64_t rmi_hip_gguf_alignment(const rmi_hip_gguf *g);   /* general.alignment, default 32 */
uint64_t rmi_hip_gguf_data_offset(const rmi_hip_gguf *g); /* GGUFLoader::data_offset */
uint64_t rmi_hip_gguf_n_tensors(const rmi_hip_gguf *g);
uint64_t rmi_hip_gguf_n_kv(const rmi_hip_gguf *g);
const char *rmi_hip_gguf_kv_key(const rmi_hip_gguf *g, uint64_t index); /* NULL past the end */
/* Metadata (GGUFLoader::metadata + the MetaValue conversions, src/core/tensor.rs:146-187).  meta_type gives the
 * value tag (0 u8 .. 12 f64, 8 string, 9 array) or -1 when the key is absent; the getters return 1 and store
 * the value, or 0 when the key is absent or the conversion is one the reference refuses (to_u64: every
 * integer and float type, `as u64` semantics; to_f64: f32, f64 and the 32/64-bit integers). */
int rmi_hip_gguf_meta_type(const rmi_hip_gguf *g, const char *key);
int rmi_hip_gguf_meta_u64(const rmi_hip_gguf *g, const char *key, uint64_t *out);
int rmi_hip_gguf_meta_f64(const rmi_hip_gguf *g, const char *key, double *out);
int rmi_hip_gguf_meta_bool(const rmi_hip_gguf *g, const char *key, int *out);
/* to_string_val: length of the string or -1; up to cap - 1 bytes and a terminator are stored in buf */
int64_t rmi_hip_gguf_meta_str(const rmi_hip_gguf *g, const char *key, char *buf, size_t cap);
/* to_arr: element count (and element tag) or -1; element `index` of a numeric array through to_u64 */
int64_t rmi_hip_gguf_meta_array_len(const rmi_hip_gguf *g, const char *key, int *elem_type);
int rmi_hip_gguf_meta_array_u64(const rmi_hip_gguf *g, const char *key, uint64_t index, uint64_t *out);
/* Tensors (GGUFLoader::tensor_info / tensor_data).  find: index or -1.  dims are [columns, rows, ..]. */
int64_t rmi_hip_gguf_find_tensor(const rmi_hip_gguf *g, const char *name);
int rmi_hip_gguf_tensor_info(const rmi_hip_gguf *g, uint64_t index, const char **name, uint32_t *n_dims,
                             uint64_t *dims, uint32_t dims_cap, int *ggml_type, uint64_t *offset, uint64_t *nbytes);
const uint8_t *rmi_hip_gguf_tensor_data(const rmi_hip_gguf *g, uint64_t index); /* into the mapping */
/* A 2-D Q8_0, Q4_0, Q4K or Q6K tensor as a device weight (the same result as rmi_hip_upload_* on its bytes). */
rmi_hip_weight *rmi_hip_gguf_upload(const rmi_hip_gguf *g, const char *name);
/* Up to 16 tensors of one type and column count as one weight, rows one below the other ([q ; k ; v],
 * [gate ; up]): what rmi_hip_fuse_vstack gives, written in place. */
rmi_hip_weight *rmi_hip_gguf_upload_stack(const rmi_hip_gguf *g, const char *const *names, int n_names);
/* Qwen3Config::from_source (src/models/qwen3.rs:46-94, keys of src/core/loader.rs:379-461, has_qk_norm of
 * :556) for the architectures that use rope_neox; capacity is checked against context_length as
 * checked_session_capacity does (src/models/qwen3.rs:108-121). */
int rmi_hip_gguf_qwen3_config(const rmi_hip_gguf *g, uint32_t capacity, int rounding, rmi_hip_qwen3_config *out);
/* Qwen3Model::from_source + Qwen3Session::new over the file (tensor names, shapes and types of
 * src/models/qwen3.rs:262-349; "Missing tensor: .." / "Invalid tensor ..: .." as checked_tensor, :1350-1380). */
rmi_hip_qwen3 *rmi_hip_qwen3_create_from_gguf(const rmi_hip_gguf *g, uint32_t capacity, int rounding);

#ifdef __cplusplus
}
#endif
#endif /* RMI_HIP_H */
