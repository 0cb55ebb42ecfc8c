// Internal declarations shared by the translation units of librmi_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "../../include/rmi_hip.h"

// ---------------------------------------------------------------- layouts
//
// Q8_0 weights in HBM ("tile stream").  Rows are grouped in tiles of 8, the
// blocks of a row in octets of 8 (256 elements).  One tile is contiguous:
//
//   [ scales : n_oct x (8 rows x 8 f16)           ]  n_oct x 128 B
//   [ quants : 2*n_oct quads x (8 rows x 8 L x 16) ]  n_oct x 2048 B
//
// A quad is 4 consecutive blocks; inside it, for row r and lane L (0..7) the
// 16 bytes are the 4-byte slices k = 4L..4L+3 of blocks 4q+0..4q+3.  A wave
// (8 rows x 8 lanes) therefore reads one quad with a single fully coalesced
// 1 KiB load, and lane L owns exactly the elements that lane L of the
// reference's 8-lane f32 accumulator sums (avx2.rs:128-147).  Rows beyond
// n_out and blocks beyond n_in/32 are zero (scale 0, quants 0).  The stream
// carries 34 bytes per block, the same as the source format.
constexpr uint32_t kTileRows = 8;
constexpr uint32_t kOctetBytes = 128 + 2048;  // per tile per octet

// Q4_K weights in HBM.  Tiles of 8 rows; per tile and super-block:
//
//   [ header : 8 rows x 16 B ]  f16 d, f16 dmin, the 12 packed scale bytes
//   [ quants : 8 rows x 8 L x 16 B ]  1024 B
//
// The 16 bytes of (row r, lane L) are four dwords, one per 32-byte group g of
// the 128 nibble bytes: bytes 32g+4L..32g+4L+3, i.e. elements 64g+4L.. (low
// nibbles, sub-block 2g) and 64g+32+4L.. (high nibbles, sub-block 2g+1).  Lane
// L thus owns what lane L of the reference's 8-lane integer accumulator sums
// (quant/mod.rs:770-790), and a wave reads a super-block of 8 rows with one
// coalesced 1 KiB load.  144 bytes per super-block, as in the source format.
constexpr uint32_t kQ4KSuperBytes = 8 * 16 + 1024;  // per tile per super-block

// Q4_0 weights in HBM.  Tiles of 8 rows, blocks in octets of 8; per tile and octet:
//
//   [ scales : 8 rows x 8 f16 ]            128 B
//   [ quants : 8 rows x 8 L x 16 B ]      1024 B   lane L of row r = the 16 nibble bytes of block 8o + L
//
// 18 bytes per block, as in the source format; rows beyond n_out and blocks beyond n_in/32 are zero.
constexpr uint32_t kQ40OctetBytes = 128 + 1024;  // per tile per octet

// Q6_K weights in HBM.  Tiles of 8 rows; per tile and super-block:
//
//   [ scales : 8 rows x 16 int8 ]           128 B
//   [ d      : 8 rows x f16 ]                16 B
//   [ ql     : 8 rows x 8 L x 16 B ]       1024 B   bytes 4L.. of ql[0..32), [32..64), [64..96), [96..128)
//   [ qh     : 8 rows x 8 L x 8 B ]         512 B   bytes 4L.. of qh[0..32), [32..64)
//
// Lane L of a row thus holds the quants 4L..4L+3 of each of the eight 32-element groups, which is
// what lane L of the reference's 8-lane integer accumulator sums (quant/mod.rs:1010-1050).
// 210 bytes per super-block, as in the source format.
constexpr uint32_t kQ6KSuperBytes = 128 + 16 + 1024 + 512;  // per tile per super-block

struct rmi_hip_weight {
    int dtype;
    uint32_t n_in;
    uint32_t n_out;
    uint32_t n_tiles;   // ceil(n_out / 8)
    uint32_t n_units;   // Q8_0, Q4_0: octets per row; Q4_K, Q6_K: super-blocks per row
    size_t tile_bytes;  // bytes of one tile
    size_t nbytes;      // device allocation
    uint8_t *data;      // device pointer
};

// ------------------------------------------------------------------ errors
void rmi_set_error(const char *fmt, ...);
int rmi_fail(int code, const char *fmt, ...);
bool rmi_ready();

#define RMI_HIP_CHECK(expr)                                                                        \
    do {                                                                                           \
        hipError_t _e = (expr);                                                                    \
        if (_e != hipSuccess)                                                                      \
            return rmi_fail(RMI_HIP_E_RUNTIME, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, \
                            __LINE__);                                                             \
    } while (0)

// Activation quants are read with 16-byte loads; scales, sums and outputs with 4-byte ones.
inline bool rmi_misaligned(const void *quants, const void *a = nullptr, const void *b = nullptr, const void *c = nullptr) {
    return (reinterpret_cast<uintptr_t>(quants) & 15) != 0 ||
           ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 3) != 0;
}
#define RMI_ALIGNMENT_MESSAGE "activation quants must be 16-byte aligned, scales / sums / outputs 4-byte aligned"

// How the 8 XCDs divide a GEMM's grid_n x grid_t tiles (rmi_gemm_tile_of, device_common.h): the split along the rows
// that makes the XCDs together fetch the fewest operand bytes, 8 * (w_bytes / split + x_bytes * split / 8), among
// those that divide the tile grid evenly; 0 = the one-dimensional renumbering, which takes any grid.
inline uint32_t rmi_gemm_xcd_split(uint32_t grid_n, uint32_t grid_t, double w_bytes, double x_bytes) {
    if (const char *e = getenv("RMI_GEMM_XCD_SPLIT")) {  // for measurements: 2 or 4 where the grid allows it, else 0
        const uint32_t f = uint32_t(atoi(e));
        return (f == 2 || f == 4) && grid_n % f == 0 && grid_t % (8 / f) == 0 ? f : 0u;
    }
    const double one_dim = w_bytes < x_bytes ? 8.0 * w_bytes + x_bytes : w_bytes + 8.0 * x_bytes;
    uint32_t best = 0;
    double best_cost = one_dim;
    for (uint32_t split : {2u, 4u}) {
        if (grid_n % split != 0 || grid_t % (8 / split) != 0) continue;
        const double cost = w_bytes * (8 / split) + x_bytes * split;
        if (cost < best_cost * 0.95) {
            best_cost = cost;
            best = split;
        }
    }
    return best;
}

#define RMI_REQUIRE_INIT()                                                             \
    do {                                                                               \
        if (!rmi_ready()) return rmi_fail(RMI_HIP_E_NOT_INIT, "rmi_hip_init has not succeeded"); \
    } while (0)

// ---------------------------------------------------- per-thread staging
// One per calling host thread: its own stream plus device and pinned host
// buffers that grow on demand, so concurrent Kernel calls never share state.
struct RmiThreadCtx {
    uint64_t generation = 0;  // the library generation (count of shutdowns) its stream and buffers belong to
    hipStream_t stream = nullptr;
    // weight upload: two pinned and two device staging chunks taken in turn, an event per pair
    void *up_pin[2] = {nullptr, nullptr};
    void *up_dev[2] = {nullptr, nullptr};
    hipEvent_t up_done[2] = {nullptr, nullptr};
    size_t up_cap = 0;
    void *dev[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    size_t dev_cap[6] = {0, 0, 0, 0, 0, 0};
    void *pin[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    size_t pin_cap[6] = {0, 0, 0, 0, 0, 0};
};
RmiThreadCtx *rmi_thread_ctx();
// slot buffers, grown to at least nbytes; nullptr on failure (error is set)
void *rmi_dev_buf(RmiThreadCtx *c, int slot, size_t nbytes);
void *rmi_pin_buf(RmiThreadCtx *c, int slot, size_t nbytes);
int rmi_device_cus();
int rmi_device();  // the device rmi_hip_init bound, -1 before
int rmi_batched_mode();  // RMI_HIP_BATCHED_*: what rmi_hip_set_forward_batched_mode chose
// the device address of the no-allocation entry point's scratch array on `device`, which must be current
int rmi_noalloc_setup(int device);

// ------------------------------------------------- launchers (device ptrs)
// repack tiles [tile0, tile0 + n_tiles) of w; src = the source rows from row tile0 * 8 on (device memory)
int rmi_launch_repack_q8_0(const uint8_t *src, rmi_hip_weight *w, uint32_t tile0, uint32_t n_tiles, hipStream_t s);
int rmi_launch_repack_q4_k(const uint8_t *src, rmi_hip_weight *w, uint32_t tile0, uint32_t n_tiles, hipStream_t s);
int rmi_launch_repack_q6_k(const uint8_t *src, rmi_hip_weight *w, uint32_t tile0, uint32_t n_tiles, hipStream_t s);
int rmi_launch_repack_q4_0(const uint8_t *src, rmi_hip_weight *w, uint32_t tile0, uint32_t n_tiles, hipStream_t s);
// Host rows -> the tile stream of w from row0 (a multiple of 8) on, chunk by chunk through the thread's staging
// pair; enqueues on c->stream and returns without waiting for the last chunk.
int rmi_upload_rows(RmiThreadCtx *c, rmi_hip_weight *w, uint32_t row0, const uint8_t *blocks, uint32_t n_rows);
// One weight whose rows are the parts one below the other ([a ; b ; c]).  NULL + error text on failure.  With
// wait = false the last chunks may still be in flight on the calling thread's stream when it returns (the
// source bytes are already in the staging pair): the caller synchronises that stream before any other
// stream reads the weight.
rmi_hip_weight *rmi_upload_stack(int dtype, const uint8_t *const *parts, const uint32_t *rows, int n_parts,
                                 uint32_t n_in, bool wait);
int rmi_launch_copy_rows(const rmi_hip_weight *src, rmi_hip_weight *dst, uint32_t dst_row0, hipStream_t s);

struct RmiGemvProblem {
    const uint8_t *w;      // tile stream
    const int8_t *x_q8;    // [n_tokens][n_in]
    const float *x_scales; // [n_tokens][n_in/32]
    float *y;              // y[t*y_stride + row]
    uint32_t n_in;
    uint32_t n_oct;
    uint32_t y_stride;
    uint32_t row_start;    // rows written: [row_start, row_end)
    uint32_t row_end;
    uint32_t tile0;        // first tile touched
    uint32_t n_tiles;      // tiles touched
    uint32_t reserved;
};
// token_groups groups of n_tokens (<= 8) tokens each, consecutive in the problem's arrays, in one launch
int rmi_launch_gemv_q8_0_single(const RmiGemvProblem &p, uint32_t n_tokens, hipStream_t s, uint32_t token_groups = 1);
// rows [row_start,row_end) of n_tokens tokens of a Q8_0 or Q4_0 weight, as many GEMV launches (x86-64 order) as
// the LDS staging of the tokens asks for; device pointers, nothing allocated
bool rmi_gemv_q8_0_tokens_fits(const rmi_hip_weight *w);
int rmi_gemv_q8_0_tokens(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y, uint32_t n_tokens,
                         uint32_t y_stride, uint32_t row_start, uint32_t row_end, hipStream_t s);
// the same problem record with w = a Q4_0 tile stream (Q8_0 activation)
int rmi_launch_gemv_q4_0(const RmiGemvProblem &p, uint32_t n_tokens, hipStream_t s);
int rmi_launch_gemv_q4_0_group(const RmiGemvProblem *d_list, const uint4 *d_runs, uint32_t n_runs, uint32_t wpg,
                               uint32_t max_n_oct, uint32_t n_tokens, hipStream_t s);
int rmi_launch_block_dots_q4_0(const rmi_hip_weight *w, const int8_t *x_q8, int32_t *dots, hipStream_t s);
// y = W . Q8_0(rms_norm(x_in + resid) * norm_weight) in one launch, x_out = x_in + resid (x_out != x_in);
// for one token and matrices the fused kernel covers (rmi_gemv_q8_0_norm_fusable)
bool rmi_gemv_q8_0_norm_fusable(const rmi_hip_weight *w);
// h = up * silu(gate) of [gate; up] = W . Q8_0(rms_norm(x_in + resid) * norm_weight), quantized to Q8_0, in one
// launch; W holds the gate rows, then as many up rows (n_out = 2 * n_ff, n_ff a multiple of 32)
bool rmi_gemv_q8_0_norm_silu_fusable(const rmi_hip_weight *w);
int rmi_launch_gemv_q8_0_norm_silu(const rmi_hip_weight *w_gate_up, const float *x_in, const float *resid,
                                   const float *norm_weight, float *x_out, float eps, int rounding, int8_t *h_q8,
                                   float *h_scales, hipStream_t s);
// q|k|v = W . Q8_0(rms_norm(x_in + resid) * norm_weight) with the per-head q/k norm, the NeoX rotation and the
// f16 rounding behind it, in one launch; head dimension 128, W = q rows, k rows, v rows
bool rmi_gemv_q8_0_norm_rope_fusable(const rmi_hip_weight *w, uint32_t n_head, uint32_t n_head_kv, uint32_t head_dim_k,
                                     uint32_t head_dim_v);
int rmi_launch_gemv_q8_0_norm_rope(const rmi_hip_weight *w_qkv, const float *x_in, const float *resid,
                                   const float *norm_weight, float *x_out, float eps, int rounding, const float *q_norm,
                                   const float *k_norm, const float *cos_row, const float *sin_row, uint16_t *q16,
                                   uint16_t *k_row, uint16_t *v_row, uint32_t n_head, uint32_t n_head_kv, hipStream_t s);
int rmi_launch_gemv_q8_0_norm(const rmi_hip_weight *w, const float *x_in, const float *resid, const float *norm_weight,
                              float *x_out, float eps, int rounding, float *y, hipStream_t s);
// d_runs[w] = {problem index, first tile, tile count, 0}: the run of tiles wave w takes
// the run table holds n_runs entries, a multiple of wpg (waves per workgroup); the wpg runs of one
// workgroup belong to one problem (count 0 pads)
int rmi_launch_gemv_q8_0_group(const RmiGemvProblem *d_list, const uint4 *d_runs, uint32_t n_runs, uint32_t wpg,
                               uint32_t max_n_oct, uint32_t n_tokens, hipStream_t s);
// Small batches (1..kMfmaMaxTokens tokens) through int8 MFMA in the order of the reference's NEON kernel; the
// problem records and run tables of the GEMV.  `fits`: the tokens' activations fit the LDS staging.
constexpr uint32_t kMfmaMaxTokens = 64;
bool rmi_gemv_q8_0_mfma_fits(uint32_t n_tokens, uint32_t max_n_oct);
size_t rmi_gemv_q8_0_mfma_lds_bytes(uint32_t n_tokens, uint32_t max_n_oct);
int rmi_launch_gemv_q8_0_mfma(const RmiGemvProblem *single, const RmiGemvProblem *d_list, const uint4 *d_runs,
                              uint32_t n_waves, uint32_t wpg, uint32_t tiles_per_wave, uint32_t max_n_oct,
                              uint32_t n_tokens, hipStream_t s);
uint32_t rmi_gemv_waves_per_group(size_t lds_bytes, size_t run_bytes);
uint32_t rmi_gemv_tiles_per_wave(uint32_t n_oct, uint32_t launch_tiles, uint32_t n_tokens);
int rmi_launch_copy(const void *src, void *dst, size_t nbytes, hipStream_t s);
int rmi_launch_block_dots_q8_0(const rmi_hip_weight *w, const int8_t *x_q8, int32_t *dots, hipStream_t s);
int rmi_launch_quantize_q8_0(const float *x, int8_t *q8, float *scales, uint32_t n_tokens, uint32_t n_in,
                             int rounding, hipStream_t s);
int rmi_launch_matmul_q8_0_f32(const rmi_hip_weight *w, const float *x, float *y, hipStream_t s);
int rmi_launch_matmul_q8_0_f32_scalar(const rmi_hip_weight *w, const float *x, float *y, uint32_t row_start,
                                      uint32_t row_end, hipStream_t s);
int rmi_launch_gemm_q8_0(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                         uint32_t n_tokens, uint32_t y_stride, hipStream_t s);
// the same product for few tokens: one 32 x 32 tile per workgroup, the blocks of a row split over its waves, the
// waves' sums added in wave order (gemm_q8_0_ksplit.hip; within rounding of the single-chain result)
void rmi_gemm_q8_0_ksplit_shape(uint32_t n_in, uint32_t *quads_per_wave, uint32_t *n_waves);
// what either kernel expects a launch to take, in microseconds (rmi_gemm_q8_0_cost_us < 0: no tile shape fits)
bool rmi_gemm_q8_0_shape_forced();  // measurements: RMI_GEMM_SHAPE is set, the fast plan keeps to the tiled kernel
double rmi_gemm_q8_0_cost_us(const rmi_hip_weight *w, uint32_t n_tokens, bool single_chain, uint32_t *groups);
int rmi_launch_gemm_q8_0_grouped(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                                 uint32_t n_tokens, uint32_t y_stride, hipStream_t s);
double rmi_gemm_q8_0_ksplit_cost_us(const rmi_hip_weight *w, uint32_t n_tokens);
int rmi_launch_gemm_q8_0_ksplit(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                                uint32_t n_tokens, uint32_t y_stride, hipStream_t s);

int rmi_launch_quantize_q8_k(const float *x, float *d, int8_t *qs, int16_t *bsums, uint32_t n_tokens, uint32_t n_in,
                             hipStream_t s);
struct RmiQ4kProblem {
    const uint8_t *w;     // Q4_K tile stream
    const float *q8d;     // Q8_K activation: d[n_tokens][n_sb]
    const int8_t *q8qs;   //                  qs[n_tokens][n_in]
    const int16_t *q8bs;  //                  bsums[n_tokens][n_in/16]
    float *y;             // y[t*y_stride + row]
    uint32_t n_sb;
    uint32_t y_stride;
    uint32_t row_start;
    uint32_t row_end;
    uint32_t tile0;
    uint32_t n_tiles;
};
RmiQ4kProblem rmi_make_q4k_problem(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums,
                                   float *y, uint32_t y_stride, uint32_t row_start, uint32_t row_end);
uint32_t rmi_q4k_tiles_per_wave(uint32_t n_sb, uint32_t launch_tiles, uint32_t n_tokens);
int rmi_launch_gemv_q4_k_group(const RmiQ4kProblem *d_list, const uint4 *d_runs, uint32_t n_runs, uint32_t wpg,
                               uint32_t max_n_sb, uint32_t n_tokens, hipStream_t s);
int rmi_launch_gemv_q4_k(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums, float *y,
                         uint32_t n_tokens, uint32_t y_stride, uint32_t row_start, uint32_t row_end, hipStream_t s);
int rmi_launch_gemm_q4_k(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums, float *y,
                         uint32_t n_tokens, uint32_t y_stride, hipStream_t s);
int rmi_launch_gemm_q4_k_block_ints(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums,
                                    int32_t *ints, uint32_t n_tokens, hipStream_t s);
int rmi_launch_block_ints_q4_k(const rmi_hip_weight *w, const int8_t *qs, const int16_t *bsums, int32_t *isum,
                               int32_t *msum, hipStream_t s);
// mode 0: x = q8 * scale rebuilt per element (Q4_KKernel::forward_prequantized)
// mode 1: raw f32 x (QuantizedLinear::forward_dequant)
int rmi_launch_q4_k_dequant_dot(const rmi_hip_weight *w, const float *x_f32, const int8_t *x_q8,
                                const float *x_scales, float *y, uint32_t row_start, uint32_t row_end, int mode,
                                hipStream_t s);

// Q6_K x Q8_K: the same problem record (w = Q6_K tile stream)
uint32_t rmi_q6k_tiles_per_wave(uint32_t n_sb, uint32_t launch_tiles, uint32_t n_tokens);
int rmi_launch_gemv_q6_k_group(const RmiQ4kProblem *d_list, const uint4 *d_runs, uint32_t n_runs, uint32_t wpg,
                               uint32_t max_n_sb, uint32_t n_tokens, hipStream_t s);
int rmi_launch_gemv_q6_k(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums, float *y,
                         uint32_t n_tokens, uint32_t y_stride, uint32_t row_start, uint32_t row_end, hipStream_t s);
// lanes[(row*n_sb + sb)*8 + m]: the int32 each of the eight accumulator lanes converts to f32
int rmi_launch_block_lanes_q6_k(const rmi_hip_weight *w, const int8_t *qs, const int16_t *bsums, int32_t *lanes,
                                hipStream_t s);
// x = q8 * scale rebuilt per element (Q6_KKernel::forward_prequantized)
int rmi_launch_q6_k_dequant_dot(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                                uint32_t row_start, uint32_t row_end, hipStream_t s);

// A fixed list of independent GEMVs (Q8_0 or Q4_K) launched as one kernel.
struct rmi_hip_gemv_group {
    int dtype = 0;
    void *d_list = nullptr;  // RmiGemvProblem[] (Q8_0) or RmiQ4kProblem[] (Q4_K, Q6_K)
    uint4 *d_runs = nullptr;
    uint32_t n_problems = 0;
    uint32_t n_runs = 0;
    uint32_t wpg = 1;  // waves per workgroup
    uint32_t max_units = 0;
    uint32_t n_tokens = 0;
    bool mfma = false;  // Q8_0 only: the small-batch MFMA kernel (NEON order) instead of the GEMV (AVX2 order)
};
