// extern "C" entry points for the K-quant weights: Q4_K (Q4_KKernel and QuantizedLinear) and Q6_K (Q6_KKernel).
#include <vector>

#include "rmi_internal.h"

namespace {

constexpr uint32_t kGemmMinTokens = 16;

int check_q4k(const rmi_hip_weight *w, uint32_t n_in, uint32_t n_out) {
    if (!w || w->dtype != RMI_HIP_DTYPE_Q4_K) return rmi_fail(RMI_HIP_E_INVALID, "not a Q4_K weight handle");
    if (w->n_in != n_in || w->n_out != n_out)
        return rmi_fail(RMI_HIP_E_INVALID, "weight is %u x %u, call says %u x %u", w->n_out, w->n_in, n_out, n_in);
    return RMI_HIP_OK;
}

int check_q6k(const rmi_hip_weight *w, uint32_t n_in, uint32_t n_out) {
    if (!w || w->dtype != RMI_HIP_DTYPE_Q6_K) return rmi_fail(RMI_HIP_E_INVALID, "not a Q6_K weight handle");
    if (w->n_in != n_in || w->n_out != n_out)
        return rmi_fail(RMI_HIP_E_INVALID, "weight is %u x %u, call says %u x %u", w->n_out, w->n_in, n_out, n_in);
    return RMI_HIP_OK;
}

// q4_k.rs:30-35, q6_k.rs:55-60: per_thread = ceil(n_out / nth)
bool partition(uint32_t n_out, uint32_t ith, uint32_t nth, uint32_t *start, uint32_t *end) {
    if (nth == 0) nth = 1;
    const uint32_t per_thread = (n_out + nth - 1) / nth;
    const uint64_t s = uint64_t(ith) * per_thread;
    if (s >= n_out) return false;
    *start = uint32_t(s);
    *end = *start + per_thread < n_out ? *start + per_thread : n_out;
    return *start < *end;
}

int fetch(RmiThreadCtx *c, void *host, const void *dev, size_t nbytes, int pin_slot) {
    if (nbytes == 0) return RMI_HIP_OK;
    void *pin = rmi_pin_buf(c, pin_slot, nbytes);
    if (!pin) return RMI_HIP_E_RUNTIME;
    RMI_HIP_CHECK(hipMemcpyAsync(pin, dev, nbytes, hipMemcpyDeviceToHost, c->stream));
    RMI_HIP_CHECK(hipStreamSynchronize(c->stream));
    memcpy(host, pin, nbytes);
    return RMI_HIP_OK;
}

// host bytes -> device slot via pinned slot (same index)
void *push(RmiThreadCtx *c, int slot, const void *host, size_t nbytes) {
    void *pin = rmi_pin_buf(c, slot, nbytes);
    void *dev = rmi_dev_buf(c, slot, nbytes);
    if (!pin || !dev) return nullptr;
    memcpy(pin, host, nbytes);
    if (hipMemcpyAsync(dev, pin, nbytes, hipMemcpyHostToDevice, c->stream) != hipSuccess) {
        rmi_set_error("hipMemcpyAsync H2D failed");
        return nullptr;
    }
    return dev;
}

}  // namespace

extern "C" {

int rmi_hip_q4_k_forward_prepared(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                                  const int16_t *q8k_bsums, float *output, uint32_t n_in, uint32_t n_out, uint32_t ith,
                                  uint32_t nth) {
    RMI_REQUIRE_INIT();
    int rc = check_q4k(w, n_in, n_out);
    if (rc != RMI_HIP_OK) return rc;
    uint32_t start, end;
    if (!partition(n_out, ith, nth, &start, &end)) return RMI_HIP_OK;
    if (!q8k_d || !q8k_qs || !q8k_bsums || !output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const float *d_d = static_cast<const float *>(push(c, 0, q8k_d, size_t(n_in / 256) * 4));
    const int8_t *d_qs = static_cast<const int8_t *>(push(c, 2, q8k_qs, n_in));
    const int16_t *d_bs = static_cast<const int16_t *>(push(c, 3, q8k_bsums, size_t(n_in / 16) * 2));
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, size_t(end - start) * 4));
    if (!d_d || !d_qs || !d_bs || !d_y) return RMI_HIP_E_RUNTIME;
    rc = rmi_launch_gemv_q4_k(w, d_d, d_qs, d_bs, d_y - start, 1, end - start, start, end, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, output + start, d_y, size_t(end - start) * 4, 1);
}

// Kernel::forward_batched of a Q4_K weight.  gemm = false: every token through the GEMV in the x86-64 kernel's
// order (8 at a time), so a token's result does not depend on its batch, as in trait_.rs:78-109.  gemm = true:
// from 16 tokens on the matrix-core GEMM, whose f32 sums are one chain per output (no reference order).
static int q4_k_forward_batched(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                uint32_t n_out, uint32_t n_tokens, bool gemm) {
    RMI_REQUIRE_INIT();
    int rc = check_q4k(w, n_in, n_out);
    if (rc != RMI_HIP_OK) return rc;
    if (n_tokens == 0 || n_out == 0) return RMI_HIP_OK;
    if (!input || !output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const size_t n_x = size_t(n_tokens) * n_in;
    const float *d_x = static_cast<const float *>(push(c, 0, input, n_x * 4));
    int8_t *d_qs = static_cast<int8_t *>(rmi_dev_buf(c, 2, n_x));
    int16_t *d_bs = static_cast<int16_t *>(rmi_dev_buf(c, 3, n_x / 16 * 2));
    float *d_d = static_cast<float *>(rmi_dev_buf(c, 4, n_x / 256 * 4));
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, size_t(n_tokens) * n_out * 4));
    if (!d_x || !d_qs || !d_bs || !d_d || !d_y) return RMI_HIP_E_RUNTIME;
    rc = rmi_launch_quantize_q8_k(d_x, d_d, d_qs, d_bs, n_tokens, n_in, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    rc = gemm && n_tokens >= kGemmMinTokens
             ? rmi_launch_gemm_q4_k(w, d_d, d_qs, d_bs, d_y, n_tokens, n_out, c->stream)
             : rmi_launch_gemv_q4_k(w, d_d, d_qs, d_bs, d_y, n_tokens, n_out, 0, n_out, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, output, d_y, size_t(n_tokens) * n_out * 4, 1);
}

int rmi_hip_q4_k_forward_batched(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                 uint32_t n_out, uint32_t n_tokens) {
    return q4_k_forward_batched(w, input, output, n_in, n_out, n_tokens, rmi_batched_mode() != RMI_HIP_BATCHED_X86_ORDER);
}

int rmi_hip_q4_k_forward_batched_mfma(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                      uint32_t n_out, uint32_t n_tokens) {
    return q4_k_forward_batched(w, input, output, n_in, n_out, n_tokens, true);
}

int rmi_hip_quantize_row_q8_k(const float *input, uint32_t n, float *d, int8_t *qs, int16_t *bsums) {
    RMI_REQUIRE_INIT();
    if (n % 256 != 0) return rmi_fail(RMI_HIP_E_INVALID, "n=%u is not a multiple of 256", n);  // quant/mod.rs:144 asserts
    if (n == 0) return RMI_HIP_OK;
    if (!input || !d || !qs || !bsums) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const float *d_x = static_cast<const float *>(push(c, 0, input, size_t(n) * 4));
    int8_t *d_qs = static_cast<int8_t *>(rmi_dev_buf(c, 2, n));
    int16_t *d_bs = static_cast<int16_t *>(rmi_dev_buf(c, 3, size_t(n) / 16 * 2));
    float *d_d = static_cast<float *>(rmi_dev_buf(c, 4, size_t(n) / 256 * 4));
    if (!d_x || !d_qs || !d_bs || !d_d) return RMI_HIP_E_RUNTIME;
    int rc = rmi_launch_quantize_q8_k(d_x, d_d, d_qs, d_bs, 1, n, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    rc = fetch(c, qs, d_qs, n, 1);
    if (rc == RMI_HIP_OK) rc = fetch(c, bsums, d_bs, size_t(n) / 16 * 2, 1);
    if (rc == RMI_HIP_OK) rc = fetch(c, d, d_d, size_t(n) / 256 * 4, 1);
    return rc;
}

int rmi_hip_q4_k_forward_prequantized(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                      float *output, uint32_t n_in, uint32_t n_out, uint32_t ith, uint32_t nth) {
    RMI_REQUIRE_INIT();
    int rc = check_q4k(w, n_in, n_out);
    if (rc != RMI_HIP_OK) return rc;
    uint32_t start, end;
    if (!partition(n_out, ith, nth, &start, &end)) return RMI_HIP_OK;
    if (!input_q8 || !input_scales || !output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const int8_t *d_q8 = static_cast<const int8_t *>(push(c, 0, input_q8, n_in));
    const float *d_sc = static_cast<const float *>(push(c, 2, input_scales, size_t(n_in / 32) * 4));
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, size_t(end - start) * 4));
    if (!d_q8 || !d_sc || !d_y) return RMI_HIP_E_RUNTIME;
    rc = rmi_launch_q4_k_dequant_dot(w, nullptr, d_q8, d_sc, d_y - start, start, end, 0, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, output + start, d_y, size_t(end - start) * 4, 1);
}

int rmi_hip_quantized_linear_forward(const rmi_hip_weight *w, const float *input, float *output, uint32_t in_features,
                                     uint32_t out_features) {
    RMI_REQUIRE_INIT();
    int rc = check_q4k(w, in_features, out_features);
    if (rc != RMI_HIP_OK) return rc;
    if (out_features == 0) return RMI_HIP_OK;
    if (!input || !output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const float *d_x = static_cast<const float *>(push(c, 0, input, size_t(in_features) * 4));
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, size_t(out_features) * 4));
    if (!d_x || !d_y) return RMI_HIP_E_RUNTIME;
    rc = rmi_launch_q4_k_dequant_dot(w, d_x, nullptr, nullptr, d_y, 0, out_features, 1, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, output, d_y, size_t(out_features) * 4, 1);
}

int rmi_hip_quantized_linear_forward_dev(const rmi_hip_weight *w, const float *x, float *y, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q4_K) return rmi_fail(RMI_HIP_E_INVALID, "not a Q4_K weight handle");
    if (w->n_out == 0) return RMI_HIP_OK;
    if (!x || !y) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    return rmi_launch_q4_k_dequant_dot(w, x, nullptr, nullptr, y, 0, w->n_out, 1, static_cast<hipStream_t>(stream));
}

int rmi_hip_block_ints_q4_k(const rmi_hip_weight *w, const int8_t *q8k_qs, const int16_t *q8k_bsums, int32_t *isum,
                            int32_t *msum) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q4_K) return rmi_fail(RMI_HIP_E_INVALID, "not a Q4_K weight handle");
    const size_t n = size_t(w->n_out) * w->n_units;
    if (n == 0) return RMI_HIP_OK;
    if (!q8k_qs || !q8k_bsums || !isum || !msum) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const int8_t *d_qs = static_cast<const int8_t *>(push(c, 0, q8k_qs, w->n_in));
    const int16_t *d_bs = static_cast<const int16_t *>(push(c, 2, q8k_bsums, size_t(w->n_in / 16) * 2));
    int32_t *d_out = static_cast<int32_t *>(rmi_dev_buf(c, 1, n * 8));
    if (!d_qs || !d_bs || !d_out) return RMI_HIP_E_RUNTIME;
    int rc = rmi_launch_block_ints_q4_k(w, d_qs, d_bs, d_out, d_out + n, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    rc = fetch(c, isum, d_out, n * 4, 1);
    if (rc == RMI_HIP_OK) rc = fetch(c, msum, d_out + n, n * 4, 1);
    return rc;
}

int rmi_hip_gemv_q4_k_q8k_dev(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                              const int16_t *q8k_bsums, float *y, uint32_t n_tokens, uint32_t y_stride,
                              uint32_t row_start, uint32_t row_end, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q4_K) return rmi_fail(RMI_HIP_E_INVALID, "not a Q4_K weight handle");
    if (row_start >= row_end || n_tokens == 0) return RMI_HIP_OK;
    if (row_end > w->n_out) return rmi_fail(RMI_HIP_E_INVALID, "rows [%u,%u) exceed n_out=%u", row_start, row_end, w->n_out);
    if (y_stride < row_end && n_tokens > 1) return rmi_fail(RMI_HIP_E_INVALID, "y_stride=%u < row_end=%u", y_stride, row_end);
    if (!q8k_d || !q8k_qs || !q8k_bsums || !y) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    if (rmi_misaligned(q8k_qs, q8k_d, q8k_bsums, y)) return rmi_fail(RMI_HIP_E_INVALID, RMI_ALIGNMENT_MESSAGE);
    return rmi_launch_gemv_q4_k(w, q8k_d, q8k_qs, q8k_bsums, y, n_tokens, y_stride, row_start, row_end,
                                static_cast<hipStream_t>(stream));
}

int rmi_hip_gemm_q4_k_q8k_dev(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                              const int16_t *q8k_bsums, float *y, uint32_t n_tokens, uint32_t y_stride, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q4_K) return rmi_fail(RMI_HIP_E_INVALID, "not a Q4_K weight handle");
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    if (y_stride < w->n_out) return rmi_fail(RMI_HIP_E_INVALID, "y_stride=%u < n_out=%u", y_stride, w->n_out);
    if (!q8k_d || !q8k_qs || !q8k_bsums || !y) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    if (rmi_misaligned(q8k_qs, q8k_d, q8k_bsums, y)) return rmi_fail(RMI_HIP_E_INVALID, RMI_ALIGNMENT_MESSAGE);
    return rmi_launch_gemm_q4_k(w, q8k_d, q8k_qs, q8k_bsums, y, n_tokens, y_stride, static_cast<hipStream_t>(stream));
}

int rmi_hip_gemm_block_ints_q4_k_dev(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                                     const int16_t *q8k_bsums, int32_t *ints, uint32_t n_tokens, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q4_K) return rmi_fail(RMI_HIP_E_INVALID, "not a Q4_K weight handle");
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    if (!q8k_d || !q8k_qs || !q8k_bsums || !ints) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    if (rmi_misaligned(q8k_qs, q8k_d, q8k_bsums, ints)) return rmi_fail(RMI_HIP_E_INVALID, RMI_ALIGNMENT_MESSAGE);
    return rmi_launch_gemm_q4_k_block_ints(w, q8k_d, q8k_qs, q8k_bsums, ints, n_tokens, static_cast<hipStream_t>(stream));
}

static rmi_hip_gemv_group *group_create_kquant(int dtype, uint32_t n_problems, const rmi_hip_weight *const *weights,
                                               const float *const *q8k_d, const int8_t *const *q8k_qs,
                                               const int16_t *const *q8k_bsums, float *const *y, uint32_t n_tokens) {
    const bool q6 = dtype == RMI_HIP_DTYPE_Q6_K;
    const uint32_t super_bytes = q6 ? kQ6KSuperBytes : kQ4KSuperBytes;
    if (!rmi_ready()) {
        rmi_set_error("rmi_hip_init has not succeeded");
        return nullptr;
    }
    if (n_problems == 0 || n_tokens == 0 || n_tokens > 8 || !weights || !q8k_d || !q8k_qs || !q8k_bsums || !y) {
        rmi_set_error("gemv group needs >=1 problem and 1..8 tokens");
        return nullptr;
    }
    if (!rmi_thread_ctx()) return nullptr;
    std::vector<RmiQ4kProblem> list(n_problems);
    rmi_hip_gemv_group *g = new rmi_hip_gemv_group();
    g->dtype = dtype;
    g->n_problems = n_problems;
    g->n_tokens = n_tokens;
    uint64_t total_tiles = 0;
    for (uint32_t i = 0; i < n_problems; i++) {
        const rmi_hip_weight *w = weights[i];
        if (!w || w->dtype != dtype || !q8k_d[i] || !q8k_qs[i] || !q8k_bsums[i] || !y[i]) {
            rmi_set_error("gemv group problem %u: bad weight handle or null pointer", i);
            delete g;
            return nullptr;
        }
        if (rmi_misaligned(q8k_qs[i], q8k_d[i], q8k_bsums[i], y[i])) {
            rmi_set_error("gemv group problem %u: " RMI_ALIGNMENT_MESSAGE, i);
            delete g;
            return nullptr;
        }
        list[i] = rmi_make_q4k_problem(w, q8k_d[i], q8k_qs[i], q8k_bsums[i], y[i], w->n_out, 0, w->n_out);
        total_tiles += list[i].n_tiles;
        if (w->n_units > g->max_units) g->max_units = w->n_units;
    }
    if (total_tiles > 0x7fffffffull || size_t(n_tokens) * g->max_units * 304 > 64 * 1024) {
        rmi_set_error("gemv group too large (%llu tiles, %u tokens x %u super-blocks)", (unsigned long long)total_tiles,
                      n_tokens, g->max_units);
        delete g;
        return nullptr;
    }
    const auto tiles_per_wave = q6 ? rmi_q6k_tiles_per_wave : rmi_q4k_tiles_per_wave;
    g->wpg = rmi_gemv_waves_per_group(
        size_t(n_tokens) * g->max_units * 304,
        size_t(tiles_per_wave(g->max_units, uint32_t(total_tiles), n_tokens)) * g->max_units * super_bytes);
    std::vector<uint4> runs;
    for (uint32_t i = 0; i < n_problems; i++) {
        if (list[i].n_sb == 0) continue;
        const uint32_t tpw = tiles_per_wave(list[i].n_sb, uint32_t(total_tiles), n_tokens);
        for (uint32_t k = 0; k < list[i].n_tiles; k += tpw)
            runs.push_back(make_uint4(i, k, list[i].n_tiles - k < tpw ? list[i].n_tiles - k : tpw, 0));
        while (runs.size() % g->wpg) runs.push_back(make_uint4(i, 0, 0, 0));
    }
    g->n_runs = uint32_t(runs.size());
    hipError_t e = hipMalloc(&g->d_list, sizeof(RmiQ4kProblem) * n_problems);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&g->d_runs), sizeof(uint4) * (runs.size() + 1));
    if (e == hipSuccess) e = hipMemcpy(g->d_list, list.data(), sizeof(RmiQ4kProblem) * n_problems, hipMemcpyHostToDevice);
    if (e == hipSuccess && !runs.empty())
        e = hipMemcpy(g->d_runs, runs.data(), sizeof(uint4) * runs.size(), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        rmi_set_error("gemv group upload failed: %s", hipGetErrorString(e));
        if (g->d_list) (void)hipFree(g->d_list);
        if (g->d_runs) (void)hipFree(g->d_runs);
        delete g;
        return nullptr;
    }
    return g;
}

rmi_hip_gemv_group *rmi_hip_gemv_group_create_q4_k(uint32_t n_problems, const rmi_hip_weight *const *weights,
                                                   const float *const *q8k_d, const int8_t *const *q8k_qs,
                                                   const int16_t *const *q8k_bsums, float *const *y,
                                                   uint32_t n_tokens) {
    return group_create_kquant(RMI_HIP_DTYPE_Q4_K, n_problems, weights, q8k_d, q8k_qs, q8k_bsums, y, n_tokens);
}

rmi_hip_gemv_group *rmi_hip_gemv_group_create_q6_k(uint32_t n_problems, const rmi_hip_weight *const *weights,
                                                   const float *const *q8k_d, const int8_t *const *q8k_qs,
                                                   const int16_t *const *q8k_bsums, float *const *y,
                                                   uint32_t n_tokens) {
    return group_create_kquant(RMI_HIP_DTYPE_Q6_K, n_problems, weights, q8k_d, q8k_qs, q8k_bsums, y, n_tokens);
}

// ---- Q6_K

int rmi_hip_q6_k_forward_prepared(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                                  const int16_t *q8k_bsums, float *output, uint32_t n_in, uint32_t n_out, uint32_t ith,
                                  uint32_t nth) {
    RMI_REQUIRE_INIT();
    int rc = check_q6k(w, n_in, n_out);
    if (rc != RMI_HIP_OK) return rc;
    uint32_t start, end;
    if (!partition(n_out, ith, nth, &start, &end)) return RMI_HIP_OK;
    if (!q8k_d || !q8k_qs || !q8k_bsums || !output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const float *d_d = static_cast<const float *>(push(c, 0, q8k_d, size_t(n_in / 256) * 4));
    const int8_t *d_qs = static_cast<const int8_t *>(push(c, 2, q8k_qs, n_in));
    const int16_t *d_bs = static_cast<const int16_t *>(push(c, 3, q8k_bsums, size_t(n_in / 16) * 2));
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, size_t(end - start) * 4));
    if (!d_d || !d_qs || !d_bs || !d_y) return RMI_HIP_E_RUNTIME;
    rc = rmi_launch_gemv_q6_k(w, d_d, d_qs, d_bs, d_y - start, 1, end - start, start, end, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, output + start, d_y, size_t(end - start) * 4, 1);
}

int rmi_hip_q6_k_forward_batched(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                 uint32_t n_out, uint32_t n_tokens) {
    RMI_REQUIRE_INIT();
    int rc = check_q6k(w, n_in, n_out);
    if (rc != RMI_HIP_OK) return rc;
    if (n_tokens == 0 || n_out == 0) return RMI_HIP_OK;
    if (!input || !output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const size_t n_x = size_t(n_tokens) * n_in;
    const float *d_x = static_cast<const float *>(push(c, 0, input, n_x * 4));
    int8_t *d_qs = static_cast<int8_t *>(rmi_dev_buf(c, 2, n_x));
    int16_t *d_bs = static_cast<int16_t *>(rmi_dev_buf(c, 3, n_x / 16 * 2));
    float *d_d = static_cast<float *>(rmi_dev_buf(c, 4, n_x / 256 * 4));
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, size_t(n_tokens) * n_out * 4));
    if (!d_x || !d_qs || !d_bs || !d_d || !d_y) return RMI_HIP_E_RUNTIME;
    rc = rmi_launch_quantize_q8_k(d_x, d_d, d_qs, d_bs, n_tokens, n_in, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    rc = rmi_launch_gemv_q6_k(w, d_d, d_qs, d_bs, d_y, n_tokens, n_out, 0, n_out, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, output, d_y, size_t(n_tokens) * n_out * 4, 1);
}

int rmi_hip_q6_k_forward_prequantized(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                      float *output, uint32_t n_in, uint32_t n_out, uint32_t ith, uint32_t nth) {
    RMI_REQUIRE_INIT();
    int rc = check_q6k(w, n_in, n_out);
    if (rc != RMI_HIP_OK) return rc;
    uint32_t start, end;
    if (!partition(n_out, ith, nth, &start, &end)) return RMI_HIP_OK;
    if (!input_q8 || !input_scales || !output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const int8_t *d_q8 = static_cast<const int8_t *>(push(c, 0, input_q8, n_in));
    const float *d_sc = static_cast<const float *>(push(c, 2, input_scales, size_t(n_in / 32) * 4));
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, size_t(end - start) * 4));
    if (!d_q8 || !d_sc || !d_y) return RMI_HIP_E_RUNTIME;
    rc = rmi_launch_q6_k_dequant_dot(w, d_q8, d_sc, d_y - start, start, end, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, output + start, d_y, size_t(end - start) * 4, 1);
}

int rmi_hip_block_lanes_q6_k(const rmi_hip_weight *w, const int8_t *q8k_qs, const int16_t *q8k_bsums,
                             int32_t *lanes) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q6_K) return rmi_fail(RMI_HIP_E_INVALID, "not a Q6_K weight handle");
    const size_t n = size_t(w->n_out) * w->n_units * 8;
    if (n == 0) return RMI_HIP_OK;
    if (!q8k_qs || !q8k_bsums || !lanes) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const int8_t *d_qs = static_cast<const int8_t *>(push(c, 0, q8k_qs, w->n_in));
    const int16_t *d_bs = static_cast<const int16_t *>(push(c, 2, q8k_bsums, size_t(w->n_in / 16) * 2));
    int32_t *d_out = static_cast<int32_t *>(rmi_dev_buf(c, 1, n * 4));
    if (!d_qs || !d_bs || !d_out) return RMI_HIP_E_RUNTIME;
    int rc = rmi_launch_block_lanes_q6_k(w, d_qs, d_bs, d_out, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, lanes, d_out, n * 4, 1);
}

int rmi_hip_gemv_q6_k_q8k_dev(const rmi_hip_weight *w, const float *q8k_d, const int8_t *q8k_qs,
                              const int16_t *q8k_bsums, float *y, uint32_t n_tokens, uint32_t y_stride,
                              uint32_t row_start, uint32_t row_end, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q6_K) return rmi_fail(RMI_HIP_E_INVALID, "not a Q6_K weight handle");
    if (row_start >= row_end || n_tokens == 0) return RMI_HIP_OK;
    if (row_end > w->n_out) return rmi_fail(RMI_HIP_E_INVALID, "rows [%u,%u) exceed n_out=%u", row_start, row_end, w->n_out);
    if (y_stride < row_end && n_tokens > 1) return rmi_fail(RMI_HIP_E_INVALID, "y_stride=%u < row_end=%u", y_stride, row_end);
    if (!q8k_d || !q8k_qs || !q8k_bsums || !y) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    if (rmi_misaligned(q8k_qs, q8k_d, q8k_bsums, y)) return rmi_fail(RMI_HIP_E_INVALID, RMI_ALIGNMENT_MESSAGE);
    return rmi_launch_gemv_q6_k(w, q8k_d, q8k_qs, q8k_bsums, y, n_tokens, y_stride, row_start, row_end,
                                static_cast<hipStream_t>(stream));
}

int rmi_hip_quantize_row_q8_k_dev(const float *x, float *d, int8_t *qs, int16_t *bsums, uint32_t n_tokens,
                                  uint32_t n_in, void *stream) {
    RMI_REQUIRE_INIT();
    if (n_in % 256 != 0) return rmi_fail(RMI_HIP_E_INVALID, "n_in=%u is not a multiple of 256", n_in);
    if (!x || !d || !qs || !bsums) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    return rmi_launch_quantize_q8_k(x, d, qs, bsums, n_tokens, n_in, static_cast<hipStream_t>(stream));
}

}  // extern "C"
