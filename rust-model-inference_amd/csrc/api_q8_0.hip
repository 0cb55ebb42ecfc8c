// extern "C" entry points for Q8_0 weights: the host-slice calls that stand in
// for the Kernel trait methods, the device-resident calls, and GEMV groups.
#include <vector>

#include "rmi_internal.h"

namespace {

// GEMV launches take at most 8 tokens; at or above this many the MFMA GEMM runs.
constexpr uint32_t kGemmMinTokens = 16;

int check_q8(const rmi_hip_weight *w, uint32_t n_in, uint32_t n_out) {
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (w->n_in != n_in || w->n_out != n_out)
        return rmi_fail(RMI_HIP_E_INVALID, "weight is %u x %u, call says %u x %u", w->n_out, w->n_in, n_out, n_in);
    return RMI_HIP_OK;
}

RmiGemvProblem make_problem(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                            uint32_t y_stride, uint32_t row_start, uint32_t row_end) {
    RmiGemvProblem p{};
    p.w = w->data;
    p.x_q8 = x_q8;
    p.x_scales = x_scales;
    p.y = y;
    p.n_in = w->n_in;
    p.n_oct = w->n_units;
    p.y_stride = y_stride;
    p.row_start = row_start;
    p.row_end = row_end;
    p.tile0 = row_start / kTileRows;
    p.n_tiles = row_end > row_start ? (row_end + kTileRows - 1) / kTileRows - p.tile0 : 0;
    p.reserved = 0;
    return p;
}

// tokens per GEMV launch so that the LDS staging fits
uint32_t gemv_chunk(const rmi_hip_weight *w) {
    const size_t per_token = size_t(w->n_units) * (w->dtype == RMI_HIP_DTYPE_Q4_0 ? 320 : 288);
    uint32_t c = per_token ? uint32_t((64 * 1024) / per_token) : 8;
    return c > 8 ? 8 : c;
}

}  // namespace

// whether rmi_gemv_q8_0_tokens can stage a row of this weight at all (callers that must not enqueue anything
// before every check has passed ask first)
bool rmi_gemv_q8_0_tokens_fits(const rmi_hip_weight *w) { return gemv_chunk(w) != 0; }

// device pointers in, rows [row_start,row_end) of n_tokens tokens
int rmi_gemv_q8_0_tokens(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y, uint32_t n_tokens,
                         uint32_t y_stride, uint32_t row_start, uint32_t row_end, hipStream_t s) {
    const uint32_t chunk = gemv_chunk(w);
    if (chunk == 0) return rmi_fail(RMI_HIP_E_INVALID, "n_in=%u is too long for the GEMV staging", w->n_in);
    const uint32_t nb = w->n_in / 32;
    uint32_t t0 = 0;
    if (w->dtype != RMI_HIP_DTYPE_Q4_0 && n_tokens >= 2 * chunk) {
        // every full group of `chunk` tokens in one launch (the groups re-read the weight from L2), up to what a
        // grid's second dimension holds
        const uint32_t groups = n_tokens / chunk < 65535 ? n_tokens / chunk : 65535;
        RmiGemvProblem p = make_problem(w, x_q8, x_scales, y, y_stride, row_start, row_end);
        int rc = rmi_launch_gemv_q8_0_single(p, chunk, s, groups);
        if (rc != RMI_HIP_OK) return rc;
        t0 = groups * chunk;
    }
    for (; t0 < n_tokens; t0 += chunk) {
        const uint32_t nt = n_tokens - t0 < chunk ? n_tokens - t0 : chunk;
        RmiGemvProblem p = make_problem(w, x_q8 + size_t(t0) * w->n_in, x_scales + size_t(t0) * nb,
                                        y + size_t(t0) * y_stride, y_stride, row_start, row_end);
        int rc = w->dtype == RMI_HIP_DTYPE_Q4_0 ? rmi_launch_gemv_q4_0(p, nt, s) : rmi_launch_gemv_q8_0_single(p, nt, s);
        if (rc != RMI_HIP_OK) return rc;
    }
    return RMI_HIP_OK;
}

namespace {

// Runs of an even number of tiles (the small-batch kernel takes them in pairs), long enough to amortise the
// staging of the tokens, short enough to fill the chip.  Measured on the Qwen3-0.6B set at 8 / 16 / 32 tokens:
// twice the GEMV's run length with eight waves per workgroup is within 1 % of the best of {1,2,4,8} x {2,4,8}.
uint32_t mfma_tiles_per_wave(uint32_t n_oct, uint32_t launch_tiles, uint32_t n_tokens) {
    const uint32_t base = rmi_gemv_tiles_per_wave(n_oct, launch_tiles, n_tokens);
    uint32_t mul = n_tokens > 16 ? 4 : 2;
    const uint32_t fill = uint32_t(rmi_device_cus()) * 8;  // a launch too small to fill the chip keeps short runs
    while (mul > 1 && launch_tiles / (base * mul) < fill) mul >>= 1;
    return (base * mul + 1) & ~1u;
}

// 1..kMfmaMaxTokens tokens in one launch of the small-batch MFMA kernel (NEON order)
int mfma_tokens(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y, uint32_t n_tokens,
                uint32_t y_stride, uint32_t row_start, uint32_t row_end, hipStream_t s) {
    const RmiGemvProblem p = make_problem(w, x_q8, x_scales, y, y_stride, row_start, row_end);
    if (p.n_tiles == 0 || p.n_oct == 0) return RMI_HIP_OK;
    const uint32_t tpw = mfma_tiles_per_wave(p.n_oct, p.n_tiles, n_tokens);
    const uint32_t wpg = rmi_gemv_waves_per_group(rmi_gemv_q8_0_mfma_lds_bytes(n_tokens, p.n_oct),
                                                  size_t(tpw) * p.n_oct * kOctetBytes);
    return rmi_launch_gemv_q8_0_mfma(&p, nullptr, nullptr, (p.n_tiles + tpw - 1) / tpw, wpg, tpw, p.n_oct, n_tokens, s);
}

// host activation (q8 + scales) -> one pinned + one device buffer
struct StagedX {
    int8_t *d_q8;
    float *d_scales;
};
int stage_x(RmiThreadCtx *c, const uint8_t *q8, const float *scales, size_t n_q8, size_t n_scales, StagedX *out) {
    const size_t q_bytes = (n_q8 + 15) & ~size_t(15);
    const size_t total = q_bytes + n_scales * 4;
    uint8_t *pin = static_cast<uint8_t *>(rmi_pin_buf(c, 0, total));
    uint8_t *dev = static_cast<uint8_t *>(rmi_dev_buf(c, 0, total));
    if (!pin || !dev) return RMI_HIP_E_RUNTIME;
    memcpy(pin, q8, n_q8);
    memcpy(pin + q_bytes, scales, n_scales * 4);
    RMI_HIP_CHECK(hipMemcpyAsync(dev, pin, total, hipMemcpyHostToDevice, c->stream));
    out->d_q8 = reinterpret_cast<int8_t *>(dev);
    out->d_scales = reinterpret_cast<float *>(dev + q_bytes);
    return RMI_HIP_OK;
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

int host_gemv_range(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales, float *out_row_start,
                    uint32_t n_tokens, uint32_t out_stride, uint32_t row_start, uint32_t row_end) {
    if (row_start >= row_end) return RMI_HIP_OK;
    if (row_end > w->n_out) return rmi_fail(RMI_HIP_E_INVALID, "rows [%u,%u) exceed n_out=%u", row_start, row_end, w->n_out);
    if (!input_q8 || !input_scales || !out_row_start) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    StagedX x;
    int rc = stage_x(c, input_q8, input_scales, size_t(n_tokens) * w->n_in, size_t(n_tokens) * (w->n_in / 32), &x);
    if (rc != RMI_HIP_OK) return rc;
    const uint32_t n_rows = row_end - row_start;
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, size_t(n_tokens) * n_rows * 4));
    if (!d_y) return RMI_HIP_E_RUNTIME;
    // device y holds only the row slice: y[t][row - row_start]
    rc = rmi_gemv_q8_0_tokens(w, x.d_q8, x.d_scales, d_y - row_start, n_tokens, n_rows, row_start, row_end, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    if (out_stride == n_rows) return fetch(c, out_row_start, d_y, size_t(n_tokens) * n_rows * 4, 1);
    float *pin = static_cast<float *>(rmi_pin_buf(c, 1, size_t(n_tokens) * n_rows * 4));
    if (!pin) return RMI_HIP_E_RUNTIME;
    RMI_HIP_CHECK(hipMemcpyAsync(pin, d_y, size_t(n_tokens) * n_rows * 4, hipMemcpyDeviceToHost, c->stream));
    RMI_HIP_CHECK(hipStreamSynchronize(c->stream));
    for (uint32_t t = 0; t < n_tokens; t++)
        memcpy(out_row_start + size_t(t) * out_stride, pin + size_t(t) * n_rows, size_t(n_rows) * 4);
    return RMI_HIP_OK;
}

}  // namespace

extern "C" {

int rmi_hip_matmul_q8_0_quantized_range(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                        float *output, uint32_t n_in, uint32_t row_start, uint32_t row_end) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (w->n_in != n_in) return rmi_fail(RMI_HIP_E_INVALID, "weight has n_in=%u, call says %u", w->n_in, n_in);
    return host_gemv_range(w, input_q8, input_scales, output, 1, row_end > row_start ? row_end - row_start : 0,
                           row_start, row_end);
}

int rmi_hip_q8_0_forward_prequantized(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                      float *output, uint32_t n_in, uint32_t n_out, uint32_t ith, uint32_t nth) {
    RMI_REQUIRE_INIT();
    int rc = check_q8(w, n_in, n_out);
    if (rc != RMI_HIP_OK) return rc;
    uint32_t start = 0, end = n_out;
    if (nth > 1 && n_out != 0) {  // parallel.rs:114-138
        const uint32_t per_thread = (n_out + nth - 1) / nth;
        const uint64_t s64 = uint64_t(ith) * per_thread;
        if (s64 >= n_out) return RMI_HIP_OK;
        start = uint32_t(s64);
        end = start + per_thread < n_out ? start + per_thread : n_out;
    }
    if (start >= end) return RMI_HIP_OK;
    if (!output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    return host_gemv_range(w, input_q8, input_scales, output + start, 1, end - start, start, end);
}

int rmi_hip_matmul_q8_0_quantized_batch(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                        float *output, uint32_t n_in, uint32_t n_out, uint32_t n_tokens) {
    RMI_REQUIRE_INIT();
    int rc = check_q8(w, n_in, n_out);
    if (rc != RMI_HIP_OK) return rc;
    if (n_tokens == 0 || n_out == 0) return RMI_HIP_OK;
    return host_gemv_range(w, input_q8, input_scales, output, n_tokens, n_out, 0, n_out);
}

// Kernel::forward / forward_batched on host slices.  x86_order: every token through the GEMV in the x86-64 kernel's
// order, so a token's result does not depend on the batch it arrives in (forward_batched(x)[t] == forward(x[t]), as
// in trait_.rs:78-109).  Otherwise the aarch64 kernel's order on the matrix cores, equally batch-independent: the
// small-batch kernel while the tokens fit its LDS staging, the tiled GEMM for more.
static int forward_batched(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in, uint32_t n_out,
                           uint32_t n_tokens, int rounding, int mode) {
    // FAST: up to 8 tokens the GEMV (one launch, the x86-64 order); beyond, the matrix cores
    const bool x86_order = mode == RMI_HIP_BATCHED_X86_ORDER || (mode == RMI_HIP_BATCHED_FAST && n_tokens <= 8);
    const bool fast = mode == RMI_HIP_BATCHED_FAST;
    RMI_REQUIRE_INIT();
    int rc = check_q8(w, n_in, n_out);
    if (rc != RMI_HIP_OK) return rc;
    if (n_tokens == 0 || n_out == 0) return RMI_HIP_OK;
    if (!input || !output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const size_t n_x = size_t(n_tokens) * n_in;
    float *pin = static_cast<float *>(rmi_pin_buf(c, 0, n_x * 4));
    float *d_x = static_cast<float *>(rmi_dev_buf(c, 0, n_x * 4));
    int8_t *d_q8 = static_cast<int8_t *>(rmi_dev_buf(c, 2, n_x));
    float *d_sc = static_cast<float *>(rmi_dev_buf(c, 3, n_x / 32 * 4));
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, size_t(n_tokens) * n_out * 4));
    if (!pin || !d_x || !d_q8 || !d_sc || !d_y) return RMI_HIP_E_RUNTIME;
    memcpy(pin, input, n_x * 4);
    RMI_HIP_CHECK(hipMemcpyAsync(d_x, pin, n_x * 4, hipMemcpyHostToDevice, c->stream));
    rc = rmi_launch_quantize_q8_0(d_x, d_q8, d_sc, n_tokens, n_in, rounding, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    // (measured per launch: the small-batch kernel is level with the GEMM or ahead up to 16 tokens for any matrix
    // and up to 32 for one of lm_head's size; the GEMM leads from 17 tokens on for matrices of a few MB)
    const bool small_batch = n_tokens <= 16 || (n_tokens <= 32 && w->n_tiles >= 4096);
    if (x86_order)
        rc = rmi_gemv_q8_0_tokens(w, d_q8, d_sc, d_y, n_tokens, n_out, 0, n_out, c->stream);
    else if (small_batch && rmi_gemv_q8_0_mfma_fits(n_tokens, w->n_units))
        rc = mfma_tokens(w, d_q8, d_sc, d_y, n_tokens, n_out, 0, n_out, c->stream);
    else if (n_tokens >= kGemmMinTokens && fast)
        rc = rmi_hip_gemm_q8_0_fast_dev(w, d_q8, d_sc, d_y, n_tokens, n_out, c->stream);
    else if (n_tokens >= kGemmMinTokens)
        rc = rmi_launch_gemm_q8_0(w, d_q8, d_sc, d_y, n_tokens, n_out, c->stream);
    else {  // up to 15 tokens of a row too long for that: the same kernel, as many tokens at a time as fit
        uint32_t chunk = n_tokens;
        while (chunk > 0 && !rmi_gemv_q8_0_mfma_fits(chunk, w->n_units)) chunk--;
        if (chunk == 0) return rmi_fail(RMI_HIP_E_INVALID, "n_in=%u is too long for the small-batch staging", n_in);
        for (uint32_t t0 = 0; t0 < n_tokens && rc == RMI_HIP_OK; t0 += chunk)
            rc = mfma_tokens(w, d_q8 + size_t(t0) * n_in, d_sc + size_t(t0) * (n_in / 32), d_y + size_t(t0) * n_out,
                             n_tokens - t0 < chunk ? n_tokens - t0 : chunk, n_out, 0, n_out, c->stream);
    }
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, output, d_y, size_t(n_tokens) * n_out * 4, 1);
}

int rmi_hip_q8_0_forward_batched(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                 uint32_t n_out, uint32_t n_tokens, int rounding) {
    return forward_batched(w, input, output, n_in, n_out, n_tokens, rounding, rmi_batched_mode());
}

int rmi_hip_q8_0_forward_batched_neon(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                      uint32_t n_out, uint32_t n_tokens, int rounding) {
    return forward_batched(w, input, output, n_in, n_out, n_tokens, rounding, RMI_HIP_BATCHED_AARCH64_ORDER);
}

int rmi_hip_quantize_q8_0(const float *input, uint32_t n, uint8_t *q8, float *scales, int rounding) {
    RMI_REQUIRE_INIT();
    const uint32_t blocks = n / 32;  // a ragged tail is left untouched, as in q8_0.rs:4
    if (blocks == 0) return RMI_HIP_OK;
    if (!input || !q8 || !scales) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const size_t n_x = size_t(blocks) * 32;
    float *pin = static_cast<float *>(rmi_pin_buf(c, 0, n_x * 4));
    float *d_x = static_cast<float *>(rmi_dev_buf(c, 0, n_x * 4));
    const size_t q_bytes = (n_x + 15) & ~size_t(15);
    uint8_t *d_out = static_cast<uint8_t *>(rmi_dev_buf(c, 2, q_bytes + size_t(blocks) * 4));
    if (!pin || !d_x || !d_out) return RMI_HIP_E_RUNTIME;
    memcpy(pin, input, n_x * 4);
    RMI_HIP_CHECK(hipMemcpyAsync(d_x, pin, n_x * 4, hipMemcpyHostToDevice, c->stream));
    int rc = rmi_launch_quantize_q8_0(d_x, reinterpret_cast<int8_t *>(d_out), reinterpret_cast<float *>(d_out + q_bytes),
                                      1, blocks * 32, rounding, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    uint8_t *pout = static_cast<uint8_t *>(rmi_pin_buf(c, 1, q_bytes + size_t(blocks) * 4));
    if (!pout) return RMI_HIP_E_RUNTIME;
    RMI_HIP_CHECK(hipMemcpyAsync(pout, d_out, q_bytes + size_t(blocks) * 4, hipMemcpyDeviceToHost, c->stream));
    RMI_HIP_CHECK(hipStreamSynchronize(c->stream));
    memcpy(q8, pout, n_x);
    memcpy(scales, pout + q_bytes, size_t(blocks) * 4);
    return RMI_HIP_OK;
}

int rmi_hip_block_dots_q8_0(const rmi_hip_weight *w, const uint8_t *input_q8, int32_t *dots) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    const size_t n = size_t(w->n_out) * (w->n_in / 32);
    if (n == 0) return RMI_HIP_OK;
    if (!input_q8 || !dots) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    uint8_t *pin = static_cast<uint8_t *>(rmi_pin_buf(c, 0, w->n_in));
    int8_t *d_x = static_cast<int8_t *>(rmi_dev_buf(c, 0, w->n_in));
    int32_t *d_dots = static_cast<int32_t *>(rmi_dev_buf(c, 1, n * 4));
    if (!pin || !d_x || !d_dots) return RMI_HIP_E_RUNTIME;
    memcpy(pin, input_q8, w->n_in);
    RMI_HIP_CHECK(hipMemcpyAsync(d_x, pin, w->n_in, hipMemcpyHostToDevice, c->stream));
    int rc = rmi_launch_block_dots_q8_0(w, d_x, d_dots, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, dots, d_dots, n * 4, 1);
}

int rmi_hip_matmul_q8_0_f32(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in, uint32_t n_out) {
    RMI_REQUIRE_INIT();
    int rc = check_q8(w, n_in, n_out);
    if (rc != RMI_HIP_OK) return rc;
    if (n_out == 0) return RMI_HIP_OK;
    if (!input || !output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    float *pin = static_cast<float *>(rmi_pin_buf(c, 0, size_t(n_in) * 4));
    float *d_x = static_cast<float *>(rmi_dev_buf(c, 0, size_t(n_in) * 4));
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, size_t(n_out) * 4));
    if (!pin || !d_x || !d_y) return RMI_HIP_E_RUNTIME;
    memcpy(pin, input, size_t(n_in) * 4);
    RMI_HIP_CHECK(hipMemcpyAsync(d_x, pin, size_t(n_in) * 4, hipMemcpyHostToDevice, c->stream));
    rc = rmi_launch_matmul_q8_0_f32(w, d_x, d_y, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, output, d_y, size_t(n_out) * 4, 1);
}

int rmi_hip_matmul_q8_0_fallback_range(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                       uint32_t row_start, uint32_t row_end) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (n_in != w->n_in) return rmi_fail(RMI_HIP_E_INVALID, "n_in=%u, the weight has %u", n_in, w->n_in);
    if (row_start > row_end || row_end > w->n_out)
        return rmi_fail(RMI_HIP_E_INVALID, "rows [%u,%u) outside 0..%u", row_start, row_end, w->n_out);
    if (row_end == row_start) return RMI_HIP_OK;
    if (!input || !output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const size_t n_rows = row_end - row_start;
    float *pin = static_cast<float *>(rmi_pin_buf(c, 0, size_t(n_in) * 4));
    float *d_x = static_cast<float *>(rmi_dev_buf(c, 0, size_t(n_in) * 4));
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, n_rows * 4));
    if (!pin || !d_x || !d_y) return RMI_HIP_E_RUNTIME;
    memcpy(pin, input, size_t(n_in) * 4);
    RMI_HIP_CHECK(hipMemcpyAsync(d_x, pin, size_t(n_in) * 4, hipMemcpyHostToDevice, c->stream));
    int rc = rmi_launch_matmul_q8_0_f32_scalar(w, d_x, d_y, row_start, row_end, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, output, d_y, n_rows * 4, 1);
}

// ------------------------------------------------------ device-resident

int rmi_hip_gemv_q8_0_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                          uint32_t n_tokens, uint32_t y_stride, uint32_t row_start, uint32_t row_end, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (row_start >= row_end || n_tokens == 0) return RMI_HIP_OK;
    if (row_end > w->n_out) return rmi_fail(RMI_HIP_E_INVALID, "rows [%u,%u) exceed n_out=%u", row_start, row_end, w->n_out);
    if (y_stride < row_end && n_tokens > 1) return rmi_fail(RMI_HIP_E_INVALID, "y_stride=%u < row_end=%u", y_stride, row_end);
    if (!x_q8 || !x_scales || !y) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    if (rmi_misaligned(x_q8, x_scales, y)) return rmi_fail(RMI_HIP_E_INVALID, RMI_ALIGNMENT_MESSAGE);
    return rmi_gemv_q8_0_tokens(w, x_q8, x_scales, y, n_tokens, y_stride, row_start, row_end, static_cast<hipStream_t>(stream));
}

int rmi_hip_gemv_q8_0_neon_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                               uint32_t n_tokens, uint32_t y_stride, uint32_t row_start, uint32_t row_end, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (row_start >= row_end || n_tokens == 0) return RMI_HIP_OK;
    if (row_end > w->n_out) return rmi_fail(RMI_HIP_E_INVALID, "rows [%u,%u) exceed n_out=%u", row_start, row_end, w->n_out);
    if (y_stride < row_end && n_tokens > 1) return rmi_fail(RMI_HIP_E_INVALID, "y_stride=%u < row_end=%u", y_stride, row_end);
    if (!x_q8 || !x_scales || !y) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    if (rmi_misaligned(x_q8, x_scales, y)) return rmi_fail(RMI_HIP_E_INVALID, RMI_ALIGNMENT_MESSAGE);
    if (!rmi_gemv_q8_0_mfma_fits(n_tokens, w->n_units))
        return rmi_fail(RMI_HIP_E_INVALID, "%u tokens x %u elements: at most %u tokens whose activations fit the LDS staging",
                        n_tokens, w->n_in, kMfmaMaxTokens);
    return mfma_tokens(w, x_q8, x_scales, y, n_tokens, y_stride, row_start, row_end, static_cast<hipStream_t>(stream));
}

int rmi_hip_quantize_q8_0_dev(const float *x, int8_t *q8, float *scales, uint32_t n_tokens, uint32_t n_in,
                              int rounding, void *stream) {
    RMI_REQUIRE_INIT();
    if (n_in % 32 != 0) return rmi_fail(RMI_HIP_E_INVALID, "n_in=%u is not a multiple of 32", n_in);
    if (!x || !q8 || !scales) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    return rmi_launch_quantize_q8_0(x, q8, scales, n_tokens, n_in, rounding, static_cast<hipStream_t>(stream));
}

int rmi_hip_gemm_q8_0_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                          uint32_t n_tokens, uint32_t y_stride, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    if (y_stride < w->n_out) return rmi_fail(RMI_HIP_E_INVALID, "y_stride=%u < n_out=%u", y_stride, w->n_out);
    if (!x_q8 || !x_scales || !y) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    if (rmi_misaligned(x_q8, x_scales, y)) return rmi_fail(RMI_HIP_E_INVALID, RMI_ALIGNMENT_MESSAGE);
    return rmi_launch_gemm_q8_0(w, x_q8, x_scales, y, n_tokens, y_stride, static_cast<hipStream_t>(stream));
}

int rmi_hip_gemm_q8_0_ksplit_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                                 uint32_t n_tokens, uint32_t y_stride, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    if (y_stride < w->n_out) return rmi_fail(RMI_HIP_E_INVALID, "y_stride=%u < n_out=%u", y_stride, w->n_out);
    if (!x_q8 || !x_scales || !y) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    if (rmi_misaligned(x_q8, x_scales, y)) return rmi_fail(RMI_HIP_E_INVALID, RMI_ALIGNMENT_MESSAGE);
    return rmi_launch_gemm_q8_0_ksplit(w, x_q8, x_scales, y, n_tokens, y_stride, static_cast<hipStream_t>(stream));
}

// which kernel rmi_hip_gemm_q8_0_fast_dev takes for this product, and how it cuts the chain
static int fast_plan(const rmi_hip_weight *w, uint32_t n_tokens, uint32_t *param) {
    uint32_t groups = 1;
    const double tiled = rmi_gemm_q8_0_cost_us(w, n_tokens, false, &groups);
    if (tiled < 0.0 || (!rmi_gemm_q8_0_shape_forced() && rmi_gemm_q8_0_ksplit_cost_us(w, n_tokens) < tiled)) {
        uint32_t per = 1, n_waves = 1;
        rmi_gemm_q8_0_ksplit_shape(w->n_in, &per, &n_waves);
        *param = per;
        return RMI_HIP_GEMM_PLAN_KSPLIT;
    }
    *param = groups;
    return groups > 1 ? RMI_HIP_GEMM_PLAN_TILED_GROUPS : RMI_HIP_GEMM_PLAN_TILED_SINGLE_CHAIN;
}

int rmi_hip_gemm_q8_0_fast_plan(const rmi_hip_weight *w, uint32_t n_tokens, uint32_t *param) {
    uint32_t dummy = 0;
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0 || n_tokens == 0 || w->n_out == 0 || w->n_in < 32) {
        if (param) *param = 1;
        return RMI_HIP_GEMM_PLAN_TILED_SINGLE_CHAIN;
    }
    return fast_plan(w, n_tokens, param ? param : &dummy);
}

int rmi_hip_gemm_q8_0_fast_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                               uint32_t n_tokens, uint32_t y_stride, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q8_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q8_0 weight handle");
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    if (y_stride < w->n_out) return rmi_fail(RMI_HIP_E_INVALID, "y_stride=%u < n_out=%u", y_stride, w->n_out);
    if (!x_q8 || !x_scales || !y) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    if (rmi_misaligned(x_q8, x_scales, y)) return rmi_fail(RMI_HIP_E_INVALID, RMI_ALIGNMENT_MESSAGE);
    if (w->n_in < 32) return rmi_fail(RMI_HIP_E_INVALID, "GEMM needs at least one block per row");
    uint32_t param = 1;
    if (fast_plan(w, n_tokens, &param) == RMI_HIP_GEMM_PLAN_KSPLIT)
        return rmi_launch_gemm_q8_0_ksplit(w, x_q8, x_scales, y, n_tokens, y_stride, static_cast<hipStream_t>(stream));
    return rmi_launch_gemm_q8_0_grouped(w, x_q8, x_scales, y, n_tokens, y_stride, static_cast<hipStream_t>(stream));
}

uint32_t rmi_hip_gemm_q8_0_ksplit_quads_per_part(uint32_t n_in) {
    uint32_t per = 1, n_waves = 1;
    rmi_gemm_q8_0_ksplit_shape(n_in, &per, &n_waves);
    return per;
}

int rmi_hip_copy_dev(void *dst, const void *src, size_t nbytes, void *stream) {
    RMI_REQUIRE_INIT();
    if (!dst || !src || nbytes % 16 != 0) return rmi_fail(RMI_HIP_E_INVALID, "copy needs non-null pointers and a multiple of 16 bytes");
    return rmi_launch_copy(src, dst, nbytes, static_cast<hipStream_t>(stream));
}

static rmi_hip_gemv_group *group_create_q8_0(uint32_t n_problems, const rmi_hip_weight *const *weights,
                                             const int8_t *const *x_q8, const float *const *x_scales, float *const *y,
                                             uint32_t n_tokens, bool mfma) {
    if (!rmi_ready()) {
        rmi_set_error("rmi_hip_init has not succeeded");
        return nullptr;
    }
    const uint32_t max_tokens = mfma ? kMfmaMaxTokens : 8;
    if (n_problems == 0 || n_tokens == 0 || n_tokens > max_tokens || !weights || !x_q8 || !x_scales || !y) {
        rmi_set_error("gemv group needs >=1 problem and 1..%u tokens", max_tokens);
        return nullptr;
    }
    if (!rmi_thread_ctx()) return nullptr;
    std::vector<RmiGemvProblem> list(n_problems);
    rmi_hip_gemv_group *g = new rmi_hip_gemv_group();
    // Q8_0 weights, or Q4_0 weights (the same Q8_0 activations); one type per group
    g->dtype = !mfma && weights[0] && weights[0]->dtype == RMI_HIP_DTYPE_Q4_0 ? RMI_HIP_DTYPE_Q4_0 : RMI_HIP_DTYPE_Q8_0;
    g->mfma = mfma;
    const size_t oct_bytes = g->dtype == RMI_HIP_DTYPE_Q4_0 ? kQ40OctetBytes : kOctetBytes;
    const size_t lds_per_oct = g->dtype == RMI_HIP_DTYPE_Q4_0 ? 320 : 288;  // staged activation, per token and octet
    g->n_problems = n_problems;
    g->n_tokens = n_tokens;
    uint64_t total_tiles = 0;
    for (uint32_t i = 0; i < n_problems; i++) {
        const rmi_hip_weight *w = weights[i];
        if (!w || w->dtype != g->dtype || !x_q8[i] || !x_scales[i] || !y[i]) {
            rmi_set_error("gemv group problem %u: bad weight handle or null pointer", i);
            delete g;
            return nullptr;
        }
        if (rmi_misaligned(x_q8[i], x_scales[i], y[i])) {
            rmi_set_error("gemv group problem %u: " RMI_ALIGNMENT_MESSAGE, i);
            delete g;
            return nullptr;
        }
        list[i] = make_problem(w, x_q8[i], x_scales[i], y[i], w->n_out, 0, w->n_out);
        total_tiles += list[i].n_tiles;
        if (w->n_units > g->max_units) g->max_units = w->n_units;
    }
    const size_t lds_bytes = mfma ? rmi_gemv_q8_0_mfma_lds_bytes(n_tokens, g->max_units)
                                  : size_t(n_tokens) * g->max_units * lds_per_oct;
    if (total_tiles > 0x7fffffffull || (mfma ? !rmi_gemv_q8_0_mfma_fits(n_tokens, g->max_units) : lds_bytes > 64 * 1024)) {
        rmi_set_error("gemv group too large (%llu tiles, %u tokens x %u octets)", (unsigned long long)total_tiles,
                      n_tokens, g->max_units);
        delete g;
        return nullptr;
    }
    // one run of consecutive tiles per wave, never across two matrices; the waves of a workgroup share a matrix
    auto tiles_per_wave = [&](uint32_t n_oct) {
        return mfma ? mfma_tiles_per_wave(n_oct, uint32_t(total_tiles), n_tokens)
                    : rmi_gemv_tiles_per_wave(n_oct, uint32_t(total_tiles), n_tokens);
    };
    g->wpg = rmi_gemv_waves_per_group(lds_bytes, size_t(tiles_per_wave(g->max_units)) * g->max_units * oct_bytes);
    // the kernel for four tokens and more holds four waves a SIMD at most (registers): with workgroups of four waves
    // a compute unit turns them over one at a time instead of in halves (measured at 8 tokens: 4.53 -> 4.76 TB/s)
    if (!mfma && g->dtype == RMI_HIP_DTYPE_Q8_0 && n_tokens >= 4 && g->wpg > 4) g->wpg = 4;
    std::vector<uint4> runs;
    for (uint32_t i = 0; i < n_problems; i++) {
        if (list[i].n_oct == 0) continue;
        const uint32_t tpw = tiles_per_wave(list[i].n_oct);
        for (uint32_t k = 0; k < list[i].n_tiles; k += tpw)
            runs.push_back(make_uint4(i, k, list[i].n_tiles - k < tpw ? list[i].n_tiles - k : tpw, 0));
        while (runs.size() % g->wpg) runs.push_back(make_uint4(i, 0, 0, 0));
    }
    g->n_runs = uint32_t(runs.size());
    hipError_t e = hipMalloc(&g->d_list, sizeof(RmiGemvProblem) * n_problems);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&g->d_runs), sizeof(uint4) * (runs.size() + 1));
    if (e == hipSuccess)
        e = hipMemcpy(g->d_list, list.data(), sizeof(RmiGemvProblem) * n_problems, hipMemcpyHostToDevice);
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

rmi_hip_gemv_group *rmi_hip_gemv_group_create(uint32_t n_problems, const rmi_hip_weight *const *weights,
                                              const int8_t *const *x_q8, const float *const *x_scales,
                                              float *const *y, uint32_t n_tokens) {
    return group_create_q8_0(n_problems, weights, x_q8, x_scales, y, n_tokens, false);
}

rmi_hip_gemv_group *rmi_hip_gemv_group_create_neon(uint32_t n_problems, const rmi_hip_weight *const *weights,
                                                   const int8_t *const *x_q8, const float *const *x_scales,
                                                   float *const *y, uint32_t n_tokens) {
    return group_create_q8_0(n_problems, weights, x_q8, x_scales, y, n_tokens, true);
}

int rmi_hip_gemv_group_shape(const rmi_hip_gemv_group *g, uint32_t *n_workgroups, uint32_t *waves_per_workgroup) {
    if (!g) return rmi_fail(RMI_HIP_E_INVALID, "null gemv group");
    if (n_workgroups) *n_workgroups = g->n_runs / g->wpg;
    if (waves_per_workgroup) *waves_per_workgroup = g->wpg;
    return RMI_HIP_OK;
}

void rmi_hip_gemv_group_destroy(rmi_hip_gemv_group *g) {
    if (!g) return;
    if (g->d_list) (void)hipFree(g->d_list);
    if (g->d_runs) (void)hipFree(g->d_runs);
    delete g;
}

int rmi_hip_gemv_group_run_dev(const rmi_hip_gemv_group *g, void *stream) {
    RMI_REQUIRE_INIT();
    if (!g) return rmi_fail(RMI_HIP_E_INVALID, "null group");
    if (g->dtype == RMI_HIP_DTYPE_Q6_K)
        return rmi_launch_gemv_q6_k_group(static_cast<const RmiQ4kProblem *>(g->d_list), g->d_runs, g->n_runs,
                                          g->wpg, g->max_units, g->n_tokens, static_cast<hipStream_t>(stream));
    if (g->dtype == RMI_HIP_DTYPE_Q4_K)
        return rmi_launch_gemv_q4_k_group(static_cast<const RmiQ4kProblem *>(g->d_list), g->d_runs, g->n_runs,
                                          g->wpg, g->max_units, g->n_tokens, static_cast<hipStream_t>(stream));
    if (g->dtype == RMI_HIP_DTYPE_Q4_0)
        return rmi_launch_gemv_q4_0_group(static_cast<const RmiGemvProblem *>(g->d_list), g->d_runs, g->n_runs,
                                          g->wpg, g->max_units, g->n_tokens, static_cast<hipStream_t>(stream));
    if (g->mfma)
        return rmi_launch_gemv_q8_0_mfma(nullptr, static_cast<const RmiGemvProblem *>(g->d_list), g->d_runs, g->n_runs,
                                         g->wpg, 0, g->max_units, g->n_tokens, static_cast<hipStream_t>(stream));
    return rmi_launch_gemv_q8_0_group(static_cast<const RmiGemvProblem *>(g->d_list), g->d_runs, g->n_runs,
                                      g->wpg, g->max_units, g->n_tokens, static_cast<hipStream_t>(stream));
}

// ---- Q4_0 weights (Q8_0 activations): the same staging and row partition as the Q8_0 calls

int rmi_hip_q4_0_forward_prequantized(const rmi_hip_weight *w, const uint8_t *input_q8, const float *input_scales,
                                      float *output, uint32_t n_in, uint32_t n_out, uint32_t ith, uint32_t nth) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q4_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q4_0 weight handle");
    if (w->n_in != n_in || w->n_out != n_out)
        return rmi_fail(RMI_HIP_E_INVALID, "weight is %u x %u, call says %u x %u", w->n_out, w->n_in, n_out, n_in);
    if (nth == 0) nth = 1;
    if (n_out == 0) return RMI_HIP_OK;
    const uint32_t per_thread = (n_out + nth - 1) / nth;  // q4_0/mod.rs:46-51
    const uint64_t s64 = uint64_t(ith) * per_thread;
    if (s64 >= n_out) return RMI_HIP_OK;
    const uint32_t start = uint32_t(s64), end = start + per_thread < n_out ? start + per_thread : n_out;
    if (!output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    return host_gemv_range(w, input_q8, input_scales, output + start, 1, end - start, start, end);
}

int rmi_hip_q4_0_forward_batched(const rmi_hip_weight *w, const float *input, float *output, uint32_t n_in,
                                 uint32_t n_out, uint32_t n_tokens, int rounding) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q4_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q4_0 weight handle");
    if (w->n_in != n_in || w->n_out != n_out)
        return rmi_fail(RMI_HIP_E_INVALID, "weight is %u x %u, call says %u x %u", w->n_out, w->n_in, n_out, n_in);
    if (n_tokens == 0 || n_out == 0) return RMI_HIP_OK;
    if (!input || !output) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    const size_t n_x = size_t(n_tokens) * n_in;
    float *pin = static_cast<float *>(rmi_pin_buf(c, 2, n_x * 4));
    float *d_x = static_cast<float *>(rmi_dev_buf(c, 2, n_x * 4));
    int8_t *d_q8 = static_cast<int8_t *>(rmi_dev_buf(c, 0, n_x));
    float *d_sc = static_cast<float *>(rmi_dev_buf(c, 3, n_x / 32 * 4));
    float *d_y = static_cast<float *>(rmi_dev_buf(c, 1, size_t(n_tokens) * n_out * 4));
    if (!pin || !d_x || !d_q8 || !d_sc || !d_y) return RMI_HIP_E_RUNTIME;
    memcpy(pin, input, n_x * 4);
    RMI_HIP_CHECK(hipMemcpyAsync(d_x, pin, n_x * 4, hipMemcpyHostToDevice, c->stream));
    int rc = rmi_launch_quantize_q8_0(d_x, d_q8, d_sc, n_tokens, n_in, rounding, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    rc = rmi_gemv_q8_0_tokens(w, d_q8, d_sc, d_y, n_tokens, n_out, 0, n_out, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, output, d_y, size_t(n_tokens) * n_out * 4, 1);
}

int rmi_hip_block_dots_q4_0(const rmi_hip_weight *w, const uint8_t *input_q8, int32_t *dots) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q4_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q4_0 weight handle");
    const size_t n = size_t(w->n_out) * (w->n_in / 32);
    if (n == 0) return RMI_HIP_OK;
    if (!input_q8 || !dots) return rmi_fail(RMI_HIP_E_INVALID, "null slice");
    RmiThreadCtx *c = rmi_thread_ctx();
    if (!c) return RMI_HIP_E_RUNTIME;
    uint8_t *pin = static_cast<uint8_t *>(rmi_pin_buf(c, 0, w->n_in));
    int8_t *d_q8 = static_cast<int8_t *>(rmi_dev_buf(c, 0, w->n_in));
    int32_t *d_out = static_cast<int32_t *>(rmi_dev_buf(c, 1, n * 4));
    if (!pin || !d_q8 || !d_out) return RMI_HIP_E_RUNTIME;
    memcpy(pin, input_q8, w->n_in);
    RMI_HIP_CHECK(hipMemcpyAsync(d_q8, pin, w->n_in, hipMemcpyHostToDevice, c->stream));
    int rc = rmi_launch_block_dots_q4_0(w, d_q8, d_out, c->stream);
    if (rc != RMI_HIP_OK) return rc;
    return fetch(c, dots, d_out, n * 4, 1);
}

int rmi_hip_gemv_q4_0_dev(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                          uint32_t n_tokens, uint32_t y_stride, uint32_t row_start, uint32_t row_end, void *stream) {
    RMI_REQUIRE_INIT();
    if (!w || w->dtype != RMI_HIP_DTYPE_Q4_0) return rmi_fail(RMI_HIP_E_INVALID, "not a Q4_0 weight handle");
    if (row_start >= row_end || n_tokens == 0) return RMI_HIP_OK;
    if (row_end > w->n_out) return rmi_fail(RMI_HIP_E_INVALID, "rows [%u,%u) exceed n_out=%u", row_start, row_end, w->n_out);
    if (y_stride < row_end && n_tokens > 1) return rmi_fail(RMI_HIP_E_INVALID, "y_stride=%u < row_end=%u", y_stride, row_end);
    if (!x_q8 || !x_scales || !y) return rmi_fail(RMI_HIP_E_INVALID, "null device pointer");
    if (rmi_misaligned(x_q8, x_scales, y)) return rmi_fail(RMI_HIP_E_INVALID, RMI_ALIGNMENT_MESSAGE);
    return rmi_gemv_q8_0_tokens(w, x_q8, x_scales, y, n_tokens, y_stride, row_start, row_end, static_cast<hipStream_t>(stream));
}

}  // extern "C"
