// Q8_0 x Q8_0 prefill GEMM on int8 MFMA: Y[t][n] = sum_b (f32(wd[n][b]) * xs[t][b]) * dot_b(W[n], X[t]).
//
// One 32x32x32 MFMA is one Q8_0 block (K = 32) of a 32-token x 32-row tile, so
// the int32 accumulator is the per-block dot and starts from zero every block.
// f32 order: acc = fma(float(dot), wd*xs, acc), blocks in sequence — the order
// of matmul_q8_0_vs_q8_0_neon (src/ops/kernel/q8_0/neon.rs:49-73).
//
// Operands come straight from the GEMV tile stream.  MFMA lane (c, h) supplies
// 16 of the 32 k values of its row/column; which 16 is free as long as both
// operands agree.  A weight lane loads the 64 contiguous bytes that hold the
// slices L = 4h..4h+3 of its row's quad (4 blocks): dword j of each of the four
// 16-byte pieces is k = 16h+4L'..+3 of block j, which is exactly bytes
// 16h..16h+15 of that block in the natural activation layout.
#include "rmi_internal.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kTT = 2;  // 32-token sub-tiles per wave

__device__ __forceinline__ float h2f(uint32_t bits16) {
    return float(__builtin_bit_cast(_Float16, uint16_t(bits16)));
}

// grid.x = ceil(n_out/32), grid.y = ceil(n_tokens/64); one wave per workgroup.
__global__ __launch_bounds__(64) void gemm_q8_0_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ x_q8,
                                                        const float *__restrict__ x_scales, float *__restrict__ y,
                                                        uint32_t n_out, uint32_t n_in, uint32_t n_oct, uint32_t n_tiles,
                                                        uint32_t n_tokens, uint32_t y_stride) {
    extern __shared__ float lds_xs[];  // [block][tt][h][16] activation scales of this wave's 64 tokens
    const uint32_t lane = threadIdx.x, c = lane & 31, h = lane >> 5;
    const uint32_t n0 = blockIdx.x * 32, t0 = blockIdx.y * 64;
    const uint32_t nb = n_in >> 5;

    // stage xs: element (b, tt, h', i) = xs[t0 + 32tt + 8(i/4) + 4h' + i%4][b]
    for (uint32_t idx = lane; idx < nb * 64; idx += 64) {
        const uint32_t b = idx >> 6, rem = idx & 63;
        const uint32_t tt = rem >> 5, hh = (rem >> 4) & 1, i = rem & 15;
        const uint32_t t = t0 + 32 * tt + 8 * (i >> 2) + 4 * hh + (i & 3);
        lds_xs[idx] = t < n_tokens ? x_scales[size_t(t) * nb + b] : 0.0f;
    }
    __syncthreads();

    // this lane's weight row (column of the MFMA) and token rows
    const uint32_t n = n0 + c;
    uint32_t wtile = n >> 3;
    if (wtile >= n_tiles) wtile = n_tiles - 1;  // rows past the padded stream: loads stay in bounds, stores are masked
    const uint8_t *tile = w + size_t(wtile) * n_oct * kOctetBytes;
    const uint8_t *wq = tile + size_t(n_oct) * 128 + (n & 7) * 128 + h * 64;
    const uint8_t *wsc = tile + (n & 7) * 16;
    const int8_t *xrow[kTT];
    bool xok[kTT];
#pragma unroll
    for (int tt = 0; tt < kTT; tt++) {
        const uint32_t t = t0 + 32 * tt + c;
        xok[tt] = t < n_tokens;
        xrow[tt] = x_q8 + size_t(xok[tt] ? t : 0) * n_in + 16 * h;
    }

    float acc[kTT][16];
#pragma unroll
    for (int tt = 0; tt < kTT; tt++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[tt][i] = 0.0f;

    const uint32_t n_quads = (nb + 3) >> 2;
    for (uint32_t q = 0; q < n_quads; q++) {
        const uint4 *wp = reinterpret_cast<const uint4 *>(wq + size_t(q) * 1024);
        const uint4 u0 = wp[0], u1 = wp[1], u2 = wp[2], u3 = wp[3];
        const uint2 sc = *reinterpret_cast<const uint2 *>(wsc + size_t(q >> 1) * 128 + (q & 1) * 8);
        const float wd[4] = {h2f(sc.x & 0xffffu), h2f(sc.x >> 16), h2f(sc.y & 0xffffu), h2f(sc.y >> 16)};
        const v4i wj[4] = {v4i{int(u0.x), int(u1.x), int(u2.x), int(u3.x)}, v4i{int(u0.y), int(u1.y), int(u2.y), int(u3.y)},
                           v4i{int(u0.z), int(u1.z), int(u2.z), int(u3.z)}, v4i{int(u0.w), int(u1.w), int(u2.w), int(u3.w)}};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t b = q * 4 + j;
            if (b < nb) {
#pragma unroll
                for (int tt = 0; tt < kTT; tt++) {
                    uint4 xv = make_uint4(0, 0, 0, 0);
                    if (xok[tt]) xv = *reinterpret_cast<const uint4 *>(xrow[tt] + size_t(b) * 32);
                    const v4i a = v4i{int(xv.x), int(xv.y), int(xv.z), int(xv.w)};
                    v16i d = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    d = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, wj[j], d, 0, 0, 0);
                    const float4 *xs4 = reinterpret_cast<const float4 *>(lds_xs + ((b * kTT + tt) * 2 + h) * 16);
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const float4 s = xs4[g];
                        acc[tt][4 * g + 0] = __builtin_fmaf(float(d[4 * g + 0]), wd[j] * s.x, acc[tt][4 * g + 0]);
                        acc[tt][4 * g + 1] = __builtin_fmaf(float(d[4 * g + 1]), wd[j] * s.y, acc[tt][4 * g + 1]);
                        acc[tt][4 * g + 2] = __builtin_fmaf(float(d[4 * g + 2]), wd[j] * s.z, acc[tt][4 * g + 2]);
                        acc[tt][4 * g + 3] = __builtin_fmaf(float(d[4 * g + 3]), wd[j] * s.w, acc[tt][4 * g + 3]);
                    }
                }
            }
        }
    }

    if (n < n_out) {
#pragma unroll
        for (int tt = 0; tt < kTT; tt++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t t = t0 + 32 * tt + 8 * (i >> 2) + 4 * h + (i & 3);
                if (t < n_tokens) y[size_t(t) * y_stride + n] = acc[tt][i];
            }
    }
}

}  // namespace

int rmi_launch_gemm_q8_0(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                         uint32_t n_tokens, uint32_t y_stride, hipStream_t s) {
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    const size_t lds_bytes = size_t(w->n_in / 32) * 64 * 4;
    if (lds_bytes > 64 * 1024) return rmi_fail(RMI_HIP_E_INVALID, "n_in=%u is too long for the GEMM scale staging", w->n_in);
    dim3 grid((w->n_out + 31) / 32, (n_tokens + 63) / 64);
    hipLaunchKernelGGL(gemm_q8_0_kernel, grid, dim3(64), lds_bytes, s, w->data, x_q8, x_scales, y, w->n_out, w->n_in,
                       w->n_units, w->n_tiles, n_tokens, y_stride);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
