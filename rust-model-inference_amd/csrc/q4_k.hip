// Q4_K kernels: the Q8_K activation quantizer, the Q4_K x Q8_K integer GEMV,
// its exact per-super-block integers, and the dequantise-and-dot paths.
//
// GEMV arithmetic order = vec_dot_q4k_q8k_avx2 (src/ops/quant/mod.rs:701-799):
// per row eight f32 accumulators (lane T sums the 4-element groups k=4T..4T+3
// of every 32-element sub-block, scale-weighted, as one int32 per super-block,
// then acc_T = fma(d*q8d, float(sumi_T), acc_T)) and four min accumulators
// (acc_m[t] = fma(-dmin*q8d, float(mn[2t]*s[2t] + mn[2t+1]*s[2t+1]), acc_m[t]));
// result hsum(acc) + ((m0+m2)+(m1+m3)).  Eight GPU lanes per row hold them.
#include "rmi_internal.h"

namespace {

__device__ __forceinline__ float h2f(uint32_t bits16) {
    return float(__builtin_bit_cast(_Float16, uint16_t(bits16)));
}

__device__ __forceinline__ float hsum8_lanes(float a) {
    a = a + __shfl_xor(a, 4, 64);
    a = a + __shfl_xor(a, 1, 64);
    a = a + __shfl_xor(a, 2, 64);
    return a;
}

// the kmask unpack of quant/mod.rs:237-258: sm.x,.y = 8 scales, sm.z,.w = 8 mins
__device__ __forceinline__ uint4 unpack_scales(uint32_t u0, uint32_t u1, uint32_t u2) {
    const uint32_t kmask1 = 0x3f3f3f3fu, kmask2 = 0x0f0f0f0fu, kmask3 = 0x03030303u;
    uint4 o;
    o.w = ((u2 >> 4) & kmask2) | (((u1 >> 6) & kmask3) << 4);
    o.z = u1 & kmask1;
    o.y = (u2 & kmask2) | (((u0 >> 6) & kmask3) << 4);
    o.x = u0 & kmask1;
    return o;
}

__device__ __forceinline__ uint32_t byte_of(uint32_t lo, uint32_t hi, uint32_t j) {
    const uint32_t wsel = j < 4 ? lo : hi;
    return (wsel >> (8 * (j & 3))) & 0xffu;
}

// ---- quantize_row_q8_k: one wave per 256-element block, lane l owns 4l..4l+3
__global__ __launch_bounds__(64) void quantize_q8_k_kernel(const float *__restrict__ x, float *__restrict__ d,
                                                            int8_t *__restrict__ qs, int16_t *__restrict__ bsums) {
    const uint32_t blk = blockIdx.x, lane = threadIdx.x;
    const float4 v = reinterpret_cast<const float4 *>(x)[size_t(blk) * 64 + lane];
    const float e[4] = {v.x, v.y, v.z, v.w};
    // first element with the strictly largest magnitude keeps its sign (mod.rs:148-152)
    float amax = 0.0f, maxv = 0.0f;
    uint32_t src = lane * 4;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float ax = fabsf(e[j]);
        if (ax > amax) {
            amax = ax;
            maxv = e[j];
            src = lane * 4 + j;
        }
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float oa = __shfl_xor(amax, off, 64);
        const float ov = __shfl_xor(maxv, off, 64);
        const uint32_t os = __shfl_xor(src, off, 64);
        if (oa > amax || (oa == amax && os < src)) {
            amax = oa;
            maxv = ov;
            src = os;
        }
    }
    int q[4] = {0, 0, 0, 0};
    float dd = 0.0f;
    if (amax != 0.0f) {
        const float iscale = -127.0f / maxv;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int r = int(rintf(e[j] * iscale));
            q[j] = r < -127 ? -127 : (r > 127 ? 127 : r);
        }
        dd = 1.0f / iscale;
    }
    reinterpret_cast<uint32_t *>(qs)[size_t(blk) * 64 + lane] =
        uint32_t(q[0] & 0xff) | (uint32_t(q[1] & 0xff) << 8) | (uint32_t(q[2] & 0xff) << 16) | (uint32_t(q[3] & 0xff) << 24);
    int s = q[0] + q[1] + q[2] + q[3];
    s += __shfl_xor(s, 1, 64);
    s += __shfl_xor(s, 2, 64);
    if ((lane & 3) == 0) bsums[size_t(blk) * 16 + (lane >> 2)] = int16_t(s);
    if (lane == 0) d[blk] = dd;
}

// LDS per token and super-block: 64 dwords of quants ordered [T][g][lo,hi],
// 8 dwords of pair sums s_j = bsums[2j]+bsums[2j+1] (i16 wrap, as _mm_hadd_epi16),
// 1 dword d (+3 pad) = 76 dwords.
constexpr uint32_t kSbDwords = 76;

template <int B>
__global__ __launch_bounds__(64) void gemv_q4_k_kernel(const uint8_t *__restrict__ w, const float *__restrict__ q8d,
                                                        const int8_t *__restrict__ q8qs,
                                                        const int16_t *__restrict__ q8bs, float *__restrict__ y,
                                                        uint32_t n_in, uint32_t n_sb, uint32_t y_stride,
                                                        uint32_t row_start, uint32_t row_end, uint32_t tile0,
                                                        uint32_t n_tiles, uint32_t n_waves) {
    extern __shared__ uint4 lds[];
    const uint32_t lane = threadIdx.x, r = lane >> 3, T = lane & 7;
    uint32_t *lds_dw = reinterpret_cast<uint32_t *>(lds);
    for (int t = 0; t < B; t++) {
        uint32_t *dst = lds_dw + size_t(t) * n_sb * kSbDwords;
        const uint32_t *xq = reinterpret_cast<const uint32_t *>(q8qs + size_t(t) * n_in);
        for (uint32_t i = lane; i < n_sb * 64; i += 64) {
            // source dword i of the row: super-block sb, element offset 4*(i%64) = 64g + 32*hi + 4T'
            const uint32_t sb = i >> 6, e = i & 63;
            const uint32_t g = e >> 4, hi = (e >> 3) & 1, tq = e & 7;
            dst[sb * kSbDwords + tq * 8 + g * 2 + hi] = xq[i];
        }
        const int16_t *bs = q8bs + size_t(t) * (n_in / 16);
        for (uint32_t i = lane; i < n_sb * 8; i += 64) {
            const uint32_t sb = i >> 3, j = i & 7;
            const int16_t s = int16_t(bs[sb * 16 + 2 * j] + bs[sb * 16 + 2 * j + 1]);
            dst[sb * kSbDwords + 64 + j] = uint32_t(int32_t(s));
        }
        for (uint32_t i = lane; i < n_sb; i += 64) dst[i * kSbDwords + 72] = __float_as_uint(q8d[size_t(t) * n_sb + i]);
    }
    __syncthreads();

    for (uint32_t k = blockIdx.x; k < n_tiles; k += n_waves) {
        const uint8_t *tile = w + size_t(tile0 + k) * n_sb * kQ4KSuperBytes;
        float acc[B], acc_m[B];
#pragma unroll
        for (int t = 0; t < B; t++) acc[t] = acc_m[t] = 0.0f;
        for (uint32_t sb = 0; sb < n_sb; sb++) {
            const uint8_t *chunk = tile + size_t(sb) * kQ4KSuperBytes;
            const uint4 hdr = reinterpret_cast<const uint4 *>(chunk)[r];
            const uint4 qv = reinterpret_cast<const uint4 *>(chunk + 128)[lane];
            const float wd = h2f(hdr.x & 0xffffu), wdmin = h2f(hdr.x >> 16);
            const uint4 sm = unpack_scales(hdr.y, hdr.z, hdr.w);
            const uint32_t qd[4] = {qv.x, qv.y, qv.z, qv.w};
            const int mn0 = int(byte_of(sm.z, sm.w, (2 * T) & 7)), mn1 = int(byte_of(sm.z, sm.w, (2 * T + 1) & 7));
#pragma unroll
            for (int t = 0; t < B; t++) {
                const uint32_t *xs = lds_dw + (size_t(t) * n_sb + sb) * kSbDwords;
                const uint4 xa = reinterpret_cast<const uint4 *>(xs + T * 8)[0];
                const uint4 xb = reinterpret_cast<const uint4 *>(xs + T * 8)[1];
                const uint32_t xd[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
                int sumi = 0;
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int lo = int(qd[g] & 0x0f0f0f0fu), hi = int((qd[g] >> 4) & 0x0f0f0f0fu);
                    const int dl = __builtin_amdgcn_sdot4(lo, int(xd[2 * g]), 0, false);
                    const int dh = __builtin_amdgcn_sdot4(hi, int(xd[2 * g + 1]), 0, false);
                    sumi += int(byte_of(sm.x, sm.y, 2 * g)) * dl + int(byte_of(sm.x, sm.y, 2 * g + 1)) * dh;
                }
                const float d8 = __uint_as_float(xs[72]);
                const float dd = wd * d8;
                const float dm = (-wdmin) * d8;
                acc[t] = __builtin_fmaf(dd, float(sumi), acc[t]);
                const int s0 = int(xs[64 + ((2 * T) & 7)]), s1 = int(xs[64 + ((2 * T + 1) & 7)]);
                const int prod = mn0 * s0 + mn1 * s1;
                acc_m[t] = __builtin_fmaf(dm, float(prod), acc_m[t]);
            }
        }
        const uint32_t row = (tile0 + k) * kTileRows + r;
#pragma unroll
        for (int t = 0; t < B; t++) {
            const float main_val = hsum8_lanes(acc[t]);
            float m = acc_m[t];  // lanes T<4 hold acc_m[T]
            m = m + __shfl_xor(m, 2, 64);
            m = m + __shfl_xor(m, 1, 64);
            if (T == 0 && row >= row_start && row < row_end) y[size_t(t) * y_stride + row] = main_val + m;
        }
    }
}

// ---- exact integers per (row, super-block), read back from the repacked stream
__global__ __launch_bounds__(256) void block_ints_q4_k_kernel(const uint8_t *__restrict__ w,
                                                               const int8_t *__restrict__ q8qs,
                                                               const int16_t *__restrict__ q8bs,
                                                               int32_t *__restrict__ isum, int32_t *__restrict__ msum,
                                                               uint32_t n_out, uint32_t n_sb) {
    const uint64_t total = uint64_t(n_out) * n_sb;
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < total;
         i += uint64_t(gridDim.x) * blockDim.x) {
        const uint32_t row = uint32_t(i / n_sb), sb = uint32_t(i % n_sb);
        const uint8_t *chunk = w + (size_t(row >> 3) * n_sb + sb) * kQ4KSuperBytes;
        const uint4 hdr = reinterpret_cast<const uint4 *>(chunk)[row & 7];
        const uint4 sm = unpack_scales(hdr.y, hdr.z, hdr.w);
        const uint32_t *qrow = reinterpret_cast<const uint32_t *>(chunk + 128 + (row & 7) * 128);
        const uint32_t *xq = reinterpret_cast<const uint32_t *>(q8qs + size_t(sb) * 256);
        int si = 0, sm_acc = 0;
        for (uint32_t g = 0; g < 4; g++) {
            int dl = 0, dh = 0;
            for (uint32_t T = 0; T < 8; T++) {
                const uint32_t v = qrow[T * 4 + g];
                dl = __builtin_amdgcn_sdot4(int(v & 0x0f0f0f0fu), int(xq[16 * g + T]), dl, false);
                dh = __builtin_amdgcn_sdot4(int((v >> 4) & 0x0f0f0f0fu), int(xq[16 * g + 8 + T]), dh, false);
            }
            si += int(byte_of(sm.x, sm.y, 2 * g)) * dl + int(byte_of(sm.x, sm.y, 2 * g + 1)) * dh;
        }
        for (uint32_t j = 0; j < 8; j++)
            sm_acc += int(byte_of(sm.z, sm.w, j)) * (int(q8bs[sb * 16 + 2 * j]) + int(q8bs[sb * 16 + 2 * j + 1]));
        isum[i] = si;
        msum[i] = sm_acc;
    }
}

// ---- dequantise-and-dot, one lane per row, strictly sequential f32 sum over
// the elements of the row (q4_k.rs:38-53, core/model.rs:77-84); element value
// (d*sc)*q - dmin*mn as in dequantize_row_q4_k (quant/mod.rs:456-490).
__global__ __launch_bounds__(64) void q4_k_dequant_dot_kernel(const uint8_t *__restrict__ w,
                                                               const float *__restrict__ x_f32,
                                                               const int8_t *__restrict__ x_q8,
                                                               const float *__restrict__ x_scales,
                                                               float *__restrict__ y, uint32_t n_sb, uint32_t row_start,
                                                               uint32_t row_end, int mode) {
    const uint32_t row = row_start + blockIdx.x * 64 + threadIdx.x;
    if (row >= row_end) return;
    float sum = 0.0f;
    for (uint32_t sb = 0; sb < n_sb; sb++) {
        const uint8_t *chunk = w + (size_t(row >> 3) * n_sb + sb) * kQ4KSuperBytes;
        const uint4 hdr = reinterpret_cast<const uint4 *>(chunk)[row & 7];
        const float d = h2f(hdr.x & 0xffffu), dmin = h2f(hdr.x >> 16);
        const uint4 sm = unpack_scales(hdr.y, hdr.z, hdr.w);
        const uint4 *qrow = reinterpret_cast<const uint4 *>(chunk + 128 + (row & 7) * 128);
        uint4 qv[8];
#pragma unroll
        for (int T = 0; T < 8; T++) qv[T] = qrow[T];
#pragma unroll
        for (int g = 0; g < 4; g++) {
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const float dsc = d * float(byte_of(sm.x, sm.y, 2 * g + half));
                const float mm = dmin * float(byte_of(sm.z, sm.w, 2 * g + half));
#pragma unroll
                for (int T = 0; T < 8; T++) {
                    const uint32_t dw = g == 0 ? qv[T].x : (g == 1 ? qv[T].y : (g == 2 ? qv[T].z : qv[T].w));
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const uint32_t nib = (dw >> (8 * i + 4 * half)) & 0xfu;
                        const float wv = dsc * float(nib) - mm;
                        const uint32_t k = sb * 256 + 64 * g + 32 * half + 4 * T + i;
                        const float xv = mode == 1 ? x_f32[k] : float(int(x_q8[k])) * x_scales[k >> 5];
                        const float prod = wv * xv;
                        sum = sum + prod;
                    }
                }
            }
        }
    }
    y[row] = sum;
}

template <int B>
int launch_gemv_q4k(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums, float *y,
                    uint32_t y_stride, uint32_t row_start, uint32_t row_end, hipStream_t s) {
    const uint32_t tile0 = row_start / kTileRows;
    const uint32_t n_tiles = (row_end + kTileRows - 1) / kTileRows - tile0;
    const size_t lds_bytes = size_t(B) * w->n_units * kSbDwords * 4;
    if (lds_bytes > 64 * 1024)
        return rmi_fail(RMI_HIP_E_INVALID, "activation of %d tokens x %u elements does not fit the LDS staging", B, w->n_in);
    uint32_t n_waves = uint32_t(rmi_device_cus()) * 16;
    if (n_waves > n_tiles) n_waves = n_tiles;
    hipLaunchKernelGGL(gemv_q4_k_kernel<B>, dim3(n_waves), dim3(64), lds_bytes, s, w->data, d, qs, bsums, y, w->n_in,
                       w->n_units, y_stride, row_start, row_end, tile0, n_tiles, n_waves);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

}  // namespace

int rmi_launch_quantize_q8_k(const float *x, float *d, int8_t *qs, int16_t *bsums, uint32_t n_tokens, uint32_t n_in,
                             hipStream_t s) {
    const uint64_t blocks = uint64_t(n_tokens) * (n_in / 256);
    if (blocks == 0) return RMI_HIP_OK;
    if (blocks > 0x7fffffffull) return rmi_fail(RMI_HIP_E_INVALID, "activation too large for one launch");
    hipLaunchKernelGGL(quantize_q8_k_kernel, dim3(uint32_t(blocks)), dim3(64), 0, s, x, d, qs, bsums);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_launch_gemv_q4_k(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums, float *y,
                         uint32_t n_tokens, uint32_t y_stride, uint32_t row_start, uint32_t row_end, hipStream_t s) {
    if (row_start >= row_end || n_tokens == 0 || w->n_units == 0) return RMI_HIP_OK;
    const size_t per_token = size_t(w->n_units) * kSbDwords * 4;
    uint32_t chunk = uint32_t((64 * 1024) / per_token);
    if (chunk == 0) return rmi_fail(RMI_HIP_E_INVALID, "n_in=%u is too long for the GEMV staging", w->n_in);
    if (chunk > 8) chunk = 8;
    const uint32_t n_sb = w->n_units;
    for (uint32_t t0 = 0; t0 < n_tokens; t0 += chunk) {
        const uint32_t nt = n_tokens - t0 < chunk ? n_tokens - t0 : chunk;
        const float *dt = d + size_t(t0) * n_sb;
        const int8_t *qt = qs + size_t(t0) * w->n_in;
        const int16_t *bt = bsums + size_t(t0) * (w->n_in / 16);
        float *yt = y + size_t(t0) * y_stride;
        int rc;
        switch (nt) {
            case 1: rc = launch_gemv_q4k<1>(w, dt, qt, bt, yt, y_stride, row_start, row_end, s); break;
            case 2: rc = launch_gemv_q4k<2>(w, dt, qt, bt, yt, y_stride, row_start, row_end, s); break;
            case 3: rc = launch_gemv_q4k<3>(w, dt, qt, bt, yt, y_stride, row_start, row_end, s); break;
            case 4: rc = launch_gemv_q4k<4>(w, dt, qt, bt, yt, y_stride, row_start, row_end, s); break;
            case 5: rc = launch_gemv_q4k<5>(w, dt, qt, bt, yt, y_stride, row_start, row_end, s); break;
            case 6: rc = launch_gemv_q4k<6>(w, dt, qt, bt, yt, y_stride, row_start, row_end, s); break;
            case 7: rc = launch_gemv_q4k<7>(w, dt, qt, bt, yt, y_stride, row_start, row_end, s); break;
            default: rc = launch_gemv_q4k<8>(w, dt, qt, bt, yt, y_stride, row_start, row_end, s); break;
        }
        if (rc != RMI_HIP_OK) return rc;
    }
    return RMI_HIP_OK;
}

int rmi_launch_block_ints_q4_k(const rmi_hip_weight *w, const int8_t *qs, const int16_t *bsums, int32_t *isum,
                               int32_t *msum, hipStream_t s) {
    const uint64_t total = uint64_t(w->n_out) * w->n_units;
    if (total == 0) return RMI_HIP_OK;
    const uint32_t grid = uint32_t(total / 256 + 1 < 65535 ? total / 256 + 1 : 65535);
    hipLaunchKernelGGL(block_ints_q4_k_kernel, dim3(grid), dim3(256), 0, s, w->data, qs, bsums, isum, msum, w->n_out,
                       w->n_units);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_launch_q4_k_dequant_dot(const rmi_hip_weight *w, const float *x_f32, const int8_t *x_q8,
                                const float *x_scales, float *y, uint32_t row_start, uint32_t row_end, int mode,
                                hipStream_t s) {
    if (row_start >= row_end) return RMI_HIP_OK;
    const uint32_t grid = (row_end - row_start + 63) / 64;
    hipLaunchKernelGGL(q4_k_dequant_dot_kernel, dim3(grid), dim3(64), 0, s, w->data, x_f32, x_q8, x_scales, y,
                       w->n_units, row_start, row_end, mode);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
