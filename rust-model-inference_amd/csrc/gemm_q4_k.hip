// Q4_K x Q8_K prefill GEMM on the matrix cores: Y[t][n] = vec_dot_q4k_q8k(W[n], Q8_K(X[t])) for many tokens
// (Kernel::forward_batched semantics, src/ops/kernel/trait_.rs:78-109, with the dot of
// src/ops/quant/mod.rs:210-289 / 701-799).
//
// Per super-block (256 elements) and 32-token x 32-row tile:
//   * eight int8 MFMAs 32x32x32, one per 32-element sub-block, on the nibbles widened to int8 and the Q8_K
//     quants; each int32 result is scaled by the sub-block's 6-bit scale into sumi (one 24-bit multiply-add per
//     output: the scale is a per-lane scalar because a lane holds one weight row);
//   * the min term sum_j mn_j * (bsums[2j] + bsums[2j+1]) as two more int8 MFMAs: the pair sums (13 bits) are
//     split s = 128 h + l into two int8 operands, prod = 128 D_h + D_l;
//   * d * q8d and -dmin * q8d for the tile as one f32 outer-product MFMA (two blocks per instruction);
//   * acc = fma(d*q8d, float(sumi), acc), acc_m = fma(-dmin*q8d, float(prod), acc_m).
// All integers are exact (sumi is the sum of the reference's eight lane integers, prod of its four), and the
// f32 scale products are the reference's; the f32 accumulation runs over super-blocks in one chain per output
// instead of the AVX2 kernel's 8 + 4 lane chains, so results agree with it to rounding, not bit for bit.
//
// Workgroup = 4 waves (2 x 2) on a (64*NTW) x 64 tile.  Weights come from the GEMV tile stream; a 16-byte
// piece (the four dwords of lane T) is widened and scattered into natural element order by the LDS store.
#include "rmi_internal.h"

#include "device_common.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));

constexpr int kRow = 272;  // bytes between LDS rows of 256 quants: 16-byte reads of 8 lanes hit 8 bank groups

// the kmask unpack of quant/mod.rs:237-258: .x,.y = 8 scales, .z,.w = 8 mins, one byte each
__device__ __forceinline__ uint4 unpack_scales(uint32_t u0, uint32_t u1, uint32_t u2) {
    const uint32_t kmask1 = 0x3f3f3f3fu, kmask2 = 0x0f0f0f0fu, kmask3 = 0x03030303u;
    uint4 o;
    o.w = ((u2 >> 4) & kmask2) | (((u1 >> 6) & kmask3) << 4);
    o.z = u1 & kmask1;
    o.y = (u2 & kmask2) | (((u0 >> 6) & kmask3) << 4);
    o.x = u0 & kmask1;
    return o;
}

template <int NTW>
struct Q4kSmem {
    alignas(16) uint8_t wq[64 * NTW * kRow];
    alignas(16) uint8_t xq[64 * kRow];
    alignas(16) uint8_t xb[64 * 16];  // per token: h[8], l[8] of the bsums pair sums
};

template <int NTW>
__global__ __launch_bounds__(256) void gemm_q4_k_kernel(const uint8_t *__restrict__ w, const float *__restrict__ q8d,
                                                         const int8_t *__restrict__ q8qs,
                                                         const int16_t *__restrict__ q8bs, float *__restrict__ y,
                                                         uint32_t n_out, uint32_t n_sb, uint32_t n_tiles,
                                                         uint32_t n_tokens, uint32_t y_stride, uint32_t grid_n,
                                                         uint32_t grid_t, uint32_t t_fastest) {
    constexpr int kTileN = 64 * NTW, kTileT = 64;
    constexpr int kWPieces = kTileN * 8 / 256, kXPieces = kTileT * 16 / 256;
    __shared__ Q4kSmem<NTW> sm;

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t c = lane & 31, h = lane >> 5;
    const uint32_t n_off = (wave & 1) * 32 * NTW, t_off = (wave >> 1) * 32;
    // one XCD's workgroups are consecutive tiles, fastest along the smaller operand (see gemm_q8_0.hip)
    const uint32_t n_groups = grid_n * grid_t, lin = blockIdx.x;
    const uint32_t xcd = lin & 7, slot = lin >> 3;
    const uint32_t tile_id = xcd * (n_groups >> 3) + (xcd < (n_groups & 7) ? xcd : (n_groups & 7)) + slot;
    const uint32_t n0 = (t_fastest ? tile_id / grid_t : tile_id % grid_n) * kTileN;
    const uint32_t t0 = (t_fastest ? tile_id % grid_t : tile_id / grid_n) * kTileT;
    const uint32_t n_in = n_sb * 256;

    // --- staging addresses: uniform base + 32-bit offsets
    const uint32_t tile_first = (n0 >> 3) < n_tiles ? (n0 >> 3) : n_tiles - 1;
    const uint8_t *w_base = w + size_t(tile_first) * n_sb * kQ4KSuperBytes;
    uint32_t w_off[kWPieces], w_dst[kWPieces];
#pragma unroll
    for (int i = 0; i < kWPieces; i++) {
        const uint32_t p = tid + 256 * i, row = p >> 3, T = p & 7;
        uint32_t tile = (n0 + row) >> 3;
        if (tile >= n_tiles) tile = n_tiles - 1;  // rows past the padded stream: in bounds, never stored
        w_off[i] = (tile - tile_first) * n_sb * kQ4KSuperBytes + 128 + ((n0 + row) & 7) * 128 + T * 16;
        w_dst[i] = row * kRow + T * 4;
    }
    const uint32_t last_tok = n_tokens - 1 - t0;  // tokens past the end read the last token; never stored
    const int8_t *x_base = q8qs + size_t(t0) * n_in;
    uint32_t x_off[kXPieces], x_dst[kXPieces];
#pragma unroll
    for (int i = 0; i < kXPieces; i++) {
        const uint32_t p = tid + 256 * i, tok = p >> 4, piece = p & 15;
        x_off[i] = (tok < last_tok ? tok : last_tok) * n_in + piece * 16;
        x_dst[i] = tok * kRow + piece * 16;
    }
    const int16_t *bs_base = q8bs + size_t(t0) * n_sb * 16;
    const uint32_t bs_off = ((tid & 63) < last_tok ? (tid & 63) : last_tok) * n_sb * 16;
    // --- per-lane scalars: the header of this lane's weight rows, the Q8_K scale of this lane's token
    uint32_t hd_off[NTW];
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
        const uint32_t row = n0 + n_off + nt * 32 + c;
        uint32_t tile = row >> 3;
        if (tile >= n_tiles) tile = n_tiles - 1;
        hd_off[nt] = (tile - tile_first) * n_sb * kQ4KSuperBytes + (row & 7) * 16;
    }
    const float *d_base = q8d + size_t(t0) * n_sb;
    const uint32_t d_off = ((t_off + c) < last_tok ? (t_off + c) : last_tok) * n_sb;

    struct Stage {
        u32x4 w[kWPieces], x[kXPieces], bs[2];
        u32x4 hdr[NTW];
        float xd;
    };
    auto load_sb = [&](Stage &g, uint32_t sb) {
#pragma unroll
        for (int i = 0; i < kWPieces; i++)
            g.w[i] = *reinterpret_cast<const u32x4 *>(w_base + (w_off[i] + sb * kQ4KSuperBytes));
#pragma unroll
        for (int i = 0; i < kXPieces; i++) g.x[i] = *reinterpret_cast<const u32x4 *>(x_base + (x_off[i] + sb * 256));
        if (tid < 64) {
            const u32x4 *b = reinterpret_cast<const u32x4 *>(bs_base + (bs_off + sb * 16));
            g.bs[0] = b[0];
            g.bs[1] = b[1];
        }
#pragma unroll
        for (int nt = 0; nt < NTW; nt++)
            g.hdr[nt] = *reinterpret_cast<const u32x4 *>(w_base + (hd_off[nt] + sb * kQ4KSuperBytes));
        g.xd = d_base[d_off + sb];
    };
    auto store_sb = [&](const Stage &g) {
#pragma unroll
        for (int i = 0; i < kWPieces; i++) {
            uint8_t *dst = sm.wq + w_dst[i];
            const uint32_t dw[4] = {g.w[i].x, g.w[i].y, g.w[i].z, g.w[i].w};
#pragma unroll
            for (int gq = 0; gq < 4; gq++) {  // dword g: low nibbles = sub-block 2g, high nibbles = 2g+1
                *reinterpret_cast<uint32_t *>(dst + (2 * gq) * 32) = dw[gq] & 0x0f0f0f0fu;
                *reinterpret_cast<uint32_t *>(dst + (2 * gq + 1) * 32) = (dw[gq] >> 4) & 0x0f0f0f0fu;
            }
        }
#pragma unroll
        for (int i = 0; i < kXPieces; i++) *reinterpret_cast<u32x4 *>(sm.xq + x_dst[i]) = g.x[i];
        if (tid < 64) {  // pair sums of bsums, split s = 128 hi + lo with lo in [-64, 63]
            const uint32_t b[8] = {g.bs[0].x, g.bs[0].y, g.bs[0].z, g.bs[0].w, g.bs[1].x, g.bs[1].y, g.bs[1].z, g.bs[1].w};
            uint32_t hi[2] = {0, 0}, lo[2] = {0, 0};
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int s = int(int16_t(b[j] & 0xffffu)) + int(int16_t(b[j] >> 16));
                const int hv = (s + 64) >> 7, lv = s - hv * 128;
                hi[j >> 2] |= uint32_t(hv & 0xff) << (8 * (j & 3));
                lo[j >> 2] |= uint32_t(lv & 0xff) << (8 * (j & 3));
            }
            *reinterpret_cast<u32x4 *>(sm.xb + tid * 16) = u32x4{hi[0], hi[1], lo[0], lo[1]};
        }
    };

    float acc[NTW][16], acc_m[NTW][16];
#pragma unroll
    for (int nt = 0; nt < NTW; nt++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[nt][i] = acc_m[nt][i] = 0.0f;

    Stage st;
    if (n_sb > 0) load_sb(st, 0);
    for (uint32_t sb = 0; sb < n_sb; sb++) {
        __syncthreads();  // everyone is done with the previous super-block
        store_sb(st);
        u32x4 hdr[NTW];
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) hdr[nt] = st.hdr[nt];
        const float xd = st.xd;
        __syncthreads();
        if (sb + 1 < n_sb) load_sb(st, sb + 1);

        const uint8_t *xrow = sm.xq + (t_off + c) * kRow + h * 16;
        const u32x4 xbv = *reinterpret_cast<const u32x4 *>(sm.xb + (t_off + c) * 16);
        // the min-term operands live in k = 0..7, i.e. in the first two dwords of the h = 0 lanes
        const v4i x_hi = h == 0 ? v4i{int(xbv.x), int(xbv.y), 0, 0} : v4i{0, 0, 0, 0};
        const v4i x_lo = h == 0 ? v4i{int(xbv.z), int(xbv.w), 0, 0} : v4i{0, 0, 0, 0};
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) {
            const float wd = h2f(hdr[nt].x & 0xffffu), wdmin = h2f(hdr[nt].x >> 16);
            const uint4 s8 = unpack_scales(hdr[nt].y, hdr[nt].z, hdr[nt].w);
            v32f zero32;
#pragma unroll
            for (int i = 0; i < 32; i++) zero32[i] = 0.0f;
            // block 0 (lanes 0-31): q8d * d; block 1 (lanes 32-63): q8d * (-dmin)
            const v32f sc = __builtin_amdgcn_mfma_f32_32x32x1f32(xd, h == 0 ? wd : -wdmin, zero32, 0, 0, 0);
            const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const uint8_t *wrow = sm.wq + (n_off + nt * 32 + c) * kRow + h * 16;
            int sumi[16];
#pragma unroll
            for (int i = 0; i < 16; i++) sumi[i] = 0;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const u32x4 xu = *reinterpret_cast<const u32x4 *>(xrow + j * 32);
                const u32x4 wu = *reinterpret_cast<const u32x4 *>(wrow + j * 32);
                const v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(v4i{int(xu.x), int(xu.y), int(xu.z), int(xu.w)},
                                                                      v4i{int(wu.x), int(wu.y), int(wu.z), int(wu.w)},
                                                                      zero16, 0, 0, 0);
                const int scale = int(((j < 4 ? s8.x : s8.y) >> (8 * (j & 3))) & 0xffu);
#pragma unroll
                for (int i = 0; i < 16; i++) sumi[i] += __mul24(d[i], scale);  // |dot| < 2^16, scale < 2^6
            }
            const v4i mn = h == 0 ? v4i{int(s8.z), int(s8.w), 0, 0} : v4i{0, 0, 0, 0};
            const v16i d_hi = __builtin_amdgcn_mfma_i32_32x32x32_i8(x_hi, mn, zero16, 0, 0, 0);
            const v16i d_lo = __builtin_amdgcn_mfma_i32_32x32x32_i8(x_lo, mn, zero16, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                acc[nt][i] = __builtin_fmaf(sc[i], float(sumi[i]), acc[nt][i]);
                acc_m[nt][i] = __builtin_fmaf(sc[16 + i], float(d_hi[i] * 128 + d_lo[i]), acc_m[nt][i]);
            }
        }
    }

#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
        const uint32_t n = n0 + n_off + nt * 32 + c;
        if (n < n_out) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t t = t0 + t_off + 8 * (i >> 2) + 4 * h + (i & 3);
                if (t < n_tokens) y[size_t(t) * y_stride + n] = acc[nt][i] + acc_m[nt][i];
            }
        }
    }
}

template <int NTW>
void launch(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bs, float *y, uint32_t n_tokens,
            uint32_t y_stride, hipStream_t s) {
    const uint32_t grid_n = (w->n_out + 64 * NTW - 1) / (64 * NTW), grid_t = (n_tokens + 63) / 64;
    hipLaunchKernelGGL((gemm_q4_k_kernel<NTW>), dim3(grid_n * grid_t), dim3(256), 0, s, w->data, d, qs, bs, y, w->n_out,
                       w->n_units, w->n_tiles, n_tokens, y_stride, grid_n, grid_t, n_tokens < w->n_out ? 1u : 0u);
}

}  // namespace

int rmi_launch_gemm_q4_k(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums, float *y,
                         uint32_t n_tokens, uint32_t y_stride, hipStream_t s) {
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    const uint64_t groups128 = uint64_t((w->n_out + 127) / 128) * ((n_tokens + 63) / 64);
    const uint64_t groups64 = uint64_t((w->n_out + 63) / 64) * ((n_tokens + 63) / 64);
    if (groups64 > 0x7fffffffull) return rmi_fail(RMI_HIP_E_INVALID, "GEMM too large for one launch");
    if (groups128 >= 2 * uint64_t(rmi_device_cus()))
        launch<2>(w, d, qs, bsums, y, n_tokens, y_stride, s);
    else
        launch<1>(w, d, qs, bsums, y, n_tokens, y_stride, s);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
