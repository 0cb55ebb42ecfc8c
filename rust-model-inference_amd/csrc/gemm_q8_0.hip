// Q8_0 x Q8_0 prefill GEMM on int8 MFMA: Y[t][n] = sum_b (f32(wd[n][b]) * xs[t][b]) * dot_b(W[n], X[t]).
//
// One 32x32x32 MFMA is one Q8_0 block (K = 32) of a 32-token x 32-row tile, so
// the int32 accumulator is the per-block dot and starts from zero every block.
// f32 order: acc = fma(float(dot), wd*xs, acc), blocks in sequence — the order
// of matmul_q8_0_vs_q8_0_neon (src/ops/kernel/q8_0/neon.rs:49-73).
//
// Workgroup = 4 waves (2 x 2); wave (wn, wt) owns NTW x TTW MFMA tiles, i.e.
// 32*NTW weight rows x 32*TTW tokens.  The launcher picks the largest tile that
// still gives every SIMD about two waves.  Per quad (4 blocks,
// 128 k) the workgroup stages into LDS, through registers so that the global
// loads of the next DEPTH quads fly while quad q is multiplied:
//   Ws  128 rows x 128 B, straight from the GEMV tile stream (quad order),
//   Xs  TILE_T tokens x 128 B in natural order,
//   wd  128 rows x 4 f32, xs 4 blocks x TILE_T f32 in accumulator order.
// MFMA lane (c, h) supplies 16 of the 32 k values of its row/column; which 16
// is free as long as both operands agree.  The 64 bytes at Ws[row][64h..] hold
// the slices L = 4h..4h+3 of the row's quad: dword j of each 16-byte piece is
// k = 16h+4L'..+3 of block j, i.e. bytes 16h..16h+15 of that block in the
// natural activation order, which is what Xs[token][32j+16h..] holds.  Rows of
// both LDS tiles are 144 B apart so that 16-byte reads of 8 consecutive lanes
// fall into 8 different bank groups.
//
// The f32 rescale is 3 VALU instructions per output per block (convert,
// scale product, fma) against 32 MFMA cycles per 1024 outputs: the kernel is
// bound by the VALU at about 1/6 of the int8 MFMA peak.
#include "rmi_internal.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kRowStride = 144;  // bytes between rows of Ws / Xs

__device__ __forceinline__ float h2f(uint32_t bits16) {
    return float(__builtin_bit_cast(_Float16, uint16_t(bits16)));
}

template <int NTW, int TTW>  // 32-row and 32-token sub-tiles per wave
struct GemmSmem {
    static constexpr int kTileN = 64 * NTW;
    static constexpr int kTileT = 64 * TTW;
    alignas(16) uint8_t ws[kTileN * kRowStride];
    alignas(16) uint8_t xs_q[kTileT * kRowStride];
    alignas(16) float wd[kTileN * 4];
    alignas(16) float xs[4 * kTileT];  // [block j][32-token tile][h][16]
};

// DEPTH = quads whose global loads are in flight (held in registers) ahead of the multiply
template <int NTW, int TTW, int DEPTH>
__global__ __launch_bounds__(256) void gemm_q8_0_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ x_q8,
                                                         const float *__restrict__ x_scales, float *__restrict__ y,
                                                         uint32_t n_out, uint32_t n_in, uint32_t n_oct,
                                                         uint32_t n_tiles, uint32_t n_tokens, uint32_t y_stride) {
    constexpr int kTileN = 64 * NTW, kTileT = 64 * TTW;
    constexpr int kWPieces = kTileN * 8 / 256;  // 16-byte pieces of Ws per thread
    constexpr int kXPieces = kTileT * 8 / 256;  // 16-byte pieces of Xs per thread
    __shared__ GemmSmem<NTW, TTW> sm;

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t c = lane & 31, h = lane >> 5;
    const uint32_t n_off = (wave & 1) * 32 * NTW, t_off = (wave >> 1) * 32 * TTW;
    const uint32_t n0 = blockIdx.x * kTileN, t0 = blockIdx.y * kTileT;
    const uint32_t nb = n_in >> 5, n_quads = (nb + 3) >> 2;

    // --- what this thread stages per quad
    // Ws: pieces p = tid + 256 i -> row p>>3, piece p&7
    const uint8_t *w_src[kWPieces];
    uint32_t w_dst[kWPieces];
#pragma unroll
    for (int i = 0; i < kWPieces; i++) {
        const uint32_t p = tid + 256 * i, row = p >> 3, L = p & 7;
        uint32_t tile = (n0 + row) >> 3;
        if (tile >= n_tiles) tile = n_tiles - 1;  // rows past the padded stream: stay in bounds, never stored
        w_src[i] = w + size_t(tile) * n_oct * kOctetBytes + size_t(n_oct) * 128 + ((n0 + row) & 7) * 128 + L * 16;
        w_dst[i] = row * kRowStride + L * 16;
    }
    // Xs: pieces p -> token p>>3, piece p&7
    const int8_t *x_src[kXPieces];
    uint32_t x_dst[kXPieces];
    bool x_ok[kXPieces];
#pragma unroll
    for (int i = 0; i < kXPieces; i++) {
        const uint32_t p = tid + 256 * i, tok = p >> 3, piece = p & 7;
        x_ok[i] = t0 + tok < n_tokens;
        x_src[i] = x_q8 + size_t(x_ok[i] ? t0 + tok : 0) * n_in + piece * 16;
        x_dst[i] = tok * kRowStride + piece * 16;
    }
    // wd: threads 0..127, one row each (4 f16 of the quad)
    const uint8_t *wd_src = nullptr;
    if (tid < kTileN) {
        uint32_t tile = (n0 + tid) >> 3;
        if (tile >= n_tiles) tile = n_tiles - 1;
        wd_src = w + size_t(tile) * n_oct * kOctetBytes + ((n0 + tid) & 7) * 16;
    }
    // xs: element e = tid + 256 i of 4*kTileT -> block j = e / kTileT, token e % kTileT
    constexpr int kXsPer = 4 * kTileT / 256;
    const float *xs_src[kXsPer];
    uint32_t xs_dst[kXsPer], xs_j[kXsPer];
    bool xs_ok[kXsPer];
#pragma unroll
    for (int i = 0; i < kXsPer; i++) {
        const uint32_t e = tid + 256 * i, j = e / kTileT, tok = e % kTileT;
        const uint32_t tt = tok >> 5, within = tok & 31;
        const uint32_t hh = (within >> 2) & 1, idx = ((within >> 3) << 2) | (within & 3);
        xs_ok[i] = t0 + tok < n_tokens;
        xs_src[i] = x_scales + size_t(xs_ok[i] ? t0 + tok : 0) * nb;
        xs_j[i] = j;
        xs_dst[i] = ((j * (kTileT / 32) + tt) * 2 + hh) * 16 + idx;
    }

    struct Stage {
        u32x4 w[kWPieces], x[kXPieces];
        u32x2 wd;
        float xs[kXsPer];
    };
    Stage st[DEPTH];

    auto load_quad = [&](Stage &g, uint32_t q) {
#pragma unroll
        for (int i = 0; i < kWPieces; i++) g.w[i] = *reinterpret_cast<const u32x4 *>(w_src[i] + size_t(q) * 1024);
#pragma unroll
        for (int i = 0; i < kXPieces; i++) {
            // the last quad of a row may hold fewer than 4 blocks: pieces beyond n_in read as zero
            const bool in_row = q * 128 + (tid & 7) * 16 < n_in;
            g.x[i] = (x_ok[i] && in_row) ? *reinterpret_cast<const u32x4 *>(x_src[i] + size_t(q) * 128) : u32x4{0, 0, 0, 0};
        }
        g.wd = u32x2{0, 0};
        if (tid < kTileN) g.wd = *reinterpret_cast<const u32x2 *>(wd_src + size_t(q >> 1) * 128 + (q & 1) * 8);
#pragma unroll
        for (int i = 0; i < kXsPer; i++) {
            const uint32_t b = q * 4 + xs_j[i];
            g.xs[i] = (xs_ok[i] && b < nb) ? xs_src[i][b] : 0.0f;
        }
    };
    auto store_quad = [&](const Stage &g) {
#pragma unroll
        for (int i = 0; i < kWPieces; i++) *reinterpret_cast<u32x4 *>(sm.ws + w_dst[i]) = g.w[i];
#pragma unroll
        for (int i = 0; i < kXPieces; i++) *reinterpret_cast<u32x4 *>(sm.xs_q + x_dst[i]) = g.x[i];
        if (tid < kTileN) {
            float4 f = make_float4(h2f(g.wd.x & 0xffffu), h2f(g.wd.x >> 16), h2f(g.wd.y & 0xffffu), h2f(g.wd.y >> 16));
            *reinterpret_cast<float4 *>(sm.wd + tid * 4) = f;
        }
#pragma unroll
        for (int i = 0; i < kXsPer; i++) sm.xs[xs_dst[i]] = g.xs[i];
    };

    float acc[NTW][TTW][16];
#pragma unroll
    for (int nt = 0; nt < NTW; nt++)
#pragma unroll
        for (int tt = 0; tt < TTW; tt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[nt][tt][i] = 0.0f;

#pragma unroll
    for (int d = 0; d < DEPTH; d++)
        if (uint32_t(d) < n_quads) load_quad(st[d], d);
    for (uint32_t q0 = 0; q0 < n_quads; q0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; d++) {
        const uint32_t q = q0 + d;
        if (q >= n_quads) break;
        __syncthreads();  // everyone is done reading the previous quad
        store_quad(st[d]);
        __syncthreads();
        if (q + DEPTH < n_quads) load_quad(st[d], q + DEPTH);

        v4i wj[NTW][4];
        float wdv[NTW][4];
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) {
            const uint32_t row = n_off + nt * 32 + c;
            const u32x4 *wp = reinterpret_cast<const u32x4 *>(sm.ws + row * kRowStride + h * 64);
            const u32x4 u0 = wp[0], u1 = wp[1], u2 = wp[2], u3 = wp[3];
            wj[nt][0] = v4i{int(u0.x), int(u1.x), int(u2.x), int(u3.x)};
            wj[nt][1] = v4i{int(u0.y), int(u1.y), int(u2.y), int(u3.y)};
            wj[nt][2] = v4i{int(u0.z), int(u1.z), int(u2.z), int(u3.z)};
            wj[nt][3] = v4i{int(u0.w), int(u1.w), int(u2.w), int(u3.w)};
            const float4 f = *reinterpret_cast<const float4 *>(sm.wd + row * 4);
            wdv[nt][0] = f.x;
            wdv[nt][1] = f.y;
            wdv[nt][2] = f.z;
            wdv[nt][3] = f.w;
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // blocks past n_in/32 in the last quad are all-zero on both sides (scale 0, quants 0):
            // fma(float(0), 0, acc) leaves acc unchanged, so they are multiplied like the rest
            {
#pragma unroll
                for (int tt = 0; tt < TTW; tt++) {
                    const uint32_t tok = t_off + tt * 32 + c;
                    const u32x4 xv = *reinterpret_cast<const u32x4 *>(sm.xs_q + tok * kRowStride + j * 32 + h * 16);
                    const v4i a = v4i{int(xv.x), int(xv.y), int(xv.z), int(xv.w)};
                    const float4 *xs4 =
                        reinterpret_cast<const float4 *>(sm.xs + ((j * (kTileT / 32) + (t_off >> 5) + tt) * 2 + h) * 16);
                    float s[16];
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const float4 v = xs4[g];
                        s[4 * g] = v.x;
                        s[4 * g + 1] = v.y;
                        s[4 * g + 2] = v.z;
                        s[4 * g + 3] = v.w;
                    }
#pragma unroll
                    for (int nt = 0; nt < NTW; nt++) {
                        v16i d = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                        d = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, wj[nt][j], d, 0, 0, 0);
#pragma unroll
                        for (int i = 0; i < 16; i++)
                            acc[nt][tt][i] = __builtin_fmaf(float(d[i]), wdv[nt][j] * s[i], acc[nt][tt][i]);
                    }
                }
            }
        }
      }
    }

#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
        const uint32_t n = n0 + n_off + nt * 32 + c;
        if (n < n_out) {
#pragma unroll
            for (int tt = 0; tt < TTW; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const uint32_t t = t0 + t_off + tt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                    if (t < n_tokens) y[size_t(t) * y_stride + n] = acc[nt][tt][i];
                }
        }
    }
}

template <int NTW, int TTW, int DEPTH>
void launch_gemm(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                        uint32_t n_tokens, uint32_t y_stride, hipStream_t s) {
    dim3 grid((w->n_out + 64 * NTW - 1) / (64 * NTW), (n_tokens + 64 * TTW - 1) / (64 * TTW));
    hipLaunchKernelGGL((gemm_q8_0_kernel<NTW, TTW, DEPTH>), grid, dim3(256), 0, s, w->data, x_q8, x_scales, y, w->n_out,
                       w->n_in, w->n_units, w->n_tiles, n_tokens, y_stride);
}

}  // namespace

int rmi_launch_gemm_q8_0(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                         uint32_t n_tokens, uint32_t y_stride, hipStream_t s) {
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    // the largest workgroup tile that still yields two workgroups (eight waves) per compute unit
    const uint64_t want = uint64_t(rmi_device_cus()) * 2;
    auto groups = [&](uint32_t tn, uint32_t tt) {
        return uint64_t((w->n_out + tn - 1) / tn) * ((n_tokens + tt - 1) / tt);
    };
    if (n_tokens > 64 && groups(128, 128) >= want)
        launch_gemm<2, 2, 2>(w, x_q8, x_scales, y, n_tokens, y_stride, s);
    else if (groups(128, 64) >= want)
        launch_gemm<2, 1, 3>(w, x_q8, x_scales, y, n_tokens, y_stride, s);
    else
        launch_gemm<1, 1, 4>(w, x_q8, x_scales, y, n_tokens, y_stride, s);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
