// Q8_0 x Q8_0 prefill GEMM on the matrix cores: Y[t][n] = sum_b (f32(wd[n][b]) * xs[t][b]) * dot_b(W[n], X[t]).
//
// One 32x32x32 int8 MFMA is one Q8_0 block (K = 32) of a 32-token x 32-row
// tile, so its int32 result is the per-block dot and starts from zero every
// block.  The f32 scale products wd*xs of the same tile are a rank-1 outer
// product, which v_mfma_f32_32x32x1_2b_f32 delivers in the accumulator layout
// of the int8 result, two blocks per instruction (lanes 0-31 feed the first
// block, lanes 32-63 the second); a single product plus zero is the correctly
// rounded f32 product, subnormals included.  What is left for the VALU is
// acc = fma(float(dot), scale, acc) with the blocks in sequence: the order of
// matmul_q8_0_vs_q8_0_neon (src/ops/kernel/q8_0/neon.rs:49-73), bit for bit.
//
// Workgroup = 4 waves (2 x 2); wave (wn, wt) owns NTW x TTW MFMA tiles, i.e.
// 32*NTW weight rows x 32*TTW tokens.  Per quad (4 blocks, 128 k) the
// workgroup stages both int8 operands into LDS in the natural k order, 128
// bytes a row, rows 144 bytes apart so that the 16-byte reads of 8 consecutive
// lanes fall into 8 different bank groups.  Weights come from the GEMV tile
// stream, whose 16-byte pieces hold the 4-byte slice L of blocks 0..3: each
// piece is written back as four dwords, one into each block of the row.  LDS is
// double-buffered (one barrier per quad) and the global loads of the next quad
// stay in registers while the current one is multiplied.  MFMA lane (c, h)
// reads bytes 16h..16h+15 of block j of its row / token for both operands.
// The scales go from global memory straight into the lanes that feed the
// outer-product MFMA.
//
// Per 32x32 tile and block the VALU issues 32 instructions (convert, fma;
// 128 cycles) and the f32 outer product, which unlike the int8 MFMA does not
// overlap with VALU work, holds the SIMD for about 32 more: the rescale bounds
// the kernel at roughly a fifth of the int8 MFMA peak (measured: 958 TOP/s for
// the multiply loop alone, with operands held in registers).
#include "rmi_internal.h"

#include "device_common.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));

constexpr int kRowStride = 144;  // bytes between rows of the LDS tiles

// NTW x TTW 32x32 sub-tiles per wave, WN x WT waves per workgroup
template <int NTW, int TTW, int WN, int WT>
struct GemmSmem {
    static constexpr int kTileN = 32 * NTW * WN;
    static constexpr int kTileT = 32 * TTW * WT;
    alignas(16) uint8_t ws[2][kTileN * kRowStride];
    alignas(16) uint8_t xq[2][kTileT * kRowStride];
};

template <int NTW, int TTW, int WN, int WT, int DEPTH>
__global__ __launch_bounds__(64 * WN * WT) void gemm_q8_0_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ x_q8,
                                                         const float *__restrict__ x_scales, float *__restrict__ y,
                                                         uint32_t n_out, uint32_t n_in, uint32_t n_oct,
                                                         uint32_t n_tiles, uint32_t n_tokens, uint32_t y_stride,
                                                         uint32_t grid_n, uint32_t grid_t, uint32_t t_fastest) {
    constexpr int kThreads = 64 * WN * WT;
    constexpr int kTileN = 32 * NTW * WN, kTileT = 32 * TTW * WT;
    constexpr int kWPieces = kTileN * 8 / kThreads;  // 16-byte pieces of the weight tile per thread
    constexpr int kXPieces = kTileT * 8 / kThreads;  // 16-byte pieces of the token tile per thread
    static_assert(kWPieces * kThreads == kTileN * 8 && kXPieces * kThreads == kTileT * 8, "tile must split evenly");
    __shared__ GemmSmem<NTW, TTW, WN, WT> sm;

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t c = lane & 31, h = lane >> 5;
    const uint32_t n_off = (wave % WN) * 32 * NTW, t_off = (wave / WN) * 32 * TTW;
    // Workgroups are handed to the 8 XCDs round-robin, each XCD with its own L2.  Renumber them so that the
    // workgroups of one XCD are consecutive tiles, running fastest along the smaller operand: every XCD then
    // fetches that operand whole and only its own eighth of the larger one.
    const uint32_t n_groups = grid_n * grid_t, lin = blockIdx.x;
    const uint32_t xcd = lin & 7, slot = lin >> 3;
    const uint32_t tile_id = xcd * (n_groups >> 3) + (xcd < (n_groups & 7) ? xcd : (n_groups & 7)) + slot;
    const uint32_t n0 = (t_fastest ? tile_id / grid_t : tile_id % grid_n) * kTileN;
    const uint32_t t0 = (t_fastest ? tile_id % grid_t : tile_id / grid_n) * kTileT;
    const uint32_t nb = n_in >> 5, n_quads = (nb + 3) >> 2;

    // --- int8 staging: pieces p = tid + kThreads i -> row p>>3, piece p&7
    // Addresses are a workgroup-uniform base plus a 32-bit offset per thread.
    const uint32_t tile_first = (n0 >> 3) < n_tiles ? (n0 >> 3) : n_tiles - 1;
    const uint8_t *w_base = w + size_t(tile_first) * n_oct * kOctetBytes;
    uint32_t w_off[kWPieces], w_dst[kWPieces];
#pragma unroll
    for (int i = 0; i < kWPieces; i++) {
        const uint32_t p = tid + kThreads * i, row = p >> 3, L = p & 7;
        uint32_t tile = (n0 + row) >> 3;
        if (tile >= n_tiles) tile = n_tiles - 1;  // rows past the padded stream: stay in bounds, never stored
        w_off[i] = (tile - tile_first) * n_oct * kOctetBytes + n_oct * 128 + ((n0 + row) & 7) * 128 + L * 16;
        w_dst[i] = row * kRowStride + L * 4;
    }
    // Tokens past n_tokens and, in the last quad, pieces past n_in are multiplied like the rest: their
    // products meet zero weight quants or are never stored.  Only the addresses are kept inside the buffer.
    const int8_t *x_base = x_q8 + size_t(t0) * n_in;
    const uint64_t x_room = uint64_t(n_tokens - t0) * n_in - 16;
    const uint32_t x_lim = x_room < 0xfffffff0ull ? uint32_t(x_room) : 0xfffffff0u;
    uint32_t x_off[kXPieces], x_dst[kXPieces];
#pragma unroll
    for (int i = 0; i < kXPieces; i++) {
        const uint32_t p = tid + kThreads * i, tok = p >> 3, piece = p & 7;
        x_off[i] = tok * n_in + piece * 16;
        x_dst[i] = tok * kRowStride + piece * 16;
    }
    // --- scales of this lane: blocks h and 2+h of the quad, of row / token c of each sub-tile
    uint32_t wd_off[NTW];
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
        const uint32_t row = n0 + n_off + nt * 32 + c;
        uint32_t tile = row >> 3;
        if (tile >= n_tiles) tile = n_tiles - 1;
        wd_off[nt] = (tile - tile_first) * n_oct * kOctetBytes + (row & 7) * 16;
    }
    const float *xs_base = x_scales + size_t(t0) * nb;
    uint32_t xs_off[TTW];
#pragma unroll
    for (int tt = 0; tt < TTW; tt++) {
        const uint32_t tok = t_off + tt * 32 + c;
        xs_off[tt] = (tok < n_tokens - t0 ? tok : n_tokens - t0 - 1) * nb;
    }

    struct Stage {
        u32x4 w[kWPieces], x[kXPieces];
    };
    struct Scales {  // as loaded: the four f16 weight scales of the quad, the two f32 token scales of this lane
        u32x2 wd[NTW];
        float xs[TTW][2];
    };
    auto load_quad = [&](Stage &g, uint32_t q) {
#pragma unroll
        for (int i = 0; i < kWPieces; i++) g.w[i] = *reinterpret_cast<const u32x4 *>(w_base + (w_off[i] + q * 1024));
#pragma unroll
        for (int i = 0; i < kXPieces; i++) {
            const uint32_t off = x_off[i] + q * 128;
            g.x[i] = *reinterpret_cast<const u32x4 *>(x_base + (off < x_lim ? off : x_lim));
        }
    };
    auto store_quad = [&](const Stage &g, uint32_t buf) {
#pragma unroll
        for (int i = 0; i < kWPieces; i++) {
            uint8_t *dst = sm.ws[buf] + w_dst[i];
            *reinterpret_cast<uint32_t *>(dst) = g.w[i].x;
            *reinterpret_cast<uint32_t *>(dst + 32) = g.w[i].y;
            *reinterpret_cast<uint32_t *>(dst + 64) = g.w[i].z;
            *reinterpret_cast<uint32_t *>(dst + 96) = g.w[i].w;
        }
#pragma unroll
        for (int i = 0; i < kXPieces; i++) *reinterpret_cast<u32x4 *>(sm.xq[buf] + x_dst[i]) = g.x[i];
    };
    auto load_scales = [&](Scales &sc, uint32_t q) {
        // weight scales of padded blocks are zero in the stream; token scales beyond n_in/32 are not there
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) {
            sc.wd[nt] = *reinterpret_cast<const u32x2 *>(w_base + (wd_off[nt] + (q >> 1) * 128 + (q & 1) * 8));
        }
#pragma unroll
        for (int tt = 0; tt < TTW; tt++) {
            // past n_in/32 the last scale of the row is read instead; the consumer replaces it by zero
            const uint32_t b = q * 4 + h;
            sc.xs[tt][0] = xs_base[xs_off[tt] + (b < nb ? b : nb - 1)];
            sc.xs[tt][1] = xs_base[xs_off[tt] + (b + 2 < nb ? b + 2 : nb - 1)];
        }
    };

    float acc[NTW][TTW][16];
#pragma unroll
    for (int nt = 0; nt < NTW; nt++)
#pragma unroll
        for (int tt = 0; tt < TTW; tt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[nt][tt][i] = 0.0f;

    // Rings of DEPTH quads: the global loads of quad k wait in registers slot k % DEPTH (scales for DEPTH
    // iterations, int8 pieces for DEPTH - 1: they move to LDS one iteration before they are multiplied).
    Stage st[DEPTH];
    Scales sc[DEPTH];
    if (n_quads > 0) {
        load_quad(st[0], 0);
        store_quad(st[0], 0);
    }
#pragma unroll
    for (int k = 0; k < DEPTH; k++)
        if (uint32_t(k) < n_quads) load_scales(sc[k], k);
#pragma unroll
    for (int k = 1; k <= DEPTH; k++)
        if (uint32_t(k) < n_quads) load_quad(st[k % DEPTH], k);
    for (uint32_t q0 = 0; q0 < n_quads; q0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; d++) {
        const uint32_t q = q0 + d;
        if (q >= n_quads) break;
        const uint32_t buf = q & 1;
        __syncthreads();  // quad q is in sm.*[buf]; nobody reads the other buffer any more
        float wd_cur[NTW][2], xs_cur[TTW][2];
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) {
            wd_cur[nt][0] = h2f((sc[d].wd[nt].x >> (16 * h)) & 0xffffu);
            wd_cur[nt][1] = h2f((sc[d].wd[nt].y >> (16 * h)) & 0xffffu);
        }
#pragma unroll
        for (int tt = 0; tt < TTW; tt++) {
            // a scale past n_in/32 must be a true zero: its block's dot is zero and the product must not be NaN
            xs_cur[tt][0] = q * 4 + h < nb ? sc[d].xs[tt][0] : 0.0f;
            xs_cur[tt][1] = q * 4 + h + 2 < nb ? sc[d].xs[tt][1] : 0.0f;
        }
        if (q + DEPTH < n_quads) load_scales(sc[d], q + DEPTH);
        if (q + 1 < n_quads) {
            store_quad(st[(d + 1) % DEPTH], buf ^ 1);
            if (q + 1 + DEPTH < n_quads) load_quad(st[(d + 1) % DEPTH], q + 1 + DEPTH);
        }
        const uint8_t *wrow[NTW], *xrow[TTW];
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) wrow[nt] = sm.ws[buf] + (n_off + nt * 32 + c) * kRowStride + h * 16;
#pragma unroll
        for (int tt = 0; tt < TTW; tt++) xrow[tt] = sm.xq[buf] + (t_off + tt * 32 + c) * kRowStride + h * 16;
#pragma unroll
        for (int p = 0; p < 2; p++) {  // blocks 2p and 2p+1 of the quad
            v4i wv[NTW][2], xv[TTW][2];
#pragma unroll
            for (int nt = 0; nt < NTW; nt++)
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const u32x4 u = *reinterpret_cast<const u32x4 *>(wrow[nt] + (2 * p + e) * 32);
                    wv[nt][e] = v4i{int(u.x), int(u.y), int(u.z), int(u.w)};
                }
#pragma unroll
            for (int tt = 0; tt < TTW; tt++)
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const u32x4 u = *reinterpret_cast<const u32x4 *>(xrow[tt] + (2 * p + e) * 32);
                    xv[tt][e] = v4i{int(u.x), int(u.y), int(u.z), int(u.w)};
                }
#pragma unroll
            for (int nt = 0; nt < NTW; nt++)
#pragma unroll
                for (int tt = 0; tt < TTW; tt++) {
                    // blocks past n_in/32 in the last quad are zero on both sides (scale 0, quants 0):
                    // fma(float(0), 0, acc) leaves acc unchanged, so they are multiplied like the rest
                    v32f zero32;
#pragma unroll
                    for (int i = 0; i < 32; i++) zero32[i] = 0.0f;
                    const v32f s = __builtin_amdgcn_mfma_f32_32x32x1f32(xs_cur[tt][p], wd_cur[nt][p], zero32, 0, 0, 0);
                    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    const v16i d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(xv[tt][0], wv[nt][0], zero16, 0, 0, 0);
                    const v16i d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(xv[tt][1], wv[nt][1], zero16, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 16; i++) acc[nt][tt][i] = __builtin_fmaf(float(d0[i]), s[i], acc[nt][tt][i]);
#pragma unroll
                    for (int i = 0; i < 16; i++) acc[nt][tt][i] = __builtin_fmaf(float(d1[i]), s[16 + i], acc[nt][tt][i]);
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

template <int NTW, int TTW, int WN, int WT, int DEPTH>
void launch_gemm(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y, uint32_t n_tokens,
                 uint32_t y_stride, hipStream_t s) {
    constexpr uint32_t tile_n = 32 * NTW * WN, tile_t = 32 * TTW * WT;
    const uint32_t grid_n = (w->n_out + tile_n - 1) / tile_n, grid_t = (n_tokens + tile_t - 1) / tile_t;
    hipLaunchKernelGGL((gemm_q8_0_kernel<NTW, TTW, WN, WT, DEPTH>), dim3(grid_n * grid_t), dim3(64 * WN * WT), 0, s,
                       w->data, x_q8, x_scales, y, w->n_out, w->n_in, w->n_units, w->n_tiles, n_tokens, y_stride, grid_n,
                       grid_t, n_tokens < w->n_out ? 1u : 0u);
}

}  // namespace

int rmi_launch_gemm_q8_0(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                         uint32_t n_tokens, uint32_t y_stride, hipStream_t s) {
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    // Measured on MI355X: the 128x128 tile (4 waves, 2x2 sub-tiles each) is fastest once it yields two
    // workgroups per compute unit; below that the 128x64 tile of 8 single-sub-tile waves, and for small
    // problems the 64x64 tile of 4 waves, keep more SIMDs fed.  A deeper register ring (DEPTH > 1) did not pay.
    const uint64_t cus = uint64_t(rmi_device_cus());
    auto groups = [&](uint32_t tn, uint32_t tt) {
        return uint64_t((w->n_out + tn - 1) / tn) * ((n_tokens + tt - 1) / tt);
    };
    if (groups(64, 64) > 0x7fffffffull) return rmi_fail(RMI_HIP_E_INVALID, "GEMM too large for one launch");
    if (groups(128, 128) >= 2 * cus)
        launch_gemm<2, 2, 2, 2, 1>(w, x_q8, x_scales, y, n_tokens, y_stride, s);
    else if (groups(128, 64) >= 2 * cus)
        launch_gemm<1, 1, 4, 2, 1>(w, x_q8, x_scales, y, n_tokens, y_stride, s);
    else
        launch_gemm<1, 1, 2, 2, 1>(w, x_q8, x_scales, y, n_tokens, y_stride, s);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
