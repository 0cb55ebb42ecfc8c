// Q8_0 x Q8_0 prefill GEMM for products whose tile grid is smaller than the chip (tens to a few hundred tokens):
// Y[t][n] = sum_b (f32(wd[n][b]) * xs[t][b]) * dot_b(W[n], X[t])  (Kernel::forward_batched, every token an independent
// GEMV, src/ops/kernel/trait_.rs:78-109).
//
// The tiled kernel of gemm_q8_0.hip keeps the aarch64 kernel's single f32 chain per output (neon.rs:49-73), so a tile
// walks the blocks of its rows one after the other: with 64 tokens a launch is 16 to 48 workgroups on 256 compute
// units, each running a chain of up to 96 dependent steps.  Here a workgroup is ONE 32-row x 32-token MFMA tile and
// its waves split the row's blocks between them: wave v takes the quads (4 blocks, 128 elements) [v * per, (v + 1) *
// per), adds them from zero in block order, acc = fma(float(dot_b), wd * xs, acc), with the exact int32 block dot
// from v_mfma_i32_32x32x32_i8 and the exact f32 scale product from v_mfma_f32_32x32x2_f32 (one product plus zero,
// correctly rounded whatever the scales are); the waves' sums meet in LDS and are added in wave order,
// ((p0 + p1) + p2) + ...  The result is deterministic, the same for a token whatever batch it arrives in (the split
// depends on the row length only), and built from exact integer block dots; it is not the single chain, and agrees
// with the CPU kernels within the reference's tolerance (1e-4 + 1e-4 |ref|), not bit for bit.
//
// No operand is used twice inside a workgroup, so LDS is not there for reuse but for the memory pipeline: it
// serves a quad of lanes per step, and a quad that reads 64 consecutive bytes takes one step, a quad that reads
// from four rows takes four.  A wave therefore loads its quad of the 32 rows and of the 32 tokens as it lies in
// memory (16 bytes a lane, eight lanes a row: whole lines), writes both into a region of LDS that is its own (the
// weight pieces of the GEMV tile stream, 4-byte slices of four blocks, are scattered into block order on the way),
// and reads the MFMA operands back, lane (row c, half h): bytes 16h..16h+15 of block b.  Nothing is shared between
// waves, so there is no barrier before the last one, where the sums meet.
#include "rmi_internal.h"

#include "device_common.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr uint32_t kKsplitMaxWaves = 16;
constexpr uint32_t kRowStride = 144;                   // bytes between LDS rows: 16-byte reads of 8 rows fall into 8 bank groups
constexpr uint32_t kOperandBytes = 32 * kRowStride;    // one quad of 32 rows or 32 tokens
constexpr uint32_t kWaveBytes = 2 * kOperandBytes;     // a wave's region: weights, tokens

struct QuadLoads {  // what a lane loads for one quad
    u32x4 w[4];   // load j: piece lane % 8 (4-byte slice of blocks 0..3) of row 8 j + lane / 8
    u32x4 x[4];   // load j: bytes 16 (lane % 8) .. + 15 of the quad of token 8 j + lane / 8
    u32x2 wd;     // the four f16 block scales of row lane % 32
    u32x4 xs;     // the four f32 block scales of token lane % 32
};

// RAGGED: n_in / 32 is not a multiple of 4 (the last quad is partly padding: the stream's quants and scales there are
// zero, the token's are not there) or the token scales are not 16-byte aligned.
template <bool RAGGED>
__global__ __launch_bounds__(64 * kKsplitMaxWaves) void gemm_q8_0_ksplit_kernel(
    const uint8_t *__restrict__ w, const int8_t *__restrict__ x_q8, const float *__restrict__ x_scales, float *__restrict__ y,
    uint32_t n_out, uint32_t n_in, uint32_t n_oct, uint32_t n_tiles, uint32_t n_tokens, uint32_t y_stride, uint32_t grid_n,
    uint32_t grid_t, uint32_t t_fastest, uint32_t per) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // [waves][kWaveBytes], then as float sums[waves][16][64]
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = uint32_t(__builtin_amdgcn_readfirstlane(int(tid >> 6)));
    const uint32_t n_waves = blockDim.x >> 6;
    const uint32_t c = lane & 31, h = lane >> 5;
    uint32_t n_tile, t_tile;
    rmi_gemm_tile_of(blockIdx.x, grid_n, grid_t, t_fastest, 0, n_tile, t_tile);
    const uint32_t n0 = n_tile * 32, t0 = t_tile * 32;
    const uint32_t nb = n_in >> 5, n_quads = (nb + 3) >> 2;
    const uint32_t q_begin = wave * per, q_end = q_begin + per < n_quads ? q_begin + per : n_quads;

    // ---- addresses.  Rows past the padded stream and tokens past the input read the last one again; their
    // results are not stored.
    const uint32_t r8 = lane >> 3, p8 = lane & 7;
    const uint8_t *w_ld[4];
    const int8_t *x_ld[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        uint32_t tile = (n0 >> 3) + j;
        if (tile >= n_tiles) tile = n_tiles - 1;
        w_ld[j] = w + size_t(tile) * n_oct * kOctetBytes + size_t(n_oct) * 128 + lane * 16;
        const uint32_t tok = t0 + 8 * j + r8 < n_tokens ? t0 + 8 * j + r8 : n_tokens - 1;
        x_ld[j] = x_q8 + size_t(tok) * n_in + p8 * 16;
    }
    uint32_t row_tile = (n0 + c) >> 3;
    if (row_tile >= n_tiles) row_tile = n_tiles - 1;
    const uint8_t *wd_row = w + size_t(row_tile) * n_oct * kOctetBytes + ((n0 + c) & 7) * 16;
    const float *xs_row = x_scales + size_t(t0 + c < n_tokens ? t0 + c : n_tokens - 1) * nb;

    auto load_quad = [&](QuadLoads &o, uint32_t q) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; j++) o.w[j] = *reinterpret_cast<const u32x4 *>(w_ld[j] + size_t(q) * 1024);
        o.wd = *reinterpret_cast<const u32x2 *>(wd_row + size_t(q >> 1) * 128 + (q & 1) * 8);
        if (RAGGED) {
            // a piece past the row end meets zero weight quants: any bytes will do, the last piece of the row is read
            const int32_t rel = q * 128 + p8 * 16 + 16 <= n_in ? int32_t(q * 128) : int32_t(n_in) - 16 - int32_t(p8 * 16);
#pragma unroll
            for (int j = 0; j < 4; j++) o.x[j] = *reinterpret_cast<const u32x4 *>(x_ld[j] + rel);
#pragma unroll
            for (int j = 0; j < 4; j++) o.xs[j] = __builtin_bit_cast(uint32_t, xs_row[q * 4 + j < nb ? q * 4 + j : nb - 1]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) o.x[j] = *reinterpret_cast<const u32x4 *>(x_ld[j] + size_t(q) * 128);
            o.xs = *reinterpret_cast<const u32x4 *>(xs_row + size_t(q) * 4);
        }
    };

    uint8_t *my_w = lds + wave * kWaveBytes, *my_x = my_w + kOperandBytes;
    const uint32_t w_st = r8 * kRowStride + p8 * 4, x_st = r8 * kRowStride + p8 * 16;
    const uint32_t rd = c * kRowStride + h * 16;
    auto stage_quad = [&](const QuadLoads &o) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint8_t *dst = my_w + j * 8 * kRowStride + w_st;
            *reinterpret_cast<uint32_t *>(dst) = o.w[j].x;
            *reinterpret_cast<uint32_t *>(dst + 32) = o.w[j].y;
            *reinterpret_cast<uint32_t *>(dst + 64) = o.w[j].z;
            *reinterpret_cast<uint32_t *>(dst + 96) = o.w[j].w;
            *reinterpret_cast<u32x4 *>(my_x + j * 8 * kRowStride + x_st) = o.x[j];
        }
    };

    const v16f zero16f = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    v16f acc = zero16f;

    auto fold_quad = [&](u32x2 wd, u32x4 xs, uint32_t q) __attribute__((always_inline)) {
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const u32x4 wu = *reinterpret_cast<const u32x4 *>(my_w + rd + b * 32);
            const u32x4 xu = *reinterpret_cast<const u32x4 *>(my_x + rd + b * 32);
            const v4i wo = {int(wu.x), int(wu.y), int(wu.z), int(wu.w)};
            const v4i xo = {int(xu.x), int(xu.y), int(xu.z), int(xu.w)};
            // the scale product's operands: k slot 0 in lanes 0..31, slot 1 (zero on both sides) in lanes 32..63;
            // a scale past n_in/32 must be a true zero: its block's dot is zero and the product must not be NaN
            const uint32_t wd_bits = b < 2 ? wd.x : wd.y;
            const float wd_f = h ? 0.0f : h2f((b & 1) ? wd_bits >> 16 : wd_bits & 0xffffu);
            const uint32_t xs_bits = xs[b];  // (a bit_cast of the vector element itself reads element 0)
            float xs_f = h ? 0.0f : __builtin_bit_cast(float, xs_bits);
            if (RAGGED && q * 4 + b >= nb) xs_f = 0.0f;
            const v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(xo, wo, zero16, 0, 0, 0);
            const v16f sp = __builtin_amdgcn_mfma_f32_32x32x2f32(xs_f, wd_f, zero16f, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 16; i++) acc[i] = __builtin_fmaf(float(d[i]), sp[i], acc[i]);
        }
    };

    // A wave's quads one after the other: the quad goes from its registers to LDS, the registers take the next
    // quad's loads, the quad is folded out of LDS.  The LDS unit works through a wave's accesses in order, so the
    // reads find what the writes before them put there, and the next quad's writes come after this quad's reads.
    if (q_begin < q_end) {
        QuadLoads ld;
        load_quad(ld, q_begin);
        for (uint32_t q = q_begin; q < q_end; q++) {
            const u32x2 wd = ld.wd;
            const u32x4 xs = ld.xs;
            stage_quad(ld);
            rmi_wave_lds_fence();  // the lanes read each other's pieces (the loop has no divergent branch that the next
                                   // quad's writes could be moved past this quad's reads through; a second barrier
                                   // behind the reads costs 7 %: it also keeps the fold's tail from overlapping them)
            load_quad(ld, q + 1 < q_end ? q + 1 : q);
            fold_quad(wd, xs, q);
        }
    }
    __syncthreads();  // every wave is done with its staging region: the sums take the same memory
    float *sums = reinterpret_cast<float *>(lds);
#pragma unroll
    for (int i = 0; i < 16; i++) sums[(wave * 16 + i) * 64 + lane] = acc[i];
    __syncthreads();
    // the waves' sums in wave order; output o = i * 64 + lane of the tile belongs to lane (c, h), register i:
    // row n0 + c, token t0 + 8 (i / 4) + 4 h + i % 4
    for (uint32_t o = tid; o < 1024; o += blockDim.x) {
        float total = sums[o];
        for (uint32_t v = 1; v < n_waves; v++) total += sums[v * 1024 + o];
        const uint32_t i = o >> 6, l = o & 63;
        const uint32_t n = n0 + (l & 31), t = t0 + 8 * (i >> 2) + 4 * (l >> 5) + (i & 3);
        if (n < n_out && t < n_tokens) y[size_t(t) * y_stride + n] = total;
    }
}

// LDS of a launch with this many waves: each wave's staging region (which also holds the 4 KiB of its sums later)
size_t ksplit_lds_bytes(uint32_t n_waves) { return size_t(n_waves) * kWaveBytes; }

bool ksplit_lds_opt_in() {  // 16 waves take 144 KiB: more than the 64 KiB a kernel gets without asking
    static const bool ok = [] {
        const bool a = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q8_0_ksplit_kernel<false>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, int(ksplit_lds_bytes(kKsplitMaxWaves))) == hipSuccess;
        const bool b = hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q8_0_ksplit_kernel<true>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, int(ksplit_lds_bytes(kKsplitMaxWaves))) == hipSuccess;
        if (!(a && b)) (void)hipGetLastError();
        return a && b;
    }();
    return ok;
}

}  // namespace

// quads a wave takes, and the waves of a workgroup: a function of the row length alone, so that a token's result
// does not depend on the batch it arrives in
void rmi_gemm_q8_0_ksplit_shape(uint32_t n_in, uint32_t *quads_per_wave, uint32_t *n_waves) {
    const uint32_t n_quads = (n_in / 32 + 3) / 4;
    const uint32_t per = (n_quads + kKsplitMaxWaves - 1) / kKsplitMaxWaves;
    *quads_per_wave = per ? per : 1;
    *n_waves = per ? (n_quads + per - 1) / per : 1;
}

// The launch time to expect, in microseconds, as measured on MI355X: flat while the tiles fit the chip at once
// (launch, one round trip to memory, a wave's few steps, the sums), then about a nanosecond per tile and quad (every
// tile fetches its rows and its tokens through L2 and passes them through LDS once).
double rmi_gemm_q8_0_ksplit_cost_us(const rmi_hip_weight *w, uint32_t n_tokens) {
    const double n_quads = double((w->n_in / 32 + 3) / 4);
    const double tiles = double((w->n_out + 31) / 32) * double((n_tokens + 31) / 32);
    const double at_once = double(rmi_device_cus() > 0 ? rmi_device_cus() : 1);
    return 3.7 + 0.11 * n_quads + (tiles > at_once ? (tiles - at_once) * n_quads * 1.0e-3 : 0.0);
}

int rmi_launch_gemm_q8_0_ksplit(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                                uint32_t n_tokens, uint32_t y_stride, hipStream_t s) {
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    if (w->n_in < 32) return rmi_fail(RMI_HIP_E_INVALID, "GEMM needs at least one block per row");
    uint32_t per, n_waves;
    rmi_gemm_q8_0_ksplit_shape(w->n_in, &per, &n_waves);
    const uint32_t grid_n = (w->n_out + 31) / 32, grid_t = (n_tokens + 31) / 32;
    if (uint64_t(grid_n) * grid_t > 0x7fffffffull) return rmi_fail(RMI_HIP_E_INVALID, "GEMM too large for one launch");
    const bool ragged = (w->n_in / 32) % 4 != 0 || (reinterpret_cast<uintptr_t>(x_scales) & 15) != 0;
    const size_t lds = ksplit_lds_bytes(n_waves);
    if (lds > 64 * 1024 && !ksplit_lds_opt_in()) return rmi_fail(RMI_HIP_E_RUNTIME, "the GEMM's %zu bytes of LDS were refused", lds);
    const uint32_t t_fastest = n_tokens < w->n_out ? 1u : 0u;
    if (ragged)
        hipLaunchKernelGGL(gemm_q8_0_ksplit_kernel<true>, dim3(grid_n * grid_t), dim3(64 * n_waves), lds, s, w->data, x_q8, x_scales, y,
                           w->n_out, w->n_in, w->n_units, w->n_tiles, n_tokens, y_stride, grid_n, grid_t, t_fastest, per);
    else
        hipLaunchKernelGGL(gemm_q8_0_ksplit_kernel<false>, dim3(grid_n * grid_t), dim3(64 * n_waves), lds, s, w->data, x_q8, x_scales, y,
                           w->n_out, w->n_in, w->n_units, w->n_tiles, n_tokens, y_stride, grid_n, grid_t, t_fastest, per);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
