// Q6_K kernels: the Q6_K x Q8_K integer GEMV, its exact per-super-block lane
// integers, and the dequantise-and-dot path.
//
// GEMV arithmetic order = vec_dot_q6k_q8k_avx2 (src/ops/quant/mod.rs:964-1062):
// per row eight f32 accumulators; per super-block lane m holds one int32,
//   sum over the eight 32-element groups g of scale[2g + (m>=4)] * (the products of the
//   unsigned 6-bit quants 4m..4m+3 of the group with the int8 activations)
//   - 32 * (bsums[2m]*scale[2m] + bsums[2m+1]*scale[2m+1]),
// then acc_m = fma(d*q8d, float(that), acc_m); result hsum(acc).  Eight GPU lanes
// per row hold the eight accumulators.
#include "rmi_internal.h"

#include "device_common.h"

#include "device_run_ring.h"
#include "device_stage_q8k.h"

namespace {

__device__ __forceinline__ int sbfe(uint32_t v, uint32_t off, uint32_t width) {
    return __builtin_amdgcn_sbfe(int(v), off, width);
}

// LDS per token and super-block: 64 dwords of quants ordered [m][g] (dword m*8+g =
// elements 32g+4m..), 8 dwords of bsums (dword m = bsums[2m] | bsums[2m+1] << 16),
// 1 dword d (+3 pad) = 76 dwords.
constexpr uint32_t kSbDwords = 76;

struct SuperRegs {
    u32x4 sc;    // the row's 16 int8 scales
    uint32_t d;  // f16 d of the row
    u32x4 ql;    // low nibbles: bytes 4m.. of ql[0..32), [32..64), [64..96), [96..128)
    u32x2 qh;    // high bit pairs: bytes 4m.. of qh[0..32), [32..64)
};

// the eight groups' unsigned 6-bit quants (4 per dword) of one lane
__device__ __forceinline__ void unpack_q6(const SuperRegs &g, uint32_t (&q)[8]) {
    const uint32_t k4 = 0x0f0f0f0fu, k2 = 0x30303030u;
    const uint32_t a[2] = {g.ql.x, g.ql.z}, b[2] = {g.ql.y, g.ql.w}, h[2] = {g.qh.x, g.qh.y};
#pragma unroll
    for (int j = 0; j < 2; j++) {
        q[4 * j + 0] = (a[j] & k4) | ((h[j] << 4) & k2);
        q[4 * j + 1] = (b[j] & k4) | ((h[j] << 2) & k2);
        q[4 * j + 2] = ((a[j] >> 4) & k4) | (h[j] & k2);
        q[4 * j + 3] = ((b[j] >> 4) & k4) | ((h[j] >> 2) & k2);
    }
}

template <int B>
__device__ __forceinline__ void super_fma(float (&acc)[B], const SuperRegs &g, const uint32_t *lds_dw, uint32_t n_sb,
                                          uint32_t sb, uint32_t m) {
    const float wd = h2f(g.d);
    uint32_t q[8];
    unpack_q6(g, q);
    const uint32_t scw[4] = {g.sc.x, g.sc.y, g.sc.z, g.sc.w};
    const uint32_t hi8 = (m >> 2) * 8;  // lanes 4..7 take the odd scale of each pair
    int sc[8];
#pragma unroll
    for (int gg = 0; gg < 8; gg++) sc[gg] = sbfe(scw[gg >> 1], 16 * (gg & 1) + hi8, 8);
    // scales 2m, 2m+1 for the bsums term
    const uint32_t wsel = m < 4 ? (m < 2 ? g.sc.x : g.sc.y) : (m < 6 ? g.sc.z : g.sc.w);
    const int so0 = sbfe(wsel, 16 * (m & 1), 8), so1 = sbfe(wsel, 16 * (m & 1) + 8, 8);
#pragma unroll
    for (int t = 0; t < B; t++) {
        const uint32_t *xs = lds_dw + (size_t(t) * n_sb + sb) * kSbDwords;
        const uint4 xa = reinterpret_cast<const uint4 *>(xs + m * 8)[0];
        const uint4 xb = reinterpret_cast<const uint4 *>(xs + m * 8)[1];
        const uint32_t xd[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
        int sumi = 0;
#pragma unroll
        for (int gg = 0; gg < 8; gg++) {
            // 8-bit scale x (4 products of a 6-bit quant and an int8): both factors fit 24 bits
            sumi += __mul24(sc[gg], dot4_i8(int(q[gg]), int(xd[gg])));
        }
        const uint32_t bs = xs[64 + m];
        const int off = __mul24(sbfe(bs, 0, 16), so0) + __mul24(int(bs) >> 16, so1);
        sumi -= int(uint32_t(off) << 5);
        const float dd = B == 1 ? h2f_times<true>(g.d, __uint_as_float(xs[72])) : wd * __uint_as_float(xs[72]);
        acc[t] = __builtin_fmaf(dd, float(sumi), acc[t]);
    }
}

// Same launch shapes as the Q4_K GEMV (q4_k.hip): a wave owns a short run of consecutive
// 8-row tiles of one matrix and walks it four super-blocks deep (device_run_ring.h); up to eight waves of a
// workgroup share one staged activation.
template <int B, bool GROUPED, int MAXT>
__global__ __launch_bounds__(MAXT) void gemv_q6_k_kernel(RmiQ4kProblem single, const RmiQ4kProblem *__restrict__ list,
                                                        const uint4 *__restrict__ runs, uint32_t tiles_per_wave) {
    extern __shared__ uint4 lds[];
    const uint32_t lane = threadIdx.x & 63, r = lane >> 3, m = lane & 7;
    // wave-uniform, and said so: the problem's fields and the super-block counter live in scalar registers
    const uint32_t w_idx = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    RmiQ4kProblem p;
    uint32_t k, k_end;
    if (GROUPED) {
        const uint4 run = runs[w_idx];
        p = list[run.x];
        k = run.y;
        k_end = run.y + run.z;
    } else {
        p = single;
        k = w_idx * tiles_per_wave < p.n_tiles ? w_idx * tiles_per_wave : p.n_tiles;
        k_end = k + tiles_per_wave < p.n_tiles ? k + tiles_per_wave : p.n_tiles;
    }
    const uint32_t n_sb = p.n_sb, n_in = n_sb * 256;
    // units of the run (device_run_ring.h): one super-block of one tile, 1680 bytes, tile after tile
    const uint32_t n_units = (k_end - k) * n_sb;
    // a wave without tiles (padding of the last workgroup) prefetches from the matrix's first tile: in bounds, unused
    gptr_u4 base = as_global<gptr_u4>(p.w + size_t(p.tile0 + (n_units ? k : 0)) * n_sb * kQ6KSuperBytes);
    struct Cursor {
        gptr_u4 unit;  // the same for all lanes
        uint32_t r, lane;
        __device__ __forceinline__ void load(SuperRegs &g) const {
            g.sc = unit[r];
            g.d = ((gptr_u16)(unit + 8))[r];
            g.ql = __builtin_nontemporal_load(unit + 9 + lane);  // weights are read once: not kept in cache
            g.qh = __builtin_nontemporal_load((gptr_u2)(unit + 73) + lane);
        }
        __device__ __forceinline__ void step() { unit += kQ6KSuperBytes / 16; }
    } cur{base, r, lane};
    RmiRing<SuperRegs> ring;
    rmi_ring_fill(ring, n_units, cur);
    uint32_t *lds_dw = reinterpret_cast<uint32_t *>(lds);
    for (int t = 0; t < B; t++)
        rmi_stage_q8k_token<false, 2>(lds_dw + size_t(t) * n_sb * kSbDwords, p.q8qs + size_t(t) * n_in,
                                      p.q8bs + size_t(t) * (n_in / 16), p.q8d + size_t(t) * n_sb, n_sb, threadIdx.x,
                                      blockDim.x);
    __syncthreads();

    float acc[B];
#pragma unroll
    for (int t = 0; t < B; t++) acc[t] = 0.0f;
    RmiRunResults<B> out{};
    uint32_t sb = 0;
    gptr_f32_w yp = as_global<gptr_f32_w>(p.y);
    auto consume = [&](const SuperRegs &g) {
        super_fma<B>(acc, g, lds_dw, n_sb, sb, m);
        if (++sb == n_sb) {
            float y[B];
#pragma unroll
            for (int t = 0; t < B; t++) {
                y[t] = hsum8_lanes(acc[t]);  // the same in the row's eight lanes
                acc[t] = 0.0f;
            }
            sb = 0;
            out.keep(y, m);
            if (out.group_full()) out.flush(yp, p.y_stride, p.tile0 + k, r, m, p.row_start, p.row_end);
        }
    };
    rmi_ring_walk(ring, n_units, cur, consume);
    if (out.pending()) out.flush(yp, p.y_stride, p.tile0 + k, r, m, p.row_start, p.row_end);
}

// ---- the eight exact lane integers per (row, super-block), read back from the repacked stream
__global__ __launch_bounds__(256) void block_lanes_q6_k_kernel(const uint8_t *__restrict__ w,
                                                                const int8_t *__restrict__ q8qs,
                                                                const int16_t *__restrict__ q8bs,
                                                                int32_t *__restrict__ lanes, uint32_t n_out,
                                                                uint32_t n_sb) {
    const uint64_t total = uint64_t(n_out) * n_sb * 8;
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < total;
         i += uint64_t(gridDim.x) * blockDim.x) {
        const uint32_t m = uint32_t(i & 7), sb = uint32_t((i >> 3) % n_sb), row = uint32_t((i >> 3) / n_sb);
        const uint8_t *chunk = w + (size_t(row >> 3) * n_sb + sb) * kQ6KSuperBytes;
        const int8_t *sc = reinterpret_cast<const int8_t *>(chunk + (row & 7) * 16);
        const uint4 qlv = reinterpret_cast<const uint4 *>(chunk + 144)[(row & 7) * 8 + m];
        const uint2 qhv = reinterpret_cast<const uint2 *>(chunk + 144 + 1024)[(row & 7) * 8 + m];
        SuperRegs g;
        g.ql.x = qlv.x, g.ql.y = qlv.y, g.ql.z = qlv.z, g.ql.w = qlv.w;
        g.qh.x = qhv.x, g.qh.y = qhv.y;
        uint32_t q[8];
        unpack_q6(g, q);
        const uint32_t *xq = reinterpret_cast<const uint32_t *>(q8qs + size_t(sb) * 256);
        int s = 0;
        for (uint32_t gg = 0; gg < 8; gg++) s += int(sc[2 * gg + (m >> 2)]) * dot4_i8(int(q[gg]), int(xq[8 * gg + m]));
        const int off = int(q8bs[sb * 16 + 2 * m]) * int(sc[2 * m]) + int(q8bs[sb * 16 + 2 * m + 1]) * int(sc[2 * m + 1]);
        lanes[i] = s - int(uint32_t(off) << 5);
    }
}

// ---- dequantise-and-dot, one lane per row, strictly sequential f32 sum over the
// elements of the row (q6_k.rs:83-119); element value (d*sc)*q as in
// dequantize_row_q6_k (quant/mod.rs:530-569); x rebuilt as q8*scale per element.
__global__ __launch_bounds__(64) void q6_k_dequant_dot_kernel(const uint8_t *__restrict__ w,
                                                               const int8_t *__restrict__ x_q8,
                                                               const float *__restrict__ x_scales,
                                                               float *__restrict__ y, uint32_t n_sb, uint32_t row_start,
                                                               uint32_t row_end) {
    const uint32_t row = row_start + blockIdx.x * 64 + threadIdx.x;
    if (row >= row_end) return;
    float sum = 0.0f;
    for (uint32_t sb = 0; sb < n_sb; sb++) {
        const uint8_t *chunk = w + (size_t(row >> 3) * n_sb + sb) * kQ6KSuperBytes;
        const int8_t *sc = reinterpret_cast<const int8_t *>(chunk + (row & 7) * 16);
        const float d = h2f(reinterpret_cast<const uint16_t *>(chunk + 128)[row & 7]);
        uint32_t q[8][8];  // [m][g]
#pragma unroll
        for (int m = 0; m < 8; m++) {
            const uint4 qlv = reinterpret_cast<const uint4 *>(chunk + 144)[(row & 7) * 8 + m];
            const uint2 qhv = reinterpret_cast<const uint2 *>(chunk + 144 + 1024)[(row & 7) * 8 + m];
            SuperRegs g;
            g.ql.x = qlv.x, g.ql.y = qlv.y, g.ql.z = qlv.z, g.ql.w = qlv.w;
            g.qh.x = qhv.x, g.qh.y = qhv.y;
            unpack_q6(g, q[m]);
        }
#pragma unroll
        for (int gg = 0; gg < 8; gg++) {
#pragma unroll
            for (int m = 0; m < 8; m++) {
                const float dsc = d * float(int(sc[2 * gg + (m >> 2)]));
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int qv = int((q[m][gg] >> (8 * i)) & 0xffu) - 32;
                    const float wv = dsc * float(qv);
                    const uint32_t k = sb * 256 + 32 * gg + 4 * m + i;
                    const float xv = float(int(x_q8[k])) * x_scales[k >> 5];
                    const float prod = wv * xv;
                    sum = sum + prod;
                }
            }
        }
    }
    y[row] = sum;
}

// The same sum for 16 rows per workgroup with the work split by kind, as for Q4_K (q4_k.hip): the sum of a row
// is one chain of f32 adds in element order, about eight clocks an add on one lane; what feeds it has no order.
// Two producer waves turn one super-block of the 16 rows into products in LDS (a lane takes piece m of a row:
// 32 elements) while a third wave, one lane per row, adds the previous super-block's products in order, its
// LDS reads 32 values ahead; one barrier per super-block.  The activation is rebuilt as q8 * scale once, in LDS.
constexpr uint32_t kDdRows = 16, kDdProducers = kDdRows * 8, kDdThreads = kDdProducers + 64;
__global__ __launch_bounds__(kDdThreads) void q6_k_dequant_dot_split_kernel(
    const uint8_t *__restrict__ w, const int8_t *__restrict__ x_q8, const float *__restrict__ x_scales,
    float *__restrict__ y, uint32_t n_sb, uint32_t n_tiles, uint32_t row_start, uint32_t row_end) {
    extern __shared__ float4 dd_lds[];
    float4 *prod = dd_lds;                                             // [2][64 float4 per row][16 rows]
    float *xs = reinterpret_cast<float *>(dd_lds + 2 * 64 * kDdRows);  // [n_in]
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t row0 = (row_start / kDdRows + blockIdx.x) * kDdRows;  // first row of this workgroup
    const uint32_t n_in = n_sb * 256;
    for (uint32_t k = tid; k < n_in; k += kDdThreads) xs[k] = float(int(x_q8[k])) * x_scales[k >> 5];
    __syncthreads();

    // producer lane: row pr of the 16, piece m of its super-block
    const uint32_t pid = tid % kDdProducers, pr = pid % kDdRows, m = pid / kDdRows;
    const bool producer = tid < kDdProducers;
    uint32_t ptile = (row0 + pr) >> 3;
    if (ptile >= n_tiles) ptile = n_tiles - 1;  // rows past the padded stream: in bounds, never stored
    const uint8_t *ptile_base = w + size_t(ptile) * n_sb * kQ6KSuperBytes;
    const uint32_t r8 = (row0 + pr) & 7;
    auto produce = [&](uint32_t sb) {
        const uint8_t *chunk = ptile_base + size_t(sb) * kQ6KSuperBytes;
        const int8_t *sc = reinterpret_cast<const int8_t *>(chunk + r8 * 16);
        const float d = h2f(reinterpret_cast<const uint16_t *>(chunk + 128)[r8]);
        const uint4 qlv = reinterpret_cast<const uint4 *>(chunk + 144)[r8 * 8 + m];
        const uint2 qhv = reinterpret_cast<const uint2 *>(chunk + 144 + 1024)[r8 * 8 + m];
        SuperRegs g;
        g.ql.x = qlv.x, g.ql.y = qlv.y, g.ql.z = qlv.z, g.ql.w = qlv.w;
        g.qh.x = qhv.x, g.qh.y = qhv.y;
        uint32_t q[8];
        unpack_q6(g, q);
        float4 *dst = prod + size_t(sb & 1) * 64 * kDdRows + pr;
        const float4 *xsb = reinterpret_cast<const float4 *>(xs + sb * 256);
#pragma unroll
        for (int gg = 0; gg < 8; gg++) {
            const float dsc = d * float(int(sc[2 * gg + (m >> 2)]));
            const uint32_t k4 = 8 * gg + m;  // elements 4 k4 .. 4 k4 + 3 of the super-block
            const float4 xv = xsb[k4];
            const float xe[4] = {xv.x, xv.y, xv.z, xv.w};
            float pe[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int qv = int((q[gg] >> (8 * i)) & 0xffu) - 32;
                const float wv = dsc * float(qv);
                pe[i] = wv * xe[i];
            }
            dst[size_t(k4) * kDdRows] = make_float4(pe[0], pe[1], pe[2], pe[3]);
        }
    };
    if (producer) produce(0);
    __syncthreads();
    float sum = 0.0f;
    for (uint32_t sb = 0; sb < n_sb; sb++) {
        if (producer) {
            if (sb + 1 < n_sb) produce(sb + 1);
        } else if (lane < kDdRows) {
            const float4 *src = prod + size_t(sb & 1) * 64 * kDdRows + lane;
            float4 a[8], b[8];
#pragma unroll
            for (int j = 0; j < 8; j++) a[j] = src[size_t(j) * kDdRows];
#pragma unroll
            for (int blk = 0; blk < 4; blk++) {  // 16 float4 per round, the reads 8 float4 ahead of the adds
#pragma unroll
                for (int j = 0; j < 8; j++) b[j] = src[size_t(16 * blk + 8 + j) * kDdRows];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    sum = sum + a[j].x;
                    sum = sum + a[j].y;
                    sum = sum + a[j].z;
                    sum = sum + a[j].w;
                }
                if (blk < 3) {
#pragma unroll
                    for (int j = 0; j < 8; j++) a[j] = src[size_t(16 * blk + 16 + j) * kDdRows];
                }
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    sum = sum + b[j].x;
                    sum = sum + b[j].y;
                    sum = sum + b[j].z;
                    sum = sum + b[j].w;
                }
            }
        }
        __syncthreads();
    }
    const uint32_t row = row0 + lane;
    if (!producer && lane < kDdRows && row >= row_start && row < row_end) y[row] = sum;
}

template <int B>
int launch_gemv_q6k(const RmiQ4kProblem *single, const RmiQ4kProblem *d_list, const uint4 *d_runs, uint32_t n_waves,
                    uint32_t wpg, uint32_t tiles_per_wave, uint32_t max_n_sb, hipStream_t s) {
    const size_t lds_bytes = size_t(B) * max_n_sb * kSbDwords * 4;
    if (lds_bytes > 64 * 1024)
        return rmi_fail(RMI_HIP_E_INVALID, "activation of %d tokens x %u elements does not fit the LDS staging", B,
                        max_n_sb * 256);
    const dim3 grid_single((n_waves + wpg - 1) / wpg), grid_group(n_waves / wpg), block(64 * wpg);
    if (single && wpg == 1)
        hipLaunchKernelGGL((gemv_q6_k_kernel<B, false, 64>), grid_single, block, lds_bytes, s, *single, d_list, d_runs,
                           tiles_per_wave);
    else if (single)
        hipLaunchKernelGGL((gemv_q6_k_kernel<B, false, 512>), grid_single, block, lds_bytes, s, *single, d_list, d_runs,
                           tiles_per_wave);
    else if (wpg == 1)
        hipLaunchKernelGGL((gemv_q6_k_kernel<B, true, 64>), grid_group, block, lds_bytes, s, RmiQ4kProblem{}, d_list, d_runs,
                           tiles_per_wave);
    else
        hipLaunchKernelGGL((gemv_q6_k_kernel<B, true, 512>), grid_group, block, lds_bytes, s, RmiQ4kProblem{}, d_list, d_runs,
                           tiles_per_wave);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int dispatch_q6k(uint32_t nt, const RmiQ4kProblem *single, const RmiQ4kProblem *d_list, const uint4 *d_runs,
                 uint32_t n_waves, uint32_t wpg, uint32_t tpw, uint32_t max_n_sb, hipStream_t s) {
    if (n_waves == 0) return RMI_HIP_OK;
    switch (nt) {
        case 1: return launch_gemv_q6k<1>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 2: return launch_gemv_q6k<2>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 3: return launch_gemv_q6k<3>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 4: return launch_gemv_q6k<4>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 5: return launch_gemv_q6k<5>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 6: return launch_gemv_q6k<6>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 7: return launch_gemv_q6k<7>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 8: return launch_gemv_q6k<8>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        default: return rmi_fail(RMI_HIP_E_INVALID, "gemv takes 1..8 tokens per launch, got %u", nt);
    }
}

}  // namespace

// Tiles a wave takes in one run: about 16 tile-super-blocks (26 KiB of weights), 32 with more than one token.
uint32_t rmi_q6k_tiles_per_wave(uint32_t n_sb, uint32_t launch_tiles, uint32_t n_tokens) {
    const uint32_t target = n_tokens > 1 ? 32 : 16;
    uint32_t tpw = n_sb >= target ? 1 : target / (n_sb ? n_sb : 1);
    const uint32_t fill = uint32_t(rmi_device_cus()) * 8;
    while (tpw > 1 && launch_tiles / tpw < fill) tpw >>= 1;
    return tpw ? tpw : 1;
}

int rmi_launch_gemv_q6_k(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums, float *y,
                         uint32_t n_tokens, uint32_t y_stride, uint32_t row_start, uint32_t row_end, hipStream_t s) {
    if (row_start >= row_end || n_tokens == 0 || w->n_units == 0) return RMI_HIP_OK;
    const size_t per_token = size_t(w->n_units) * kSbDwords * 4;
    uint32_t chunk = uint32_t((64 * 1024) / per_token);
    if (chunk == 0) return rmi_fail(RMI_HIP_E_INVALID, "n_in=%u is too long for the GEMV staging", w->n_in);
    if (chunk > 8) chunk = 8;
    const uint32_t n_sb = w->n_units;
    for (uint32_t t0 = 0; t0 < n_tokens; t0 += chunk) {
        const uint32_t nt = n_tokens - t0 < chunk ? n_tokens - t0 : chunk;
        RmiQ4kProblem p = rmi_make_q4k_problem(w, d + size_t(t0) * n_sb, qs + size_t(t0) * w->n_in,
                                               bsums + size_t(t0) * (w->n_in / 16), y + size_t(t0) * y_stride, y_stride,
                                               row_start, row_end);
        const uint32_t tpw = rmi_q6k_tiles_per_wave(n_sb, p.n_tiles, nt);
        const uint32_t wpg =
            rmi_gemv_waves_per_group(size_t(nt) * n_sb * kSbDwords * 4, size_t(tpw) * n_sb * kQ6KSuperBytes);
        int rc = dispatch_q6k(nt, &p, nullptr, nullptr, (p.n_tiles + tpw - 1) / tpw, wpg, tpw, n_sb, s);
        if (rc != RMI_HIP_OK) return rc;
    }
    return RMI_HIP_OK;
}

int rmi_launch_gemv_q6_k_group(const RmiQ4kProblem *d_list, const uint4 *d_runs, uint32_t n_runs, uint32_t wpg,
                               uint32_t max_n_sb, uint32_t n_tokens, hipStream_t s) {
    return dispatch_q6k(n_tokens, nullptr, d_list, d_runs, n_runs, wpg, 0, max_n_sb, s);
}

int rmi_launch_block_lanes_q6_k(const rmi_hip_weight *w, const int8_t *qs, const int16_t *bsums, int32_t *lanes,
                                hipStream_t s) {
    const uint64_t total = uint64_t(w->n_out) * w->n_units * 8;
    if (total == 0) return RMI_HIP_OK;
    const uint32_t grid = uint32_t(total / 256 + 1 < 65535 ? total / 256 + 1 : 65535);
    hipLaunchKernelGGL(block_lanes_q6_k_kernel, dim3(grid), dim3(256), 0, s, w->data, qs, bsums, lanes, w->n_out,
                       w->n_units);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_launch_q6_k_dequant_dot(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                                uint32_t row_start, uint32_t row_end, hipStream_t s) {
    if (row_start >= row_end) return RMI_HIP_OK;
    const size_t lds_bytes = size_t(2) * 64 * kDdRows * 16 + size_t(w->n_in) * 4;
    if (lds_bytes <= 160 * 1024 && w->n_units > 0) {
        static const bool raised = [] {  // more than 64 KiB of dynamic LDS has to be asked for once
            return hipFuncSetAttribute(reinterpret_cast<const void *>(q6_k_dequant_dot_split_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess;
        }();
        if (raised || lds_bytes <= 64 * 1024) {
            const uint32_t grid = (row_end - 1) / kDdRows - row_start / kDdRows + 1;
            hipLaunchKernelGGL(q6_k_dequant_dot_split_kernel, dim3(grid), dim3(kDdThreads), lds_bytes, s, w->data, x_q8,
                               x_scales, y, w->n_units, w->n_tiles, row_start, row_end);
            RMI_HIP_CHECK(hipGetLastError());
            return RMI_HIP_OK;
        }
    }
    const uint32_t grid = (row_end - row_start + 63) / 64;
    hipLaunchKernelGGL(q6_k_dequant_dot_kernel, dim3(grid), dim3(64), 0, s, w->data, x_q8, x_scales, y, w->n_units,
                       row_start, row_end);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
