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

#include "device_common.h"

#include "device_run_ring.h"
#include "device_stage_q8k.h"

namespace {

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

struct SuperRegs {
    u32x4 hdr;  // f16 d, f16 dmin, 12 packed scale bytes of the row
    u32x4 qv;   // dwords 32g+4T (g = 0..3) of the row's nibble bytes
};

template <int B>
__device__ __forceinline__ void super_fma(float (&acc)[B], float (&acc_m)[B], const SuperRegs &g,
                                          const uint32_t *lds_dw, uint32_t n_sb, uint32_t sb, uint32_t T) {
    const float wd = h2f(g.hdr.x & 0xffffu), wdmin = h2f(g.hdr.x >> 16);
    uint4 sm = unpack_scales(g.hdr.y, g.hdr.z, g.hdr.w);
    // the eight scales stay whole bytes of two registers: the multiplies below then select their byte themselves
    // (SDWA) instead of a bit-field extract per scale from the packed source
    asm("" : "+v"(sm.x), "+v"(sm.y));
    const uint32_t qd[4] = {g.qv.x, g.qv.y, g.qv.z, g.qv.w};
    // mins 2T and 2T+1 (mod 8) are neighbours in one dword of the unpacked eight
    const uint32_t mn_dw = (T & 2) ? sm.w : sm.z;
    const int mn0 = int(__builtin_amdgcn_ubfe(mn_dw, 16 * (T & 1), 8)), mn1 = int(__builtin_amdgcn_ubfe(mn_dw, 16 * (T & 1) + 8, 8));
#pragma unroll
    for (int t = 0; t < B; t++) {
        const uint32_t *xs = lds_dw + (size_t(t) * n_sb + sb) * kSbDwords;
        const uint4 xa = reinterpret_cast<const uint4 *>(xs + T * 8)[0];
        const uint4 xb = reinterpret_cast<const uint4 *>(xs + T * 8)[1];
        const uint32_t xd[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
        int sumi = 0;
#pragma unroll
        for (int gg = 0; gg < 4; gg++) {
            const int lo = int(qd[gg] & 0x0f0f0f0fu), hi = int((qd[gg] >> 4) & 0x0f0f0f0fu);
            const int dl = dot4_i8(lo, int(xd[2 * gg]));
            const int dh = dot4_i8(hi, int(xd[2 * gg + 1]));
            // 6-bit scale x (4 products of a nibble and an int8): both factors fit 24 bits, full-rate multiply-add
            sumi += __mul24(int(byte_of(sm.x, sm.y, 2 * gg)), dl) + __mul24(int(byte_of(sm.x, sm.y, 2 * gg + 1)), dh);
        }
        const float d8 = __uint_as_float(xs[72]);
        const float dd = B == 1 ? h2f_times<true>(g.hdr.x & 0xffffu, d8) : wd * d8;
        const float dm = B == 1 ? -h2f_times<true>(g.hdr.x >> 16, d8) : (-wdmin) * d8;
        acc[t] = __builtin_fmaf(dd, float(sumi), acc[t]);
        const int s0 = int(xs[64 + ((2 * T) & 7)]), s1 = int(xs[64 + ((2 * T + 1) & 7)]);
        const int prod = __mul24(mn0, s0) + __mul24(mn1, s1);  // 6-bit min x 16-bit pair sum
        acc_m[t] = __builtin_fmaf(dm, float(prod), acc_m[t]);
    }
}

// A wave owns a short run of consecutive 8-row tiles of one matrix and walks it four super-blocks deep
// (device_run_ring.h); a launch has far more waves than fit on the chip (see gemv_q8_0.hip).
// GROUPED = false: one matrix (`single`), run w starts at tile w * tiles_per_wave.
// GROUPED = true: runs[w] = {problem index, first tile, tile count, -}.
// MAXT = 64: one wave per workgroup; 512: up to eight waves sharing one staged activation
template <int B, bool GROUPED, int MAXT>
__global__ __launch_bounds__(MAXT) void gemv_q4_k_kernel(RmiQ4kProblem single, const RmiQ4kProblem *__restrict__ list,
                                                        const uint4 *__restrict__ runs, uint32_t tiles_per_wave) {
    extern __shared__ uint4 lds[];
    const uint32_t lane = threadIdx.x & 63, r = lane >> 3, T = lane & 7;
    // the same for all lanes of the wave: said so, the problem's fields, the super-block counter and the
    // staged activation's offsets live in scalar registers and the tile-end test is a scalar branch
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
    // units of the run (device_run_ring.h): one super-block of one tile, 1152 bytes, tile after tile
    const uint32_t n_units = (k_end - k) * n_sb;
    // a wave without tiles (padding of the last workgroup) prefetches from the matrix's first tile: in bounds, unused
    gptr_u4 base = as_global<gptr_u4>(p.w + size_t(p.tile0 + (n_units ? k : 0)) * n_sb * kQ4KSuperBytes);
    struct Cursor {
        gptr_u4 unit;  // the same for all lanes
        uint32_t r, lane;
        __device__ __forceinline__ void load(SuperRegs &g) const {
            g.hdr = unit[r];
            g.qv = __builtin_nontemporal_load(unit + 8 + lane);  // weights are read once: not kept in cache
        }
        __device__ __forceinline__ void step() { unit += kQ4KSuperBytes / 16; }
    } cur{base, r, lane};
    RmiRing<SuperRegs> ring;
    rmi_ring_fill(ring, n_units, cur);
    uint32_t *lds_dw = reinterpret_cast<uint32_t *>(lds);
    for (int t = 0; t < B; t++)
        rmi_stage_q8k_token<true, 2>(lds_dw + size_t(t) * n_sb * kSbDwords, p.q8qs + size_t(t) * n_in,
                                     p.q8bs + size_t(t) * (n_in / 16), p.q8d + size_t(t) * n_sb, n_sb, threadIdx.x,
                                     blockDim.x);
    __syncthreads();

    float acc[B], acc_m[B];
#pragma unroll
    for (int t = 0; t < B; t++) acc[t] = acc_m[t] = 0.0f;
    RmiRunResults<B> out{};
    uint32_t sb = 0;
    gptr_f32_w yp = as_global<gptr_f32_w>(p.y);
    auto consume = [&](const SuperRegs &g) {
        super_fma<B>(acc, acc_m, g, lds_dw, n_sb, sb, T);
        if (++sb == n_sb) {
            float y[B];
#pragma unroll
            for (int t = 0; t < B; t++) {
                const float main_val = hsum8_lanes(acc[t]);
                float m = acc_m[t];  // lanes T and T + 4 hold the same acc_m
                m = m + dpp_f32<kDppQuadXor2>(m);
                m = m + dpp_f32<kDppQuadXor1>(m);
                y[t] = main_val + m;  // the same in the row's eight lanes
                acc[t] = acc_m[t] = 0.0f;
            }
            sb = 0;
            out.keep(y, T);
            if (out.group_full()) out.flush(yp, p.y_stride, p.tile0 + k, r, T, p.row_start, p.row_end);
        }
    };
    rmi_ring_walk(ring, n_units, cur, consume);
    if (out.pending()) out.flush(yp, p.y_stride, p.tile0 + k, r, T, p.row_start, p.row_end);
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

// The same sum for 16 rows per workgroup with the work split by kind.  The sum of a row is one chain of f32 adds
// in element order, about eight clocks an add on one lane, and nothing may be reassociated; what feeds it (nibble
// extract, the two multiplies and the subtract of the dequantised weight, the product with the activation) has
// no order.  Two producer waves turn one super-block of the 16 rows into products in LDS (a lane takes one
// 16-byte piece: 32 elements) while a third wave, one lane per row, adds the previous super-block's products in
// order, reading 32 of them ahead of the chain; one barrier per super-block.  The activation is dequantised
// once into LDS.  Per super-block the chain needs 256 x 8.4 clocks and the producers about as long, against
// ten instructions per element on the chain's own lane in the kernel above (2048 x 6144: 340 -> about 30 us).
constexpr uint32_t kDdRows = 16, kDdProducers = kDdRows * 8, kDdThreads = kDdProducers + 64;
__global__ __launch_bounds__(kDdThreads) void q4_k_dequant_dot_split_kernel(
    const uint8_t *__restrict__ w, const float *__restrict__ x_f32, const int8_t *__restrict__ x_q8,
    const float *__restrict__ x_scales, float *__restrict__ y, uint32_t n_sb, uint32_t n_tiles, uint32_t row_start,
    uint32_t row_end, int mode) {
    extern __shared__ float4 dd_lds[];
    float4 *prod = dd_lds;                                             // [2][64 float4 per row][16 rows]
    float *xs = reinterpret_cast<float *>(dd_lds + 2 * 64 * kDdRows);  // [n_in]
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t row0 = (row_start / kDdRows + blockIdx.x) * kDdRows;  // first row of this workgroup
    const uint32_t n_in = n_sb * 256;
    for (uint32_t k = tid; k < n_in; k += kDdThreads)
        xs[k] = mode == 1 ? x_f32[k] : float(int(x_q8[k])) * x_scales[k >> 5];
    __syncthreads();

    // producer lane: row pr of the 16, piece T of its 128 nibble bytes
    const uint32_t pid = tid % kDdProducers, pr = pid % kDdRows, T = pid / kDdRows;
    const bool producer = tid < kDdProducers;
    uint32_t ptile = (row0 + pr) >> 3;
    if (ptile >= n_tiles) ptile = n_tiles - 1;  // rows past the padded stream: in bounds, never stored
    const uint8_t *ptile_base = w + size_t(ptile) * n_sb * kQ4KSuperBytes;
    auto produce = [&](uint32_t sb) {
        const uint8_t *chunk = ptile_base + size_t(sb) * kQ4KSuperBytes;
        const uint4 hdr = reinterpret_cast<const uint4 *>(chunk)[(row0 + pr) & 7];
        const uint4 qv = reinterpret_cast<const uint4 *>(chunk + 128)[((row0 + pr) & 7) * 8 + T];
        const float d = h2f(hdr.x & 0xffffu), dmin = h2f(hdr.x >> 16);
        const uint4 sm = unpack_scales(hdr.y, hdr.z, hdr.w);
        float4 *dst = prod + size_t(sb & 1) * 64 * kDdRows + pr;
        const float4 *xsb = reinterpret_cast<const float4 *>(xs + sb * 256);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint32_t dw = g == 0 ? qv.x : (g == 1 ? qv.y : (g == 2 ? qv.z : qv.w));
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const float dsc = d * float(byte_of(sm.x, sm.y, 2 * g + half));
                const float mm = dmin * float(byte_of(sm.z, sm.w, 2 * g + half));
                const uint32_t k4 = 16 * g + 8 * half + T;  // elements 4 k4 .. 4 k4 + 3 of the super-block
                const float4 xv = xsb[k4];
                const float xe[4] = {xv.x, xv.y, xv.z, xv.w};
                float pe[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t nib = (dw >> (8 * i + 4 * half)) & 0xfu;
                    const float wv = dsc * float(nib) - mm;
                    pe[i] = wv * xe[i];
                }
                dst[size_t(k4) * kDdRows] = make_float4(pe[0], pe[1], pe[2], pe[3]);
            }
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
int launch_gemv_q4k(const RmiQ4kProblem *single, const RmiQ4kProblem *d_list, const uint4 *d_runs, uint32_t n_waves,
                    uint32_t wpg, uint32_t tiles_per_wave, uint32_t max_n_sb, hipStream_t s) {
    const size_t lds_bytes = size_t(B) * max_n_sb * kSbDwords * 4;
    if (lds_bytes > 64 * 1024)
        return rmi_fail(RMI_HIP_E_INVALID, "activation of %d tokens x %u elements does not fit the LDS staging", B,
                        max_n_sb * 256);
    const dim3 grid_single((n_waves + wpg - 1) / wpg), grid_group(n_waves / wpg), block(64 * wpg);
    // the grouped run table is padded to whole workgroups
    if (single && wpg == 1)
        hipLaunchKernelGGL((gemv_q4_k_kernel<B, false, 64>), grid_single, block, lds_bytes, s, *single, d_list, d_runs,
                           tiles_per_wave);
    else if (single)
        hipLaunchKernelGGL((gemv_q4_k_kernel<B, false, 512>), grid_single, block, lds_bytes, s, *single, d_list, d_runs,
                           tiles_per_wave);
    else if (wpg == 1)
        hipLaunchKernelGGL((gemv_q4_k_kernel<B, true, 64>), grid_group, block, lds_bytes, s, RmiQ4kProblem{}, d_list, d_runs,
                           tiles_per_wave);
    else
        hipLaunchKernelGGL((gemv_q4_k_kernel<B, true, 512>), grid_group, block, lds_bytes, s, RmiQ4kProblem{}, d_list, d_runs,
                           tiles_per_wave);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int dispatch_q4k(uint32_t nt, const RmiQ4kProblem *single, const RmiQ4kProblem *d_list, const uint4 *d_runs,
                 uint32_t n_waves, uint32_t wpg, uint32_t tpw, uint32_t max_n_sb, hipStream_t s) {
    if (n_waves == 0) return RMI_HIP_OK;
    switch (nt) {
        case 1: return launch_gemv_q4k<1>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 2: return launch_gemv_q4k<2>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 3: return launch_gemv_q4k<3>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 4: return launch_gemv_q4k<4>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 5: return launch_gemv_q4k<5>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 6: return launch_gemv_q4k<6>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 7: return launch_gemv_q4k<7>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        case 8: return launch_gemv_q4k<8>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_sb, s);
        default: return rmi_fail(RMI_HIP_E_INVALID, "gemv takes 1..8 tokens per launch, got %u", nt);
    }
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

// Tiles a wave takes in one run: about 16 tile-super-blocks (18 KiB of weights), 32 with more than one token.
uint32_t rmi_q4k_tiles_per_wave(uint32_t n_sb, uint32_t launch_tiles, uint32_t n_tokens) {
    const uint32_t target = n_tokens > 1 ? 32 : 16;  // measured best for 1 and for 2..8 tokens
    uint32_t tpw = n_sb >= target ? 1 : target / (n_sb ? n_sb : 1);
    const uint32_t fill = uint32_t(rmi_device_cus()) * 8;
    while (tpw > 1 && launch_tiles / tpw < fill) tpw >>= 1;
    return tpw ? tpw : 1;
}

RmiQ4kProblem rmi_make_q4k_problem(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums,
                                   float *y, uint32_t y_stride, uint32_t row_start, uint32_t row_end) {
    RmiQ4kProblem p{};
    p.w = w->data;
    p.q8d = d;
    p.q8qs = qs;
    p.q8bs = bsums;
    p.y = y;
    p.n_sb = w->n_units;
    p.y_stride = y_stride;
    p.row_start = row_start;
    p.row_end = row_end;
    p.tile0 = row_start / kTileRows;
    p.n_tiles = row_end > row_start ? (row_end + kTileRows - 1) / kTileRows - p.tile0 : 0;
    return p;
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
        RmiQ4kProblem p = rmi_make_q4k_problem(w, d + size_t(t0) * n_sb, qs + size_t(t0) * w->n_in,
                                               bsums + size_t(t0) * (w->n_in / 16), y + size_t(t0) * y_stride, y_stride,
                                               row_start, row_end);
        const uint32_t tpw = rmi_q4k_tiles_per_wave(n_sb, p.n_tiles, nt);
        const uint32_t wpg =
            rmi_gemv_waves_per_group(size_t(nt) * n_sb * kSbDwords * 4, size_t(tpw) * n_sb * kQ4KSuperBytes);
        int rc = dispatch_q4k(nt, &p, nullptr, nullptr, (p.n_tiles + tpw - 1) / tpw, wpg, tpw, n_sb, s);
        if (rc != RMI_HIP_OK) return rc;
    }
    return RMI_HIP_OK;
}

int rmi_launch_gemv_q4_k_group(const RmiQ4kProblem *d_list, const uint4 *d_runs, uint32_t n_runs, uint32_t wpg,
                               uint32_t max_n_sb, uint32_t n_tokens, hipStream_t s) {
    return dispatch_q4k(n_tokens, nullptr, d_list, d_runs, n_runs, wpg, 0, max_n_sb, s);
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
    const size_t lds_bytes = size_t(2) * 64 * kDdRows * 16 + size_t(w->n_in) * 4;
    if (lds_bytes <= 160 * 1024 && w->n_units > 0) {
        static const bool raised = [] {  // more than 64 KiB of dynamic LDS has to be asked for once
            return hipFuncSetAttribute(reinterpret_cast<const void *>(q4_k_dequant_dot_split_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess;
        }();
        if (raised || lds_bytes <= 64 * 1024) {
            const uint32_t grid = (row_end - 1) / kDdRows - row_start / kDdRows + 1;
            hipLaunchKernelGGL(q4_k_dequant_dot_split_kernel, dim3(grid), dim3(kDdThreads), lds_bytes, s, w->data, x_f32,
                               x_q8, x_scales, y, w->n_units, w->n_tiles, row_start, row_end, mode);
            RMI_HIP_CHECK(hipGetLastError());
            return RMI_HIP_OK;
        }
    }
    const uint32_t grid = (row_end - row_start + 63) / 64;
    hipLaunchKernelGGL(q4_k_dequant_dot_kernel, dim3(grid), dim3(64), 0, s, w->data, x_f32, x_q8, x_scales, y,
                       w->n_units, row_start, row_end, mode);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
