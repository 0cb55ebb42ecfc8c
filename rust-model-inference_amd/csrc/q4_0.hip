// Q4_0 x Q8_0 decode GEMV (1..8 tokens), its exact per-block integer dots, and the upload-time repack.
//
// Arithmetic = matmul_q4_0_scalar_range (src/ops/kernel/q4_0/scalar.rs:13-52), which the reference's AVX2
// kernel reproduces bit for bit (q4_0/avx2.rs:24-105): one f32 accumulator per row, block after block,
//   sum = sum + (float(dot) * d) * scale,   dot = sum over the block of (nibble - 8) * q8   (int32, exact).
// The block dots of eight blocks run in parallel (eight lanes per row, one block each); the additions stay one
// chain per row: lane 0 of the row takes the products of lanes 0, 1, .. 7 in turn through lane shifts.
#include "rmi_internal.h"

#include "device_common.h"

#include "device_run_ring.h"

namespace {

// value of lane (l + K) of the same 16-lane row (only lanes 0 and 8 of a row use it, K <= 7)
template <int K>
__device__ __forceinline__ float lane_shl(float v) {
    if (K == 0) return v;
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x100 + K, 0xf, 0xf, false));
}

struct OctetRegs {
    uint32_t d;  // f16 scale of block 8o + L of the row
    u32x4 q;     // its 16 nibble bytes
};

// LDS per token: n_oct * 8 blocks x 32 int8 in source order, then per block {f32 scale, int32 8 * sum of its q8}
template <int B>
__device__ __forceinline__ void octet_fma(float (&acc)[B], const OctetRegs &g, const uint4 *lds, uint32_t tok_u4,
                                          uint32_t n_oct, uint32_t o, uint32_t L, uint32_t nb) {
    const float wd = h2f(g.d);
    const uint32_t k4 = 0x0f0f0f0fu;
    const uint32_t lo[4] = {g.q.x & k4, g.q.y & k4, g.q.z & k4, g.q.w & k4};
    const uint32_t hi[4] = {(g.q.x >> 4) & k4, (g.q.y >> 4) & k4, (g.q.z >> 4) & k4, (g.q.w >> 4) & k4};
    const uint32_t b = 8 * o + L;
    const bool live = b < nb;
#pragma unroll
    for (int t = 0; t < B; t++) {
        const uint4 *xt = lds + t * tok_u4;
        const uint4 xa = xt[2 * b], xb = xt[2 * b + 1];
        const uint2 meta = reinterpret_cast<const uint2 *>(xt + n_oct * 16)[b];
        int dot = __builtin_amdgcn_sdot4(int(lo[0]), int(xa.x), 0, false);
        dot = __builtin_amdgcn_sdot4(int(lo[1]), int(xa.y), dot, false);
        dot = __builtin_amdgcn_sdot4(int(lo[2]), int(xa.z), dot, false);
        dot = __builtin_amdgcn_sdot4(int(lo[3]), int(xa.w), dot, false);
        dot = __builtin_amdgcn_sdot4(int(hi[0]), int(xb.x), dot, false);
        dot = __builtin_amdgcn_sdot4(int(hi[1]), int(xb.y), dot, false);
        dot = __builtin_amdgcn_sdot4(int(hi[2]), int(xb.z), dot, false);
        dot = __builtin_amdgcn_sdot4(int(hi[3]), int(xb.w), dot, false);
        dot -= int(meta.y);  // sum (nibble - 8) * q8 = sum nibble * q8 - 8 * sum q8
        float p = B == 1 ? h2f_times<true>(g.d, float(dot)) : float(dot) * wd;
        p = p * __uint_as_float(meta.x);
        p = live ? p : -0.0f;  // a block past the end of the row adds nothing, not even a sign
        float a = acc[t];
        a = a + lane_shl<0>(p);
        a = a + lane_shl<1>(p);
        a = a + lane_shl<2>(p);
        a = a + lane_shl<3>(p);
        a = a + lane_shl<4>(p);
        a = a + lane_shl<5>(p);
        a = a + lane_shl<6>(p);
        a = a + lane_shl<7>(p);
        acc[t] = a;
    }
}

// Same launch shapes as the Q8_0 GEMV (gemv_q8_0.hip): a wave owns a run of consecutive 8-row tiles and walks
// it four octets deep (device_run_ring.h); up to eight waves of a workgroup share one staged activation.  GROUPED = false: one matrix (`single`), run w starts
// at tile w * tiles_per_wave.  GROUPED = true: runs[w] = {problem index, first tile, tile count, -}.
template <int B, bool GROUPED, int MAXT>
__global__ __launch_bounds__(MAXT) void gemv_q4_0_kernel(RmiGemvProblem single, const RmiGemvProblem *__restrict__ list,
                                                        const uint4 *__restrict__ runs, uint32_t tiles_per_wave) {
    extern __shared__ uint4 lds[];
    const uint32_t lane = threadIdx.x & 63, r = lane >> 3, L = lane & 7;
    // wave-uniform, and said so: the problem's fields and the octet counter live in scalar registers
    const uint32_t w_idx = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    RmiGemvProblem p;
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
    const uint32_t n_oct = p.n_oct, nb = p.n_in >> 5;
    const uint32_t tok_u4 = n_oct * 20;  // per token: 16 uint4 of quants + 4 of {scale, 8 * sum} per octet
    // units of the run (device_run_ring.h): one octet of one tile, 1152 bytes, tile after tile
    const uint32_t n_units = (k_end - k) * n_oct;
    struct Cursor {
        gptr_u4 unit;  // the same for all lanes
        uint32_t lane;
        __device__ __forceinline__ void load(OctetRegs &g) const {
            g.d = ((gptr_u16)unit)[lane];
            g.q = __builtin_nontemporal_load(unit + 8 + lane);  // weights are read once: do not keep them in cache
        }
        __device__ __forceinline__ void step() { unit += kQ40OctetBytes / 16; }
        // a wave without tiles (padding of the last workgroup) prefetches from the matrix's first tile: in bounds, unused
    } cur{as_global<gptr_u4>(p.w) + size_t(p.tile0 + (n_units ? k : 0)) * n_oct * (kQ40OctetBytes / 16), lane};
    RmiRing<OctetRegs> ring;
    rmi_ring_fill(ring, n_units, cur);
    for (int t = 0; t < B; t++) {  // a thread stages whole blocks: two 16-byte loads, the sum, the scale
        uint4 *dst = lds + t * tok_u4;
        gptr_u4 xq = as_global<gptr_u4>(p.x_q8 + size_t(t) * p.n_in);
        gptr_f32 xs = as_global<gptr_f32>(p.x_scales + size_t(t) * nb);
        for (uint32_t b = threadIdx.x; b < n_oct * 8; b += blockDim.x) {
            const uint32_t bc = b < nb ? b : nb - 1;
            u32x4 v0 = xq[2 * bc], v1 = xq[2 * bc + 1];
            float sc = xs[bc];
            if (b >= nb) {
                v0 = v1 = u32x4{0, 0, 0, 0};
                sc = 0.0f;
            }
            const int ones = 0x01010101;
            int sum = __builtin_amdgcn_sdot4(ones, int(v0.x), 0, false);
            sum = __builtin_amdgcn_sdot4(ones, int(v0.y), sum, false);
            sum = __builtin_amdgcn_sdot4(ones, int(v0.z), sum, false);
            sum = __builtin_amdgcn_sdot4(ones, int(v0.w), sum, false);
            sum = __builtin_amdgcn_sdot4(ones, int(v1.x), sum, false);
            sum = __builtin_amdgcn_sdot4(ones, int(v1.y), sum, false);
            sum = __builtin_amdgcn_sdot4(ones, int(v1.z), sum, false);
            sum = __builtin_amdgcn_sdot4(ones, int(v1.w), sum, false);
            dst[2 * b] = make_uint4(v0.x, v0.y, v0.z, v0.w);
            dst[2 * b + 1] = make_uint4(v1.x, v1.y, v1.z, v1.w);
            reinterpret_cast<uint2 *>(dst + n_oct * 16)[b] = make_uint2(__float_as_uint(sc), uint32_t(sum * 8));
        }
    }
    __syncthreads();

    float acc[B];
#pragma unroll
    for (int t = 0; t < B; t++) acc[t] = 0.0f;
    RmiRunResults<B> out{};
    uint32_t o = 0;
    gptr_f32_w yp = as_global<gptr_f32_w>(p.y);
    auto consume = [&](const OctetRegs &g) {
        octet_fma<B>(acc, g, lds, tok_u4, n_oct, o, L, nb);
        if (++o == n_oct) {
            float y[B];
#pragma unroll
            for (int t = 0; t < B; t++) {
                // the row's chain ends in its lane 0
                y[t] = __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, acc[t]), kSwizzleFirstOf8));
                acc[t] = 0.0f;
            }
            o = 0;
            out.keep(y, L);
            if (out.group_full()) out.flush(yp, p.y_stride, p.tile0 + k, r, L, p.row_start, p.row_end);
        }
    };
    rmi_ring_walk(ring, n_units, cur, consume);
    if (out.pending()) out.flush(yp, p.y_stride, p.tile0 + k, r, L, p.row_start, p.row_end);
}

// ---- per-block integer dots from the repacked stream
__global__ __launch_bounds__(256) void block_dots_q4_0_kernel(const uint8_t *__restrict__ w,
                                                               const int8_t *__restrict__ x_q8,
                                                               int32_t *__restrict__ dots, uint32_t n_out, uint32_t nb,
                                                               uint32_t n_oct) {
    const uint64_t total = uint64_t(n_out) * nb;
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < total;
         i += uint64_t(gridDim.x) * blockDim.x) {
        const uint32_t row = uint32_t(i / nb), b = uint32_t(i % nb);
        const uint8_t *chunk = w + (size_t(row >> 3) * n_oct + (b >> 3)) * kQ40OctetBytes;
        const uint8_t *q = chunk + 128 + ((row & 7) * 8 + (b & 7)) * 16;
        int dot = 0;
        for (int l = 0; l < 16; l++)
            dot += (int(q[l] & 0xF) - 8) * int(x_q8[32 * b + l]) + (int(q[l] >> 4) - 8) * int(x_q8[32 * b + 16 + l]);
        dots[i] = dot;
    }
}

// ---- upload-time repack: one workgroup per (tile, octet) of the destination, 576 16-bit units (the 18-byte
// source blocks are only 2-byte aligned); `src` holds the rows from tile `tile0` on
__global__ __launch_bounds__(256) void repack_q4_0_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                           uint32_t n_out, uint32_t nb, uint32_t n_oct, uint32_t tile0) {
    const uint32_t tile = tile0 + blockIdx.x / n_oct, o = blockIdx.x % n_oct;
    uint16_t *chunk = reinterpret_cast<uint16_t *>(dst + (size_t(tile) * n_oct + o) * kQ40OctetBytes);
    for (uint32_t idx = threadIdx.x; idx < 576; idx += 256) {
        uint32_t r, blk, half;  // destination unit idx <- unit `half` of block `blk` of row r
        if (idx < 64) {         // scales
            r = idx >> 3;
            blk = o * 8 + (idx & 7);
            half = 0;
        } else {  // quants: (r, L) x 8 units
            const uint32_t k = idx - 64;
            r = k >> 6;
            blk = o * 8 + ((k >> 3) & 7);
            half = 1 + (k & 7);
        }
        const uint32_t row = tile * kTileRows + r;
        uint16_t v = 0;
        if (row < n_out && blk < nb)
            v = reinterpret_cast<const uint16_t *>(src + (size_t(row - tile0 * kTileRows) * nb + blk) * 18)[half];
        chunk[idx] = v;
    }
}

template <int B>
int launch_q4_0(const RmiGemvProblem *single, const RmiGemvProblem *d_list, const uint4 *d_runs, uint32_t n_waves,
                uint32_t wpg, uint32_t tpw, uint32_t max_n_oct, hipStream_t s) {
    const size_t lds_bytes = size_t(B) * max_n_oct * 320;
    if (lds_bytes > 64 * 1024)
        return rmi_fail(RMI_HIP_E_INVALID, "activation of %d tokens x %u elements does not fit the LDS staging", B,
                        max_n_oct * 256);
    if (n_waves == 0) return RMI_HIP_OK;
    const dim3 grid((n_waves + wpg - 1) / wpg), block(64 * wpg);
    if (single && wpg == 1)
        hipLaunchKernelGGL((gemv_q4_0_kernel<B, false, 64>), grid, block, lds_bytes, s, *single, nullptr, nullptr, tpw);
    else if (single)
        hipLaunchKernelGGL((gemv_q4_0_kernel<B, false, 512>), grid, block, lds_bytes, s, *single, nullptr, nullptr, tpw);
    else if (wpg == 1)
        hipLaunchKernelGGL((gemv_q4_0_kernel<B, true, 64>), grid, block, lds_bytes, s, RmiGemvProblem{}, d_list, d_runs, tpw);
    else
        hipLaunchKernelGGL((gemv_q4_0_kernel<B, true, 512>), grid, block, lds_bytes, s, RmiGemvProblem{}, d_list, d_runs,
                           tpw);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int dispatch_q4_0(uint32_t n_tokens, const RmiGemvProblem *single, const RmiGemvProblem *d_list, const uint4 *d_runs,
                  uint32_t n_waves, uint32_t wpg, uint32_t tpw, uint32_t max_n_oct, hipStream_t s) {
    switch (n_tokens) {
        case 1: return launch_q4_0<1>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_oct, s);
        case 2: return launch_q4_0<2>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_oct, s);
        case 3: return launch_q4_0<3>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_oct, s);
        case 4: return launch_q4_0<4>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_oct, s);
        case 5: return launch_q4_0<5>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_oct, s);
        case 6: return launch_q4_0<6>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_oct, s);
        case 7: return launch_q4_0<7>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_oct, s);
        case 8: return launch_q4_0<8>(single, d_list, d_runs, n_waves, wpg, tpw, max_n_oct, s);
        default: return rmi_fail(RMI_HIP_E_INVALID, "gemv takes 1..8 tokens per launch, got %u", n_tokens);
    }
}

}  // namespace

int rmi_launch_gemv_q4_0(const RmiGemvProblem &p, uint32_t n_tokens, hipStream_t s) {
    if (p.n_tiles == 0 || p.n_oct == 0) return RMI_HIP_OK;
    const uint32_t tpw = rmi_gemv_tiles_per_wave(p.n_oct, p.n_tiles, n_tokens);
    const uint32_t wpg = rmi_gemv_waves_per_group(size_t(n_tokens) * p.n_oct * 320, size_t(tpw) * p.n_oct * kQ40OctetBytes);
    return dispatch_q4_0(n_tokens, &p, nullptr, nullptr, (p.n_tiles + tpw - 1) / tpw, wpg, tpw, p.n_oct, s);
}

int rmi_launch_gemv_q4_0_group(const RmiGemvProblem *d_list, const uint4 *d_runs, uint32_t n_runs, uint32_t wpg,
                               uint32_t max_n_oct, uint32_t n_tokens, hipStream_t s) {
    return dispatch_q4_0(n_tokens, nullptr, d_list, d_runs, n_runs, wpg, 0, max_n_oct, s);
}

int rmi_launch_block_dots_q4_0(const rmi_hip_weight *w, const int8_t *x_q8, int32_t *dots, hipStream_t s) {
    const uint64_t total = uint64_t(w->n_out) * (w->n_in / 32);
    if (total == 0) return RMI_HIP_OK;
    const uint32_t grid = uint32_t(total / 256 + 1 < 65535 ? total / 256 + 1 : 65535);
    hipLaunchKernelGGL(block_dots_q4_0_kernel, dim3(grid), dim3(256), 0, s, w->data, x_q8, dots, w->n_out, w->n_in / 32,
                       w->n_units);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_launch_repack_q4_0(const uint8_t *src, rmi_hip_weight *w, uint32_t tile0, uint32_t n_tiles, hipStream_t s) {
    const uint32_t grid = n_tiles * w->n_units;
    if (grid == 0) return RMI_HIP_OK;
    hipLaunchKernelGGL(repack_q4_0_kernel, dim3(grid), dim3(256), 0, s, src, w->data, w->n_out, w->n_in / 32, w->n_units,
                       tile0);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
