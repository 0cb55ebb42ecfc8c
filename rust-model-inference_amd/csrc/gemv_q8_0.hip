// Q8_0 x Q8_0 decode GEMV (1..8 tokens) over the HBM tile stream, the per-block
// integer dots, the device activation quantizer and the f32-activation GEMV.
//
// Arithmetic order of the GEMV = matmul_q8_0_vs_q8_0_avx2
// (src/ops/kernel/q8_0/avx2.rs:71-173): eight f32 accumulators per row, lane L
// taking fma(f32(wd)*xs[b], float(sum_{k=4L..4L+3} w*x), acc_L) block after
// block, then hsum_ps (src/ops/dot.rs:447-456).  Eight GPU lanes hold the eight
// accumulators of one row, so results match that kernel bit for bit.
#include "device_math.h"
#include "device_quant.h"
#include "rmi_internal.h"

#include "device_common.h"

#include "device_run_ring.h"

namespace {

// s = f32(wd) * xs with one rounding, as _mm_mul_ps(cvtph, set1(bd)), then the block's fma.  At one token the
// product reads the f16 scale in place (h2f_times<true>: a seventh of the kernel's instructions; decode 1187 ->
// 1203 token-steps/s); with more tokens the conversion is shared and the plain multiply is the cheaper instruction.
template <bool MIX>
__device__ __forceinline__ void block_fma(float &acc, uint32_t w_bits, float xs, int wq, int xq) {
    const float s = h2f_times<MIX>(w_bits, xs);
    const int p = dot4_i8(wq, xq);
    acc = __builtin_fmaf(s, float(p), acc);
}

// The three 16-byte loads one lane issues for one octet of its row.
struct OctetRegs {
    u32x4 sc;  // 8 f16 block scales of the row (same for the 8 lanes of the row)
    u32x4 qa;  // blocks 8o..8o+3, bytes 4L..4L+3 of each
    u32x4 qb;  // blocks 8o+4..8o+7
};

__device__ __forceinline__ void load_octet(OctetRegs &g, gptr_u4 sc_ptr, gptr_u4 q_ptr, uint32_t o) {
    g.sc = sc_ptr[o * 8];
    g.qa = __builtin_nontemporal_load(q_ptr + (2 * o) * 64);  // weights are read once: do not keep them in cache
    g.qb = __builtin_nontemporal_load(q_ptr + (2 * o + 1) * 64);
}

// Stages one token's activation in LDS: the int8 quants of n_oct octets, moved from source order to quad
// order (dword l of block b -> [b/4][l][b%4]), then the f32 block scales; zeros beyond the nb source blocks.
// The loads are 16 bytes wide, unconditional (clamped) and issued UNROLL at a time before the first LDS
// write waits for them: a guarded load per dword costs one memory round trip per loop iteration.
template <int UNROLL>
__device__ __forceinline__ void stage_token(uint32_t *dq, const int8_t *x_q8, const float *x_scales, uint32_t n_oct,
                                            uint32_t nb, uint32_t tid, uint32_t n_threads) {
    gptr_u4 xq = as_global<gptr_u4>(x_q8);
    gptr_f32 xs = as_global<gptr_f32>(x_scales);
    const uint32_t n_u4 = n_oct * 16, src_u4 = nb * 2;
    // the first two scales of this thread travel with the quants
    const uint32_t s0 = tid, s1 = tid + n_threads;
    const float sv0 = xs[s0 < nb ? s0 : nb - 1], sv1 = xs[s1 < nb ? s1 : nb - 1];
    for (uint32_t base = tid; base < n_u4; base += n_threads * UNROLL) {
        u32x4 v[UNROLL];
#pragma unroll
        for (int j = 0; j < UNROLL; j++) {
            const uint32_t i = base + j * n_threads;
            v[j] = xq[i < src_u4 ? i : src_u4 - 1];
        }
#pragma unroll
        for (int j = 0; j < UNROLL; j++) {
            const uint32_t i = base + j * n_threads;
            if (i < n_u4) {
                const uint32_t b = i >> 1;  // block; this uint4 holds its dwords l = 4*(i&1) .. +3
                uint32_t *d = dq + (b >> 2) * 32 + (i & 1) * 16 + (b & 3);
                const bool live = i < src_u4;
                d[0] = live ? v[j].x : 0u;
                d[4] = live ? v[j].y : 0u;
                d[8] = live ? v[j].z : 0u;
                d[12] = live ? v[j].w : 0u;
            }
        }
    }
    float *ds = reinterpret_cast<float *>(dq + n_oct * 64);
    if (s0 < n_oct * 8) ds[s0] = s0 < nb ? sv0 : 0.0f;
    if (s1 < n_oct * 8) ds[s1] = s1 < nb ? sv1 : 0.0f;
    for (uint32_t i = tid + 2 * n_threads; i < n_oct * 8; i += n_threads) {
        const float sv = xs[i < nb ? i : nb - 1];
        ds[i] = i < nb ? sv : 0.0f;
    }
}

// The same for n_tokens tokens at once, tok_dw dwords apart in LDS: the pieces of all tokens are one index space, so
// that a workgroup of eight waves has every load of a small batch in flight before the first LDS write waits (token
// after token, each token is a memory round trip of its own).
template <int UNROLL>
__device__ __forceinline__ void stage_tokens(uint32_t *dq, uint32_t tok_dw, const int8_t *x_q8, const float *x_scales,
                                             uint32_t n_tokens, uint32_t n_oct, uint32_t nb, uint32_t tid, uint32_t n_threads) {
    gptr_u4 xq = as_global<gptr_u4>(x_q8);
    gptr_f32 xs = as_global<gptr_f32>(x_scales);
    const uint32_t n_u4 = n_oct * 16, src_u4 = nb * 2, total = n_tokens * n_u4;
    for (uint32_t base = tid; base < total; base += n_threads * UNROLL) {
        u32x4 v[UNROLL];
        uint32_t tok[UNROLL], idx[UNROLL];
#pragma unroll
        for (int j = 0; j < UNROLL; j++) {
            const uint32_t e = base + j * n_threads < total ? base + j * n_threads : total - 1;
            tok[j] = e / n_u4;
            idx[j] = e - tok[j] * n_u4;
            v[j] = xq[size_t(tok[j]) * src_u4 + (idx[j] < src_u4 ? idx[j] : src_u4 - 1)];
        }
#pragma unroll
        for (int j = 0; j < UNROLL; j++) {
            if (base + j * n_threads < total) {
                const uint32_t i = idx[j], b = i >> 1;
                uint32_t *d = dq + tok[j] * tok_dw + (b >> 2) * 32 + (i & 1) * 16 + (b & 3);
                const bool live = i < src_u4;
                d[0] = live ? v[j].x : 0u;
                d[4] = live ? v[j].y : 0u;
                d[8] = live ? v[j].z : 0u;
                d[12] = live ? v[j].w : 0u;
            }
        }
    }
    const uint32_t n_sc = n_oct * 8;
    for (uint32_t e = tid; e < n_tokens * n_sc; e += n_threads) {
        const uint32_t t = e / n_sc, i = e - t * n_sc;
        const float sv = xs[size_t(t) * nb + (i < nb ? i : nb - 1)];
        reinterpret_cast<float *>(dq + t * tok_dw + n_oct * 64)[i] = i < nb ? sv : 0.0f;
    }
}

// acc = fma(s of lane K of this lane's quad, p, acc): v_fmac_f32 takes its first factor through DPP, so the
// broadcast costs no instruction of its own.  (The compiler does not fold a DPP move into the VOP3 fma it selects.)
template <int K>
__device__ __forceinline__ void fmac_quad(float &acc, float s, float p);
template <>
__device__ __forceinline__ void fmac_quad<0>(float &acc, float s, float p) {
    asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(s), "v"(p));
}
template <>
__device__ __forceinline__ void fmac_quad<1>(float &acc, float s, float p) {
    asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(s), "v"(p));
}
template <>
__device__ __forceinline__ void fmac_quad<2>(float &acc, float s, float p) {
    asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(s), "v"(p));
}
template <>
__device__ __forceinline__ void fmac_quad<3>(float &acc, float s, float p) {
    asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(s), "v"(p));
}
__device__ __forceinline__ void fmac_quad_k(float &acc, float s, float p, int k) {  // k is a constant once unrolled
    if (k == 0) fmac_quad<0>(acc, s, p);
    else if (k == 1) fmac_quad<1>(acc, s, p);
    else if (k == 2) fmac_quad<2>(acc, s, p);
    else fmac_quad<3>(acc, s, p);
}

template <int B>
__device__ __forceinline__ void octet_fma(float (&acc)[B], const OctetRegs &g, const uint4 *lds, uint32_t tok_u4,
                                          uint32_t n_oct, uint32_t o, uint32_t L) {
    if constexpr (B >= 2) {
        // The scale product of (row, block, token) is the same in the row's eight lanes: each lane of a quad
        // multiplies it for token (lane & 3) and token (lane & 3) + 4 only, and the fma takes it from there.
        const uint32_t q = L & 3;
        const uint4 *x0 = lds + (q < B ? q : 0) * tok_u4, *x1 = lds + (q + 4 < B ? q + 4 : 0) * tok_u4;
        const float4 a0 = reinterpret_cast<const float4 *>(x0 + n_oct * 16)[2 * o];
        const float4 a1 = reinterpret_cast<const float4 *>(x0 + n_oct * 16)[2 * o + 1];
        const float xs0[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        float xs1[8];
        if constexpr (B > 4) {
            const float4 b0 = reinterpret_cast<const float4 *>(x1 + n_oct * 16)[2 * o];
            const float4 b1 = reinterpret_cast<const float4 *>(x1 + n_oct * 16)[2 * o + 1];
            xs1[0] = b0.x, xs1[1] = b0.y, xs1[2] = b0.z, xs1[3] = b0.w, xs1[4] = b1.x, xs1[5] = b1.y, xs1[6] = b1.z, xs1[7] = b1.w;
        }
        const uint32_t scw[4] = {g.sc.x, g.sc.y, g.sc.z, g.sc.w};
        float s0[8], s1[8];
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const float wd = h2f((b & 1) ? scw[b >> 1] >> 16 : scw[b >> 1] & 0xffffu);
            s0[b] = wd * xs0[b];
            if constexpr (B > 4) s1[b] = wd * xs1[b];
        }
        // a DPP read of a register needs two wait states after the vector instruction that wrote it, and the
        // compiler does not look into the asm statements below: all products pass this point first
        if constexpr (B > 4)
            asm volatile("s_nop 1" : "+v"(s0[0]), "+v"(s0[1]), "+v"(s0[2]), "+v"(s0[3]), "+v"(s0[4]), "+v"(s0[5]), "+v"(s0[6]), "+v"(s0[7]),
                                     "+v"(s1[0]), "+v"(s1[1]), "+v"(s1[2]), "+v"(s1[3]), "+v"(s1[4]), "+v"(s1[5]), "+v"(s1[6]), "+v"(s1[7]));
        else
            asm volatile("s_nop 1" : "+v"(s0[0]), "+v"(s0[1]), "+v"(s0[2]), "+v"(s0[3]), "+v"(s0[4]), "+v"(s0[5]), "+v"(s0[6]), "+v"(s0[7]));
        const int wq[8] = {int(g.qa.x), int(g.qa.y), int(g.qa.z), int(g.qa.w), int(g.qb.x), int(g.qb.y), int(g.qb.z), int(g.qb.w)};
#pragma unroll
        for (int t = 0; t < B; t++) {
            const uint4 *xt = lds + t * tok_u4;
            const uint4 xa = xt[(2 * o) * 8 + L];
            const uint4 xb = xt[(2 * o + 1) * 8 + L];
            const int xq[8] = {int(xa.x), int(xa.y), int(xa.z), int(xa.w), int(xb.x), int(xb.y), int(xb.z), int(xb.w)};
            float a = acc[t];
#pragma unroll
            for (int b = 0; b < 8; b++) {
                fmac_quad_k(a, t < 4 ? s0[b] : s1[b], float(dot4_i8(wq[b], xq[b])), t & 3);
            }
            acc[t] = a;
        }
        return;
    }
#pragma unroll
    for (int t = 0; t < B; t++) {
        const uint4 *xt = lds + t * tok_u4;
        const uint4 xa = xt[(2 * o) * 8 + L];
        const uint4 xb = xt[(2 * o + 1) * 8 + L];
        const float4 s0 = reinterpret_cast<const float4 *>(xt + n_oct * 16)[2 * o];
        const float4 s1 = reinterpret_cast<const float4 *>(xt + n_oct * 16)[2 * o + 1];
        float a = acc[t];
        block_fma<B == 1>(a, g.sc.x & 0xffffu, s0.x, int(g.qa.x), int(xa.x));
        block_fma<B == 1>(a, g.sc.x >> 16, s0.y, int(g.qa.y), int(xa.y));
        block_fma<B == 1>(a, g.sc.y & 0xffffu, s0.z, int(g.qa.z), int(xa.z));
        block_fma<B == 1>(a, g.sc.y >> 16, s0.w, int(g.qa.w), int(xa.w));
        block_fma<B == 1>(a, g.sc.z & 0xffffu, s1.x, int(g.qb.x), int(xb.x));
        block_fma<B == 1>(a, g.sc.z >> 16, s1.y, int(g.qb.y), int(xb.y));
        block_fma<B == 1>(a, g.sc.w & 0xffffu, s1.z, int(g.qb.z), int(xb.z));
        block_fma<B == 1>(a, g.sc.w >> 16, s1.w, int(g.qb.w), int(xb.w));
        acc[t] = a;
    }
}

// One token's staged operands of an octet, as a lane reads them from LDS.
struct OctetX {
    uint4 xa, xb;   // bytes 4L..4L+3 of blocks 8o..8o+3 and 8o+4..8o+7
    float4 s0, s1;  // the eight block scales
};
__device__ __forceinline__ OctetX load_octet_x(const uint4 *lds, uint32_t n_oct, uint32_t o, uint32_t L) {
    OctetX x;
    x.xa = lds[(2 * o) * 8 + L];
    x.xb = lds[(2 * o + 1) * 8 + L];
    x.s0 = reinterpret_cast<const float4 *>(lds + n_oct * 16)[2 * o];
    x.s1 = reinterpret_cast<const float4 *>(lds + n_oct * 16)[2 * o + 1];
    return x;
}
// The NOCT octets of a tile whose weights are in registers already, one token: the LDS reads of octet o + 1 go out
// before octet o is multiplied.  A wave that has its compute unit to itself otherwise waits out an LDS round trip
// per octet (the reads of an octet and the wait for the first of them stood back to back).  Same arithmetic and
// order as octet_fma<1>.
template <int NOCT>
__device__ __forceinline__ void octets_fma_ahead(float &acc, const OctetRegs (&g)[NOCT], const uint4 *lds, uint32_t L,
                                                 uint32_t n_staged = NOCT) {  // octets staged in LDS (NOCT or more)
    OctetX x = load_octet_x(lds, n_staged, 0, L);
    float a = acc;
#pragma unroll
    for (int o = 0; o < NOCT; o++) {
        OctetX nx = x;
        if (o + 1 < NOCT) nx = load_octet_x(lds, n_staged, o + 1, L);
        // The sum passes a point that no memory access moves across: the reads of octet o + 1 stay in front of
        // the multiply-adds of octet o.  (Left to itself the compiler moves them back down to their uses.)
        asm volatile("" : "+v"(a) : : "memory");
        const OctetRegs &w = g[o];
        block_fma<true>(a, w.sc.x & 0xffffu, x.s0.x, int(w.qa.x), int(x.xa.x));
        block_fma<true>(a, w.sc.x >> 16, x.s0.y, int(w.qa.y), int(x.xa.y));
        block_fma<true>(a, w.sc.y & 0xffffu, x.s0.z, int(w.qa.z), int(x.xa.z));
        block_fma<true>(a, w.sc.y >> 16, x.s0.w, int(w.qa.w), int(x.xa.w));
        block_fma<true>(a, w.sc.z & 0xffffu, x.s1.x, int(w.qb.x), int(x.xb.x));
        block_fma<true>(a, w.sc.z >> 16, x.s1.y, int(w.qb.y), int(x.xb.y));
        block_fma<true>(a, w.sc.w & 0xffffu, x.s1.z, int(w.qb.z), int(x.xb.z));
        block_fma<true>(a, w.sc.w >> 16, x.s1.w, int(w.qb.w), int(x.xb.w));
        x = nx;
    }
    acc = a;
}

// A wave's N octets (the staged octets first .. first + N - 1) multiplied down to the two factors of every block's
// fma, for another wave to add: dst[(4 i + q) * 64] = {s, float(dot), s', float(dot')} of blocks 2q and 2q + 1 of its
// octet i (dst already points at this lane's float4).
template <int N>
__device__ __forceinline__ void octets_to_factors(const OctetRegs (&g)[N], const uint4 *lds, uint32_t n_staged,
                                                  uint32_t first, uint32_t L, float4 *dst) {
    OctetX x = load_octet_x(lds, n_staged, first, L);
#pragma unroll
    for (int i = 0; i < N; i++) {
        OctetX nx = x;
        if (i + 1 < N) nx = load_octet_x(lds, n_staged, first + i + 1, L);
        const OctetRegs &w = g[i];
        float4 *d = dst + i * 4 * 64;
        d[0] = make_float4(h2f_times<true>(w.sc.x & 0xffffu, x.s0.x), float(dot4_i8(int(w.qa.x), int(x.xa.x))),
                           h2f_times<true>(w.sc.x >> 16, x.s0.y), float(dot4_i8(int(w.qa.y), int(x.xa.y))));
        d[64] = make_float4(h2f_times<true>(w.sc.y & 0xffffu, x.s0.z), float(dot4_i8(int(w.qa.z), int(x.xa.z))),
                            h2f_times<true>(w.sc.y >> 16, x.s0.w), float(dot4_i8(int(w.qa.w), int(x.xa.w))));
        d[128] = make_float4(h2f_times<true>(w.sc.z & 0xffffu, x.s1.x), float(dot4_i8(int(w.qb.x), int(x.xb.x))),
                             h2f_times<true>(w.sc.z >> 16, x.s1.y), float(dot4_i8(int(w.qb.y), int(x.xb.y))));
        d[192] = make_float4(h2f_times<true>(w.sc.w & 0xffffu, x.s1.z), float(dot4_i8(int(w.qb.z), int(x.xb.z))),
                             h2f_times<true>(w.sc.w >> 16, x.s1.w), float(dot4_i8(int(w.qb.w), int(x.xb.w))));
        x = nx;
    }
}
// ... and the M octets' factors added to a lane's sum in block order (src points at this lane's float4 of the first)
template <int M>
__device__ __forceinline__ void factors_sum(float &acc, const float4 *src) {
    float4 f[4];
#pragma unroll
    for (int q = 0; q < 4; q++) f[q] = src[q * 64];
#pragma unroll
    for (int o = 0; o < M; o++) {
        float4 nf[4];
#pragma unroll
        for (int q = 0; q < 4; q++) nf[q] = o + 1 < M ? src[((o + 1) * 4 + q) * 64] : f[q];
        asm volatile("" : "+v"(acc) : : "memory");  // the next octet's reads stay in front of this octet's sums
#pragma unroll
        for (int q = 0; q < 4; q++) {
            acc = __builtin_fmaf(f[q].x, f[q].y, acc);
            acc = __builtin_fmaf(f[q].z, f[q].w, acc);
        }
#pragma unroll
        for (int q = 0; q < 4; q++) f[q] = nf[q];
    }
}

// A wave owns a short run of consecutive 8-row tiles of ONE matrix (about 34 KiB of
// weights) and walks it four octets deep (device_run_ring.h).  A launch has far more
// waves than fit on the chip at once: the dispatcher hands out runs as waves retire,
// which balances the load and keeps the waves in flight reading one compact window of
// HBM.  The activation of the matrix sits in LDS, permuted to quad order.
// GROUPED = false: one matrix (`single`), run w starts at tile w * tiles_per_wave.
// GROUPED = true: runs[w] = {problem index, first tile, tile count, -}.
// MAXT = 64: one wave per workgroup; 512: up to eight waves sharing one staged activation
template <int B, bool GROUPED, int MAXT>
__global__ __launch_bounds__(MAXT) void gemv_q8_0_kernel(RmiGemvProblem single,
                                                        const RmiGemvProblem *__restrict__ list,
                                                        const uint4 *__restrict__ runs, uint32_t tiles_per_wave) {
    extern __shared__ uint4 lds[];
    const uint32_t lane = threadIdx.x & 63, r = lane >> 3, L = lane & 7;
    // run of this wave; the waves of a workgroup always work on the same matrix and share its activation.
    // The index is the same for all lanes, and said so: the problem's fields, the octet counter and the
    // addresses of the walk then live in scalar registers.
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
        // a launch may spread its tokens over workgroups (gridDim.y groups of B tokens each): the group's B tokens
        p.x_q8 += size_t(blockIdx.y) * B * p.n_in;
        p.x_scales += size_t(blockIdx.y) * B * (p.n_in >> 5);
        p.y += size_t(blockIdx.y) * B * p.y_stride;
        k = w_idx * tiles_per_wave < p.n_tiles ? w_idx * tiles_per_wave : p.n_tiles;
        k_end = k + tiles_per_wave < p.n_tiles ? k + tiles_per_wave : p.n_tiles;
    }

    const uint32_t n_oct = p.n_oct;
    const uint32_t tok_u4 = n_oct * 18;  // per token: 16 uint4 of quants + 2 of scales per octet
    // Units of the run (device_run_ring.h): one octet of one tile.  A tile holds its n_oct scale pieces (128
    // bytes each) before its n_oct quant pieces (2048 bytes each), so the two addresses of a unit move apart
    // within a tile and jump at its end.  The first four units' loads go out before the activation is staged.
    const uint32_t n_units = (k_end - k) * n_oct;
    struct Cursor {
        gptr_u4 sc_unit, q_unit;  // the same for all lanes
        uint32_t o, n_oct, r, lane;
        __device__ __forceinline__ void load(OctetRegs &g) const {
            g.sc = sc_unit[r];
            g.qa = __builtin_nontemporal_load(q_unit + lane);  // weights are read once: do not keep them in cache
            g.qb = __builtin_nontemporal_load(q_unit + 64 + lane);
        }
        __device__ __forceinline__ void step() {
            sc_unit += 8;
            q_unit += 128;
            if (++o == n_oct) {  // over this tile's quants / the next tile's scales
                o = 0;
                sc_unit += size_t(n_oct) * 128;
                q_unit += size_t(n_oct) * 8;
            }
        }
    } cur;
    {
        // a wave without tiles (padding of the last workgroup) prefetches from the matrix's first tile: in bounds, unused
        gptr_u4 tile = as_global<gptr_u4>(p.w + size_t(p.tile0 + (n_units ? k : 0)) * n_oct * kOctetBytes);
        cur = Cursor{tile, tile + n_oct * 8, 0, n_oct, r, lane};
    }
    RmiRing<OctetRegs> ring;
    rmi_ring_fill(ring, n_units, cur);
    {
        const uint32_t nb = p.n_in >> 5;
        uint32_t *lds_dw = reinterpret_cast<uint32_t *>(lds);
        if constexpr (B == 1)
            stage_token<4>(lds_dw, p.x_q8, p.x_scales, n_oct, nb, threadIdx.x, blockDim.x);
        else
            stage_tokens<4>(lds_dw, tok_u4 * 4, p.x_q8, p.x_scales, B, n_oct, nb, threadIdx.x, blockDim.x);
        __syncthreads();
    }

    float acc[B];
#pragma unroll
    for (int t = 0; t < B; t++) acc[t] = 0.0f;
    RmiRunResults<B> out{};
    uint32_t o = 0;
    gptr_f32_w yp = as_global<gptr_f32_w>(p.y);
    auto consume = [&](const OctetRegs &g) {
        octet_fma<B>(acc, g, lds, tok_u4, n_oct, o, L);
        if (++o == n_oct) {
            float y[B];
#pragma unroll
            for (int t = 0; t < B; t++) {
                y[t] = hsum8_lanes(acc[t]);  // the same in the row's eight lanes
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

// ---- The same GEMV for four to eight tokens with the 4-byte dots on the matrix cores.
// The x86-64 order needs, per row, block, 4-byte slice and token, one dot of four byte pairs, its conversion and one
// fma; at eight tokens those three vector instructions are what the kernel above is bound by.  v_mfma_i32_4x4x4_16B_i8
// is sixteen independent 4 x 4 x 4 products: in block beta (lanes 4 beta .. 4 beta + 3) the result register v of lane
// 4 beta + j is the dot of the four bytes in the A register of lane 4 beta + v with the four bytes in the B register of
// lane 4 beta + j.  With four weight ROWS' slice s in the A registers of a block and four TOKENS' slice s in its B
// registers, one instruction delivers what 4 x 4 v_dot4 did, on the other pipe.  Lane layout (j = lane & 3,
// sl = lane >> 2 & 3, s_hi = lane >> 4 & 1, rg = lane >> 5): the lane works on slice s = 4 s_hi + sl of rows
// 4 rg .. 4 rg + 3 for tokens j and j + 4; its A register holds row 4 rg + ((j + sl) & 3), so that its result register
// v is row 4 rg + ((v + sl) & 3).  That rotation is what lets the scale products be shared without a lane-dependent
// register index: lane (sl, j) multiplies f32(wd) * xs for row 4 rg + sl and its two tokens only, and the fma on result
// register v takes the product of ITS row from the lane 4 v further on in the row of sixteen (row_ror: the lane with
// sl' = sl + v, same j), through DPP.  The weight pieces arrive in the stream's order (lane 8 r + L: slice L of row r,
// one full-line load per quad) and cross lanes once through the LDS crossbar (ds_bpermute, no LDS memory).  Every
// accumulator is one (row, slice, token) chain with the blocks in sequence and the eight slices meet in hsum_ps
// order: the same bits as the kernel above.  Finished tiles park their 64 results in LDS and leave eight tiles at a
// time, 256 bytes a token.
// 16-byte pieces per staged token: the 18 per octet of the kernel above, padded so that tokens lie 64 bytes (mod 256)
// apart.  Sixteen lanes read four tokens' 64 bytes of one quad at once; with the plain stride (a multiple of 128
// bytes for an even number of octets) two or all four of them fall on the same banks.
__host__ __device__ inline uint32_t rmi_gemv_x4_token_u4(uint32_t n_oct) {
    const uint32_t plain = n_oct * 18;
    return plain + ((4 + 16 - (plain & 15)) & 15);
}
// floats of LDS per wave behind the staged tokens: four tiles' results and the 8 x 33 partial sums of a tile's end
__host__ __device__ constexpr uint32_t kX4WaveFloats(uint32_t n_tokens) { return 4 * n_tokens * 8 + 8 * 33 + 8; }
// waves that are to share a SIMD (the register budget): five fit only with spills, and measured no faster
constexpr int kX4WavesPerSimd = 4;
template <int N>
__device__ __forceinline__ void fmac_ror4(float &acc, float s, float p);  // acc += (s of the lane 4 N on in the row) * p
template <>
__device__ __forceinline__ void fmac_ror4<0>(float &acc, float s, float p) {
    acc = __builtin_fmaf(s, p, acc);
}
template <>
__device__ __forceinline__ void fmac_ror4<1>(float &acc, float s, float p) {
    asm("v_fmac_f32_dpp %0, %1, %2 row_ror:12 row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(s), "v"(p));
}
template <>
__device__ __forceinline__ void fmac_ror4<2>(float &acc, float s, float p) {
    asm("v_fmac_f32_dpp %0, %1, %2 row_ror:8 row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(s), "v"(p));
}
template <>
__device__ __forceinline__ void fmac_ror4<3>(float &acc, float s, float p) {
    asm("v_fmac_f32_dpp %0, %1, %2 row_ror:4 row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(s), "v"(p));
}
typedef int v4i_x4 __attribute__((ext_vector_type(4)));

template <int B>
__device__ __forceinline__ void octet_fma_x4(float (&acc)[2][4], const OctetRegs &g, const uint4 *lds, uint32_t tok_u4,
                                             uint32_t n_oct, uint32_t o, uint32_t s, uint32_t j, uint32_t src_addr) {
    constexpr int TG = B > 4 ? 2 : 1;
    // the lane's tokens; one past the batch takes token 0's data, and its results are not stored
    const uint4 *xt[2] = {lds + (j < B ? j : 0) * tok_u4, lds + (j + 4 < B ? j + 4 : 0) * tok_u4};
    const uint32_t scw[4] = {g.sc.x, g.sc.y, g.sc.z, g.sc.w};  // the eight block scales of row 4 rg + sl
    const v4i_x4 zero4 = {0, 0, 0, 0};
    // a quad of blocks at a time: what is live at once (the weight pieces, the tokens' pieces, the scale products)
    // stays at half an octet
#pragma unroll
    for (int h = 0; h < 2; h++) {
        // the weight pieces of row 4 rg + ((j + sl) & 3), slice s: from the lane that loaded them
        const uint32_t nat[4] = {h ? g.qb.x : g.qa.x, h ? g.qb.y : g.qa.y, h ? g.qb.z : g.qa.z, h ? g.qb.w : g.qa.w};
        int wq[4];
#pragma unroll
        for (int b = 0; b < 4; b++) wq[b] = __builtin_amdgcn_ds_bpermute(int(src_addr), int(nat[b]));
        float wd[4];
#pragma unroll
        for (int b = 0; b < 4; b++) wd[b] = h2f((b & 1) ? scw[2 * h + (b >> 1)] >> 16 : scw[2 * h + (b >> 1)] & 0xffffu);
        float pr[2][4];
        int xq[2][4];
#pragma unroll
        for (int tg = 0; tg < TG; tg++) {
            const float4 a = reinterpret_cast<const float4 *>(xt[tg] + n_oct * 16)[2 * o + h];
            pr[tg][0] = wd[0] * a.x, pr[tg][1] = wd[1] * a.y, pr[tg][2] = wd[2] * a.z, pr[tg][3] = wd[3] * a.w;
            const uint4 x = xt[tg][(2 * o + h) * 8 + s];
            xq[tg][0] = int(x.x), xq[tg][1] = int(x.y), xq[tg][2] = int(x.z), xq[tg][3] = int(x.w);
        }
        // a DPP read of a register needs two wait states after the vector instruction that wrote it, and the compiler
        // does not look into the asm statements below: all products pass this point first
        if constexpr (TG == 2)
            asm volatile("s_nop 1" : "+v"(pr[0][0]), "+v"(pr[0][1]), "+v"(pr[0][2]), "+v"(pr[0][3]), "+v"(pr[1][0]), "+v"(pr[1][1]), "+v"(pr[1][2]), "+v"(pr[1][3]));
        else
            asm volatile("s_nop 1" : "+v"(pr[0][0]), "+v"(pr[0][1]), "+v"(pr[0][2]), "+v"(pr[0][3]));
        // one product ahead of the sums: the matrix cores' result of step i + 1 is on its way while step i is added
        v4i_x4 d = __builtin_amdgcn_mfma_i32_4x4x4i8(wq[0], xq[0][0], zero4, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4 * TG; i++) {
            const int b = i / TG, tg = i % TG;
            v4i_x4 d_next = zero4;
            if (i + 1 < 4 * TG) d_next = __builtin_amdgcn_mfma_i32_4x4x4i8(wq[(i + 1) / TG], xq[(i + 1) % TG][(i + 1) / TG], zero4, 0, 0, 0);
            fmac_ror4<0>(acc[tg][0], pr[tg][b], float(d[0]));
            fmac_ror4<1>(acc[tg][1], pr[tg][b], float(d[1]));
            fmac_ror4<2>(acc[tg][2], pr[tg][b], float(d[2]));
            fmac_ror4<3>(acc[tg][3], pr[tg][b], float(d[3]));
            d = d_next;
        }
    }
}

template <int B, bool GROUPED, int MAXT>
__global__ __launch_bounds__(MAXT, kX4WavesPerSimd) void gemv_q8_0_x4_kernel(RmiGemvProblem single, const RmiGemvProblem *__restrict__ list,
                                                           const uint4 *__restrict__ runs, uint32_t tiles_per_wave) {
    static_assert(B >= 2 && B <= 8, "two to eight tokens");
    constexpr int TG = B > 4 ? 2 : 1;
    extern __shared__ uint4 lds[];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t j = lane & 3, sl = (lane >> 2) & 3, s_hi = (lane >> 4) & 1, rg = lane >> 5, s = 4 * s_hi + sl;
    const uint32_t a_row = 4 * rg + ((j + sl) & 3);      // the row whose slice s this lane gives the matrix cores
    const uint32_t src_addr = (8 * a_row + s) * 4;       // ... and the lane that loaded that piece (byte address of ds_bpermute)
    const uint32_t sc_row = 4 * rg + sl;                 // the row whose scale products this lane multiplies
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
        p.x_q8 += size_t(blockIdx.y) * B * p.n_in;  // token group blockIdx.y of the launch
        p.x_scales += size_t(blockIdx.y) * B * (p.n_in >> 5);
        p.y += size_t(blockIdx.y) * B * p.y_stride;
        k = w_idx * tiles_per_wave < p.n_tiles ? w_idx * tiles_per_wave : p.n_tiles;
        k_end = k + tiles_per_wave < p.n_tiles ? k + tiles_per_wave : p.n_tiles;
    }
    const uint32_t n_oct = p.n_oct;
    const uint32_t tok_u4 = rmi_gemv_x4_token_u4(n_oct);
    const uint32_t n_units = (k_end - k) * n_oct;
    struct Cursor {
        gptr_u4 sc_unit, q_unit;
        uint32_t o, n_oct, sc_row, lane;
        __device__ __forceinline__ void load(OctetRegs &g) const {
            g.sc = sc_unit[sc_row];
            g.qa = __builtin_nontemporal_load(q_unit + lane);
            g.qb = __builtin_nontemporal_load(q_unit + 64 + lane);
        }
        __device__ __forceinline__ void step() {
            sc_unit += 8;
            q_unit += 128;
            if (++o == n_oct) {
                o = 0;
                sc_unit += size_t(n_oct) * 128;
                q_unit += size_t(n_oct) * 8;
            }
        }
    } cur;
    {
        gptr_u4 tile = as_global<gptr_u4>(p.w + size_t(p.tile0 + (n_units ? k : 0)) * n_oct * kOctetBytes);
        cur = Cursor{tile, tile + n_oct * 8, 0, n_oct, sc_row, lane};
    }
    RmiRing<OctetRegs> ring;
    rmi_ring_fill(ring, n_units, cur);
    {
        stage_tokens<4>(reinterpret_cast<uint32_t *>(lds), tok_u4 * 4, p.x_q8, p.x_scales, B, n_oct, p.n_in >> 5, threadIdx.x,
                        blockDim.x);
        __syncthreads();
    }
    // Per wave behind the staged tokens: the results of up to four finished tiles, [tile & 3][token][row of the tile],
    // and the 8 x 32 partial sums of one group of four tokens at a tile's end, [slice][token of the group][row], rows
    // of 33 floats (the lanes of a wave write eight different slices at once).
    float *park = reinterpret_cast<float *>(lds + size_t(B) * tok_u4) + wave * kX4WaveFloats(B);
    float *red = park + 4 * B * 8;
    uint32_t red_w[4];  // where this lane's sum of result register v goes: row 4 rg + ((v + sl) & 3) of token j, slice s
#pragma unroll
    for (int v = 0; v < 4; v++) red_w[v] = s * 33 + j * 8 + 4 * rg + ((uint32_t(v) + sl) & 3);

    float acc[2][4];
#pragma unroll
    for (int tg = 0; tg < 2; tg++)
#pragma unroll
        for (int v = 0; v < 4; v++) acc[tg][v] = 0.0f;
    uint32_t o = 0, tiles_done = 0, flushed = 0;
    gptr_f32_w yp = as_global<gptr_f32_w>(p.y);
    auto flush = [&]() {
        // lane l < 32: tile l >> 3 of the group of four, row l & 7: a token's 32 results are 128 consecutive bytes
        const uint32_t t4 = (lane >> 3) & 3, row = (p.tile0 + k + flushed + t4) * 8 + (lane & 7);
        const bool live = lane < 32 && flushed + t4 < tiles_done && row >= p.row_start && row < p.row_end;
#pragma unroll
        for (int t = 0; t < B; t++) {
            const float v = park[(t4 * B + t) * 8 + (lane & 7)];
            if (live) yp[size_t(t) * p.y_stride + row] = v;
        }
        flushed = tiles_done;
    };
    auto consume = [&](const OctetRegs &g) {
        octet_fma_x4<B>(acc, g, lds, tok_u4, n_oct, o, s, j, src_addr);
        if (++o == n_oct) {
            // a tile's end stays a branch of its own: the sums pass through a statement the compiler may not move,
            // or it computes the whole combine ahead of the branch, in every unit
            asm volatile("; tile end"
                         : "+v"(acc[0][0]), "+v"(acc[0][1]), "+v"(acc[0][2]), "+v"(acc[0][3]), "+v"(acc[1][0]), "+v"(acc[1][1]),
                           "+v"(acc[1][2]), "+v"(acc[1][3]));
            o = 0;
            // The eight slices of a (row, token) meet through LDS, a group of four tokens at a time: every lane leaves
            // its four sums where lane (token, row) of the first 32 finds the eight slices of its output, and adds them
            // in hsum_ps order, ((l0 + l4) + (l1 + l5)) + ((l2 + l6) + (l3 + l7)).  A wave's LDS instructions are
            // carried out in order, but the compiler knows nothing of lanes that talk to each other through memory: it
            // had moved the upper lanes' writes of the second group in front of the lower lanes' reads of the first.
            // The wave barriers (no instruction: a point no memory access crosses, reached by all lanes) say so.
#pragma unroll
            for (int tg = 0; tg < TG; tg++) {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    red[red_w[v]] = acc[tg][v];
                    acc[tg][v] = 0.0f;
                }
                rmi_wave_lds_fence();
                float l[8];
#pragma unroll
                for (int sx = 0; sx < 8; sx++) l[sx] = red[sx * 33 + (lane & 31)];
                const float y = ((l[0] + l[4]) + (l[1] + l[5])) + ((l[2] + l[6]) + (l[3] + l[7]));
                const uint32_t tok = ((lane >> 3) & 3) + 4 * tg;
                if (lane < 32 && tok < B) park[((tiles_done & 3) * B + tok) * 8 + (lane & 7)] = y;
                rmi_wave_lds_fence();
            }
            tiles_done++;
            if ((tiles_done & 3) == 0) flush();
        }
    };
    rmi_ring_walk(ring, n_units, cur, consume);
    if (flushed < tiles_done) flush();
}

// Launches too small to fill the chip (one token, a matrix of at most a few thousand tiles) are bound by
// latency, not bandwidth: one wave per tile, and all loads of the tile's NOCT octets go out at once, before
// the activation is staged, so the wave sees one memory round trip instead of one per pipeline refill.
// Same arithmetic and order as the streaming kernel above.
// stage_token for one wave and NOCT <= 16 octets in two halves, so that other loads can go out between the
// activation's loads and the LDS writes that wait for them.
template <int NOCT>
struct TokenRegs {
    u32x4 v[(NOCT + 3) / 4];
    float sv0, sv1;
};
template <int NOCT>
__device__ __forceinline__ void wave_token_load(TokenRegs<NOCT> &t, const int8_t *x_q8, const float *x_scales, uint32_t nb,
                                                uint32_t lane) {
    gptr_u4 xq = as_global<gptr_u4>(x_q8);
    gptr_f32 xs = as_global<gptr_f32>(x_scales);
    const uint32_t src_u4 = nb * 2, s0 = lane, s1 = lane + 64;
#pragma unroll
    for (int j = 0; j < (NOCT + 3) / 4; j++) {
        const uint32_t i = lane + j * 64;
        t.v[j] = xq[i < src_u4 ? i : src_u4 - 1];
    }
    t.sv0 = xs[s0 < nb ? s0 : nb - 1];
    t.sv1 = xs[s1 < nb ? s1 : nb - 1];
}
template <int NOCT>
__device__ __forceinline__ void wave_token_store(const TokenRegs<NOCT> &t, uint32_t *dq, uint32_t nb, uint32_t lane) {
    static_assert(NOCT <= 16, "two scales a lane cover 128 blocks");
    const uint32_t n_u4 = NOCT * 16, src_u4 = nb * 2, s0 = lane, s1 = lane + 64;
#pragma unroll
    for (int j = 0; j < (NOCT + 3) / 4; j++) {
        const uint32_t i = lane + j * 64;
        if (i < n_u4) {
            const uint32_t b = i >> 1;  // block; this uint4 holds its dwords l = 4*(i&1) .. +3
            uint32_t *d = dq + (b >> 2) * 32 + (i & 1) * 16 + (b & 3);
            const bool live = i < src_u4;
            d[0] = live ? t.v[j].x : 0u;
            d[4] = live ? t.v[j].y : 0u;
            d[8] = live ? t.v[j].z : 0u;
            d[12] = live ? t.v[j].w : 0u;
        }
    }
    float *ds = reinterpret_cast<float *>(dq + NOCT * 64);
    if (s0 < NOCT * 8) ds[s0] = s0 < nb ? t.sv0 : 0.0f;
    if (s1 < NOCT * 8) ds[s1] = s1 < nb ? t.sv1 : 0.0f;
}

// The activation's loads go out first and the weights' behind them: loads come back in the order they were issued,
// so the activation is staged while the weights arrive and octet o is multiplied as soon as ITS pieces are there
// (a compute unit takes in a lone wave's 1 KiB loads one every 30 clocks or so, and an octet takes 200 clocks to
// multiply: with the activation last, nothing started before the last piece had arrived).
template <int NOCT>
__global__ __launch_bounds__(64) void gemv_q8_0_deep_kernel(RmiGemvProblem p) {
    extern __shared__ uint4 lds[];
    const uint32_t lane = threadIdx.x, r = lane >> 3, L = lane & 7;
    const uint32_t k = blockIdx.x;
    TokenRegs<NOCT> tok;
    wave_token_load<NOCT>(tok, p.x_q8, p.x_scales, p.n_in >> 5, lane);
    asm volatile("" : : : "memory");  // the compiler keeps this order of the loads (it had moved one of these behind the weights)
    gptr_u4 tile = as_global<gptr_u4>(p.w + size_t(p.tile0 + k) * NOCT * kOctetBytes);
    OctetRegs g[NOCT];
#pragma unroll
    for (int o = 0; o < NOCT; o++) {  // octet after octet, in the order they are multiplied
        load_octet(g[o], tile + r, tile + NOCT * 8 + lane, o);
        asm volatile("" : : : "memory");
    }
    wave_token_store<NOCT>(tok, reinterpret_cast<uint32_t *>(lds), p.n_in >> 5, lane);
    __syncthreads();
    float acc[1] = {0.0f};
    octets_fma_ahead<NOCT>(acc[0], g, lds, L);
    const uint32_t row = (p.tile0 + k) * kTileRows + r;
    const float y = hsum8_lanes(acc[0]);
    if (L == 0 && row >= p.row_start && row < p.row_end) as_global<gptr_f32_w>(p.y)[row] = y;
}

// The same kernel with the preceding "x += r; rms_norm(x, weight); quantize to Q8_0" folded into its prologue
// (src/models/qwen3.rs:719-734 and :1016-1027 run those three steps before the q/k/v and the gate/up products):
// every wave normalises and quantizes the whole activation itself, straight into the staged LDS layout, instead
// of reading what one more dependent launch would have written.  n_in = NOCT * 256.  Workgroup 0 also stores the
// updated residual stream to x_out, a buffer other than x_in (the other workgroups still read x_in).
struct RmiNormArgs {
    const float *x_in;    // residual stream
    const float *resid;   // added to it first (may be null)
    const float *weight;  // norm weight
    float *x_out;         // x_in + resid
    float eps;
    int rounding;
};

template <int NOCT>
__global__ __launch_bounds__(64) void gemv_q8_0_norm_deep_kernel(RmiGemvProblem p, RmiNormArgs na) {
    extern __shared__ uint4 lds[];
    const uint32_t lane = threadIdx.x, r = lane >> 3, L = lane & 7;
    const uint32_t k = blockIdx.x;
    const float4 *xin = reinterpret_cast<const float4 *>(na.x_in), *rin = reinterpret_cast<const float4 *>(na.resid),
                 *win = reinterpret_cast<const float4 *>(na.weight);
    float4 v[NOCT], a[NOCT], wv[NOCT];
#pragma unroll
    for (int j = 0; j < NOCT; j++) {  // lane owns the float4s lane, lane + 64, ...: element blocks stay in 8 lanes
        v[j] = xin[lane + 64 * j];
        if (na.resid) a[j] = rin[lane + 64 * j];
        wv[j] = win[lane + 64 * j];
    }
    gptr_u4 tile = as_global<gptr_u4>(p.w + size_t(p.tile0 + k) * NOCT * kOctetBytes);
    OctetRegs g[NOCT];
#pragma unroll
    for (int o = 0; o < NOCT; o++) {  // octet after octet, in the order they are multiplied
        load_octet(g[o], tile + r, tile + NOCT * 8 + lane, o);
        asm volatile("" : : : "memory");
    }

    double part = 0.0;
#pragma unroll
    for (int j = 0; j < NOCT; j++) {
        if (na.resid) {
            v[j].x += a[j].x;
            v[j].y += a[j].y;
            v[j].z += a[j].z;
            v[j].w += a[j].w;
        }
        const float s0 = v[j].x * v[j].x, s1 = v[j].y * v[j].y, s2 = v[j].z * v[j].z, s3 = v[j].w * v[j].w;
        part += double(s0);
        part += double(s1);
        part += double(s2);
        part += double(s3);
    }
    if (k == 0) {
#pragma unroll
        for (int j = 0; j < NOCT; j++) reinterpret_cast<float4 *>(na.x_out)[lane + 64 * j] = v[j];
    }
    part = wave_sum_f64(part);
    const float mean_sq = float(part / double(NOCT * 256));
    const float scale = 1.0f / sqrtf(mean_sq + na.eps);
    uint32_t *dq = reinterpret_cast<uint32_t *>(lds);
    float *ds = reinterpret_cast<float *>(dq + NOCT * 64);
#pragma unroll
    for (int j = 0; j < NOCT; j++) {
        float4 o;
        o.x = (v[j].x * scale) * wv[j].x;
        o.y = (v[j].y * scale) * wv[j].y;
        o.z = (v[j].z * scale) * wv[j].z;
        o.w = (v[j].w * scale) * wv[j].w;
        float sc;
        const uint32_t q = rmi_quantize_block8(o, na.rounding, &sc);
        const uint32_t b = (lane >> 3) + 8 * j;  // block of this float4; L = its dword inside the block
        dq[(b >> 2) * 32 + L * 4 + (b & 3)] = q;
        if (L == 0) ds[b] = sc;
    }
    __syncthreads();
    float acc[1] = {0.0f};
    octets_fma_ahead<NOCT>(acc[0], g, lds, L);
    const uint32_t row = (p.tile0 + k) * kTileRows + r;
    const float y = hsum8_lanes(acc[0]);
    if (L == 0 && row >= p.row_start && row < p.row_end) as_global<gptr_f32_w>(p.y)[row] = y;
}

// The norm in front of a tile on four waves (gemv_q8_0_deep_split_kernel): every wave normalises and quantizes a
// quarter of the activation (a lone wave's 400 instructions of it stood between the activation's arrival and the
// first product), multiplies a quarter of the tile's octets, and the first wave adds.  n_in = NOCT * 256, NOCT = 4 or 8.
template <int NOCT>
__global__ __launch_bounds__(256) void gemv_q8_0_norm_deep_split_kernel(RmiGemvProblem p, RmiNormArgs na) {
    static_assert(NOCT % 4 == 0, "whole octets a wave, whole float4s a thread");
    constexpr int N = NOCT / 4, R = NOCT / 4;  // octets a wave, float4s of the activation a thread
    extern __shared__ uint4 lds[];
    __shared__ double red[4];
    const uint32_t tid = threadIdx.x, lane = tid & 63, r = lane >> 3, L = lane & 7;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t k = blockIdx.x;
    const float4 *xin = reinterpret_cast<const float4 *>(na.x_in), *rin = reinterpret_cast<const float4 *>(na.resid),
                 *win = reinterpret_cast<const float4 *>(na.weight);
    float4 v[R], a[R], wv[R];
#pragma unroll
    for (int j = 0; j < R; j++) {  // thread owns the float4s tid, tid + 256, ...: element blocks stay in 8 lanes
        v[j] = xin[tid + 256 * j];
        if (na.resid) a[j] = rin[tid + 256 * j];
        wv[j] = win[tid + 256 * j];
    }
    asm volatile("" : : : "memory");  // the activation's loads stay in front of the weights'
    gptr_u4 tile = as_global<gptr_u4>(p.w + size_t(p.tile0 + k) * NOCT * kOctetBytes);
    OctetRegs g[N];
#pragma unroll
    for (int i = 0; i < N; i++) {
        load_octet(g[i], tile + r, tile + NOCT * 8 + lane, wave * N + i);
        asm volatile("" : : : "memory");
    }
    double part = 0.0;
#pragma unroll
    for (int j = 0; j < R; j++) {
        if (na.resid) {
            v[j].x += a[j].x;
            v[j].y += a[j].y;
            v[j].z += a[j].z;
            v[j].w += a[j].w;
        }
        const float s0 = v[j].x * v[j].x, s1 = v[j].y * v[j].y, s2 = v[j].z * v[j].z, s3 = v[j].w * v[j].w;
        part += double(s0);
        part += double(s1);
        part += double(s2);
        part += double(s3);
    }
    if (k == 0) {
#pragma unroll
        for (int j = 0; j < R; j++) reinterpret_cast<float4 *>(na.x_out)[tid + 256 * j] = v[j];
    }
    part = wave_sum_f64(part);
    if (lane == 0) red[wave] = part;
    __syncthreads();
    const double total = (red[0] + red[1]) + (red[2] + red[3]);
    const float mean_sq = float(total / double(NOCT * 256));
    const float scale = 1.0f / sqrtf(mean_sq + na.eps);
    uint32_t *dq = reinterpret_cast<uint32_t *>(lds);
    float *ds = reinterpret_cast<float *>(dq + NOCT * 64);
#pragma unroll
    for (int j = 0; j < R; j++) {
        float4 o;
        o.x = (v[j].x * scale) * wv[j].x;
        o.y = (v[j].y * scale) * wv[j].y;
        o.z = (v[j].z * scale) * wv[j].z;
        o.w = (v[j].w * scale) * wv[j].w;
        float sc;
        const uint32_t q = rmi_quantize_block8(o, na.rounding, &sc);
        const uint32_t b = (tid >> 3) + 32 * j;  // block of this float4; L = its dword inside the block
        dq[(b >> 2) * 32 + L * 4 + (b & 3)] = q;
        if (L == 0) ds[b] = sc;
    }
    __syncthreads();
    float4 *hand = reinterpret_cast<float4 *>(lds + NOCT * 18);
    if (wave != 0) octets_to_factors<N>(g, lds, NOCT, wave * N, L, hand + (wave - 1) * N * 4 * 64 + lane);
    float acc = 0.0f;
    if (wave == 0) octets_fma_ahead<N>(acc, g, lds, L, NOCT);
    __syncthreads();
    if (wave != 0) return;
    factors_sum<NOCT - N>(acc, hand + lane);
    const uint32_t row = (p.tile0 + k) * kTileRows + r;
    const float y = hsum8_lanes(acc);
    if (L == 0 && row >= p.row_start && row < p.row_end) as_global<gptr_f32_w>(p.y)[row] = y;
}

template <int NOCT>
int launch_gemv_norm_deep(const RmiGemvProblem &p, const RmiNormArgs &na, hipStream_t s) {
    if constexpr (NOCT % 4 == 0) {
        if (p.n_tiles <= 512) {  // two workgroups a compute unit; beyond, one-wave workgroups fill the chip by themselves
            constexpr size_t kLds = size_t(NOCT) * 288 + size_t(NOCT - NOCT / 4) * 4 * 64 * 16;
            hipLaunchKernelGGL((gemv_q8_0_norm_deep_split_kernel<NOCT>), dim3(p.n_tiles), dim3(256), kLds, s, p, na);
            RMI_HIP_CHECK(hipGetLastError());
            return RMI_HIP_OK;
        }
    }
    hipLaunchKernelGGL((gemv_q8_0_norm_deep_kernel<NOCT>), dim3(p.n_tiles), dim3(64), size_t(NOCT) * 288, s, p, na);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

// The gate and up products of one FFN with both neighbours folded in: the norm in front (as above, here shared
// by the workgroup) and `h = up * silu(gate)` quantized to Q8_0 behind (src/models/qwen3.rs:1016-1027,
// src/ops/activation/mod.rs:137-151).  The weight is the gate matrix stacked on the up matrix (n_ff rows each).
// A workgroup of eight waves takes 32 consecutive gate rows (waves 0-3, a tile each) and the same 32 up rows
// (waves 4-7): one Q8_0 block of h, which leaves as 32 int8 and its scale.  n_in = NOCT * 256 <= 2048.
template <int NOCT>
__global__ __launch_bounds__(512) void gemv_q8_0_norm_silu_kernel(const uint8_t *__restrict__ w, uint32_t up_tile0,
                                                                   RmiNormArgs na, int8_t *__restrict__ h_q8,
                                                                   float *__restrict__ h_scales) {
    extern __shared__ uint4 lds[];
    __shared__ double red[8];
    __shared__ float gu[64];
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane >> 3, L = lane & 7;
    const uint32_t tile_idx = (wave < 4 ? 0u : up_tile0) + blockIdx.x * 4 + (wave & 3);
    constexpr uint32_t kVec = NOCT * 64;  // float4s of the activation
    const bool owner = tid < kVec;        // whole waves: kVec is a multiple of 64
    float4 v, a, wv;
    if (owner) {
        v = reinterpret_cast<const float4 *>(na.x_in)[tid];
        if (na.resid) a = reinterpret_cast<const float4 *>(na.resid)[tid];
        wv = reinterpret_cast<const float4 *>(na.weight)[tid];
    }
    gptr_u4 tile = as_global<gptr_u4>(w + size_t(tile_idx) * NOCT * kOctetBytes);
    OctetRegs g[NOCT];
#pragma unroll
    for (int o = 0; o < NOCT; o++) {  // octet after octet, in the order they are multiplied
        load_octet(g[o], tile + r, tile + NOCT * 8 + lane, o);
        asm volatile("" : : : "memory");
    }

    if (owner) {
        if (na.resid) {
            v.x += a.x;
            v.y += a.y;
            v.z += a.z;
            v.w += a.w;
        }
        if (blockIdx.x == 0) reinterpret_cast<float4 *>(na.x_out)[tid] = v;
        const float s0 = v.x * v.x, s1 = v.y * v.y, s2 = v.z * v.z, s3 = v.w * v.w;
        double part = double(s0);
        part += double(s1);
        part += double(s2);
        part += double(s3);
        part = wave_sum_f64(part);
        if (lane == 0) red[wave] = part;
    }
    __syncthreads();
    uint32_t *dq = reinterpret_cast<uint32_t *>(lds);
    if (owner) {
        double total = red[0];
#pragma unroll
        for (uint32_t i = 1; i < kVec / 64; i++) total += red[i];
        const float mean_sq = float(total / double(NOCT * 256));
        const float scale = 1.0f / sqrtf(mean_sq + na.eps);
        float4 o;
        o.x = (v.x * scale) * wv.x;
        o.y = (v.y * scale) * wv.y;
        o.z = (v.z * scale) * wv.z;
        o.w = (v.w * scale) * wv.w;
        float sc;
        const uint32_t q = rmi_quantize_block8(o, na.rounding, &sc);
        const uint32_t b = tid >> 3;  // block of this float4; L = its dword inside the block
        dq[(b >> 2) * 32 + L * 4 + (b & 3)] = q;
        if (L == 0) reinterpret_cast<float *>(dq + NOCT * 64)[b] = sc;
    }
    __syncthreads();
    float acc[1] = {0.0f};
    octets_fma_ahead<NOCT>(acc[0], g, lds, L);
    const float y = hsum8_lanes(acc[0]);
    if (L == 0) gu[wave * 8 + r] = y;  // [0,32): gate rows of this block, [32,64): up rows
    __syncthreads();
    if (tid < 64) {  // the first wave: one of the 32 values per lane (one exp each), then four per lane for the quantizer
        const uint32_t i = tid & 31;
        const float gt = gu[i], up = gu[32 + i];
        const float hv = up * (gt / (1.0f + rmi_expf(-gt)));
        float4 h;
        h.x = __shfl(hv, int(4 * (tid & 7)), 64);
        h.y = __shfl(hv, int(4 * (tid & 7) + 1), 64);
        h.z = __shfl(hv, int(4 * (tid & 7) + 2), 64);
        h.w = __shfl(hv, int(4 * (tid & 7) + 3), 64);
        float sc;
        const uint32_t q = rmi_quantize_block8(h, na.rounding, &sc);
        if (tid < 8) reinterpret_cast<uint32_t *>(h_q8)[blockIdx.x * 8 + tid] = q;
        if (tid == 0) h_scales[blockIdx.x] = sc;
    }
}

template <int NOCT>
int launch_gemv_norm_silu(const rmi_hip_weight *w, const RmiNormArgs &na, int8_t *h_q8, float *h_scales, hipStream_t s) {
    const uint32_t n_ff = w->n_out / 2;
    hipLaunchKernelGGL((gemv_q8_0_norm_silu_kernel<NOCT>), dim3(n_ff / 32), dim3(512), size_t(NOCT) * 288, s, w->data,
                       n_ff / 8, na, h_q8, h_scales);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

// The q, k and v products of one attention block with both neighbours folded in, for head dimension 128: the
// norm in front (shared by the workgroup, as above) and, behind, what src/models/qwen3.rs:776-874 does to the
// three vectors: per-head RMS norm of q and k (when the model has those weights), NeoX rotation, rounding to
// f16, k and v into their cache row.  The weight is q stacked on k stacked on v.  A workgroup of 8 waves takes
// one head (16 tiles, two per wave); its first wave finishes the head.  n_in = NOCT * 256 <= 1024.
struct RmiRopeArgs {
    const float *q_norm, *k_norm;     // [128] each, or null
    const float *cos_row, *sin_row;   // [64] each: the angles of this position
    uint16_t *q16, *k_row, *v_row;    // f16 outputs: [n_head][128], [n_head_kv][128], [n_head_kv][128]
    uint32_t n_head, n_head_kv;
    float eps;
};

template <int NOCT>
__global__ __launch_bounds__(512) void gemv_q8_0_norm_rope_kernel(const uint8_t *__restrict__ w, RmiNormArgs na,
                                                                    RmiRopeArgs ra) {
    extern __shared__ uint4 lds[];
    __shared__ double red[8];
    __shared__ float yl[128];
    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane >> 3, L = lane & 7;
    const uint32_t head = blockIdx.x;
    constexpr uint32_t kVec = NOCT * 64;
    const bool owner = tid < kVec;
    float4 v, a, wv;
    if (owner) {
        v = reinterpret_cast<const float4 *>(na.x_in)[tid];
        if (na.resid) a = reinterpret_cast<const float4 *>(na.resid)[tid];
        wv = reinterpret_cast<const float4 *>(na.weight)[tid];
    }
    // two tiles per wave: eight waves finish sooner than sixteen with a tile each
    gptr_u4 tile = as_global<gptr_u4>(w + size_t(head * 16 + wave * 2) * NOCT * kOctetBytes);
    gptr_u4 tile2 = tile + NOCT * (kOctetBytes / 16);
    OctetRegs g[NOCT], g2[NOCT];
#pragma unroll
    for (int o = 0; o < NOCT; o++) {  // octet after octet, in the order they are multiplied
        load_octet(g[o], tile + r, tile + NOCT * 8 + lane, o);
        asm volatile("" : : : "memory");
    }
#pragma unroll
    for (int o = 0; o < NOCT; o++) {
        load_octet(g2[o], tile2 + r, tile2 + NOCT * 8 + lane, o);
        asm volatile("" : : : "memory");
    }
    // what the first wave needs at the end: out now, used after the products
    const bool is_q = head < ra.n_head, is_v = head >= ra.n_head + ra.n_head_kv;
    const float *nw = is_q ? ra.q_norm : ra.k_norm;
    float cos_a = 0.0f, sin_a = 0.0f, w0 = 1.0f, w1 = 1.0f;
    if (wave == 0 && !is_v) {
        cos_a = ra.cos_row[lane];
        sin_a = ra.sin_row[lane];
        if (nw) {
            w0 = nw[lane];
            w1 = nw[lane + 64];
        }
    }

    if (owner) {
        if (na.resid) {
            v.x += a.x;
            v.y += a.y;
            v.z += a.z;
            v.w += a.w;
        }
        if (head == 0) reinterpret_cast<float4 *>(na.x_out)[tid] = v;
        const float s0 = v.x * v.x, s1 = v.y * v.y, s2 = v.z * v.z, s3 = v.w * v.w;
        double part = double(s0);
        part += double(s1);
        part += double(s2);
        part += double(s3);
        part = wave_sum_f64(part);
        if (lane == 0) red[wave] = part;
    }
    __syncthreads();
    uint32_t *dq = reinterpret_cast<uint32_t *>(lds);
    if (owner) {
        double total = red[0];
#pragma unroll
        for (uint32_t i = 1; i < kVec / 64; i++) total += red[i];
        const float mean_sq = float(total / double(NOCT * 256));
        const float scale = 1.0f / sqrtf(mean_sq + na.eps);
        float4 o;
        o.x = (v.x * scale) * wv.x;
        o.y = (v.y * scale) * wv.y;
        o.z = (v.z * scale) * wv.z;
        o.w = (v.w * scale) * wv.w;
        float sc;
        const uint32_t q = rmi_quantize_block8(o, na.rounding, &sc);
        const uint32_t b = tid >> 3;
        dq[(b >> 2) * 32 + L * 4 + (b & 3)] = q;
        if (L == 0) reinterpret_cast<float *>(dq + NOCT * 64)[b] = sc;
    }
    __syncthreads();
    float acc[1] = {0.0f}, acc2[1] = {0.0f};
    octets_fma_ahead<NOCT>(acc[0], g, lds, L);
    octets_fma_ahead<NOCT>(acc2[0], g2, lds, L);
    const float y = hsum8_lanes(acc[0]), y2 = hsum8_lanes(acc2[0]);
    if (L == 0) {
        yl[wave * 16 + r] = y;
        yl[wave * 16 + 8 + r] = y2;
    }
    __syncthreads();
    if (wave != 0) return;
    const float x0r = yl[lane], x1r = yl[lane + 64];
    if (is_v) {
        uint16_t *dst = ra.v_row + size_t(head - ra.n_head - ra.n_head_kv) * 128;
        dst[lane] = rmi_f2h(x0r);
        dst[lane + 64] = rmi_f2h(x1r);
        return;
    }
    float x0 = x0r, x1 = x1r;
    if (nw) {
        const float q0 = x0r * x0r, q1 = x1r * x1r;
        double part = double(q0);
        part += double(q1);
        part = wave_sum_f64(part);
        const float mean_sq = float(part / 128.0);
        const float sc = 1.0f / sqrtf(mean_sq + ra.eps);
        x0 = (x0r * sc) * w0;
        x1 = (x1r * sc) * w1;
    }
    uint16_t *dst = is_q ? ra.q16 + size_t(head) * 128 : ra.k_row + size_t(head - ra.n_head) * 128;
    const float ta = x1 * -sin_a;
    const float tb = x1 * cos_a;
    dst[lane] = rmi_f2h(__builtin_fmaf(x0, cos_a, ta));
    dst[lane + 64] = rmi_f2h(__builtin_fmaf(x0, sin_a, tb));
}

template <int NOCT>
int launch_gemv_norm_rope(const rmi_hip_weight *w, const RmiNormArgs &na, const RmiRopeArgs &ra, hipStream_t s) {
    hipLaunchKernelGGL((gemv_q8_0_norm_rope_kernel<NOCT>), dim3(ra.n_head + 2 * ra.n_head_kv), dim3(512),
                       size_t(NOCT) * 288, s, w->data, na, ra);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

// The same tile on W waves, for launches that leave most of the chip idle anyway.  A lone wave multiplies an octet
// in about 200 clocks (36 vector instructions, dependent ones eight clocks apart), and only one in four of them is
// the row sums' own chain: fma(scale product, float(dot), acc), block after block.  Wave w loads the octets
// [w N, (w + 1) N), N = NOCT / W; waves 1.. multiply theirs down to the two factors of every block's fma and leave
// them in LDS; wave 0 multiplies the first N octets as before and then only adds: the same operations on the same
// values in the same order, a quarter of them on the critical path.  Every wave issues a quarter of the loads.
template <int NOCT, int W>
__global__ __launch_bounds__(64 * W) void gemv_q8_0_deep_split_kernel(RmiGemvProblem p) {
    static_assert(NOCT % W == 0 && NOCT * 16 <= 64 * W, "whole octets a wave, one piece of the activation a thread");
    constexpr int N = NOCT / W;
    extern __shared__ uint4 lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63, r = lane >> 3, L = lane & 7;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t k = blockIdx.x, nb = p.n_in >> 5;
    // the activation: thread t takes the 16-byte piece t and the block scale t (zeros beyond the nb source blocks)
    gptr_u4 xq = as_global<gptr_u4>(p.x_q8);
    gptr_f32 xs = as_global<gptr_f32>(p.x_scales);
    const uint32_t src_u4 = nb * 2;
    const u32x4 xv = xq[tid < src_u4 ? tid : src_u4 - 1];
    const float xsv = xs[tid < nb ? tid : nb - 1];
    asm volatile("" : : : "memory");  // the activation's loads stay in front of the weights'
    gptr_u4 tile = as_global<gptr_u4>(p.w + size_t(p.tile0 + k) * NOCT * kOctetBytes);
    OctetRegs g[N];
#pragma unroll
    for (int i = 0; i < N; i++) {  // octet after octet, in the order they are multiplied
        load_octet(g[i], tile + r, tile + NOCT * 8 + lane, wave * N + i);
        asm volatile("" : : : "memory");
    }
    uint32_t *dq = reinterpret_cast<uint32_t *>(lds);
    if (tid < NOCT * 16) {
        const uint32_t b = tid >> 1;  // block; this piece holds its dwords l = 4*(tid&1) .. +3
        uint32_t *d = dq + (b >> 2) * 32 + (tid & 1) * 16 + (b & 3);
        const bool live = tid < src_u4;
        d[0] = live ? xv.x : 0u;
        d[4] = live ? xv.y : 0u;
        d[8] = live ? xv.z : 0u;
        d[12] = live ? xv.w : 0u;
    }
    if (tid < NOCT * 8) reinterpret_cast<float *>(dq + NOCT * 64)[tid] = tid < nb ? xsv : 0.0f;
    __syncthreads();
    // the factors of the octets N .. NOCT - 1: [octet - N][pair of blocks q][lane] = {s, float(dot), s', float(dot')}
    float4 *hand = reinterpret_cast<float4 *>(lds + NOCT * 18);
    if (wave != 0) octets_to_factors<N>(g, lds, NOCT, wave * N, L, hand + (wave - 1) * N * 4 * 64 + lane);
    float acc = 0.0f;
    if (wave == 0) octets_fma_ahead<N>(acc, g, lds, L, NOCT);
    __syncthreads();
    if (wave != 0) return;
    factors_sum<NOCT - N>(acc, hand + lane);
    const uint32_t row = (p.tile0 + k) * kTileRows + r;
    const float y = hsum8_lanes(acc);
    if (L == 0 && row >= p.row_start && row < p.row_end) as_global<gptr_f32_w>(p.y)[row] = y;
}

template <int NOCT>
int launch_gemv_deep(const RmiGemvProblem &p, hipStream_t s) {
    hipLaunchKernelGGL((gemv_q8_0_deep_kernel<NOCT>), dim3(p.n_tiles), dim3(64), size_t(NOCT) * 288, s, p);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

constexpr uint32_t kDeepMaxOct = 12, kDeepMaxTiles = 4096;
template <int NOCT, int W>
int launch_gemv_deep_split(const RmiGemvProblem &p, hipStream_t s) {
    constexpr size_t kLds = size_t(NOCT) * 288 + size_t(NOCT - NOCT / W) * 4 * 64 * 16;
    static_assert(kLds <= 64 * 1024, "staged activation and handed-over factors");
    hipLaunchKernelGGL((gemv_q8_0_deep_split_kernel<NOCT, W>), dim3(p.n_tiles), dim3(64 * W), kLds, s, p);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

// Up to a workgroup a compute unit.  Beyond, one-wave workgroups fill the chip and the split only adds work
// (independent launches back to back, 512 tiles of 12 octets: 4.4 us against 4.1; 128 tiles: the same either way,
// and in a chain of dependent launches, which is where such a matrix is found, the split is the faster one).
constexpr uint32_t kDeepSplitMaxTiles = 256;
int dispatch_gemv_deep(const RmiGemvProblem &p, hipStream_t s) {
    if (p.n_tiles <= kDeepSplitMaxTiles) {
        switch (p.n_oct) {
            case 8: return launch_gemv_deep_split<8, 4>(p, s);  // (four octets: 3.3 us a launch either way)
            case 12: return launch_gemv_deep_split<12, 4>(p, s);
            default: break;
        }
    }
    switch (p.n_oct) {
        case 1: return launch_gemv_deep<1>(p, s);
        case 2: return launch_gemv_deep<2>(p, s);
        case 3: return launch_gemv_deep<3>(p, s);
        case 4: return launch_gemv_deep<4>(p, s);
        case 5: return launch_gemv_deep<5>(p, s);
        case 6: return launch_gemv_deep<6>(p, s);
        case 7: return launch_gemv_deep<7>(p, s);
        case 8: return launch_gemv_deep<8>(p, s);
        case 9: return launch_gemv_deep<9>(p, s);
        case 10: return launch_gemv_deep<10>(p, s);
        case 11: return launch_gemv_deep<11>(p, s);
        default: return launch_gemv_deep<12>(p, s);
    }
}

template <int B>
int launch_gemv(const RmiGemvProblem *single, const RmiGemvProblem *d_list, const uint4 *d_runs, uint32_t n_waves,
                uint32_t wpg,
                uint32_t tiles_per_wave, uint32_t max_n_oct, hipStream_t s, uint32_t token_groups = 1) {
    size_t lds_bytes = size_t(B) * max_n_oct * 288;
    if (lds_bytes > 64 * 1024)
        return rmi_fail(RMI_HIP_E_INVALID, "activation of %d tokens x %u elements does not fit the LDS staging", B,
                        max_n_oct * 256);
    const dim3 grid_single((n_waves + wpg - 1) / wpg, token_groups), grid_group(n_waves / wpg), block(64 * wpg);
    if constexpr (B >= 4) {
        // the kernel with the dots on the matrix cores, where its staging fits (its tokens lie further apart, and its
        // waves park finished tiles behind them)
        const size_t x4_bytes = size_t(B) * rmi_gemv_x4_token_u4(max_n_oct) * 16 + size_t(wpg) * kX4WaveFloats(B) * 4;
        if (x4_bytes <= 64 * 1024) {
            lds_bytes = x4_bytes;
            if (single && wpg == 1)
                hipLaunchKernelGGL((gemv_q8_0_x4_kernel<B, false, 64>), grid_single, block, lds_bytes, s, *single, d_list, d_runs, tiles_per_wave);
            else if (single)
                hipLaunchKernelGGL((gemv_q8_0_x4_kernel<B, false, 512>), grid_single, block, lds_bytes, s, *single, d_list, d_runs, tiles_per_wave);
            else if (wpg == 1)
                hipLaunchKernelGGL((gemv_q8_0_x4_kernel<B, true, 64>), grid_group, block, lds_bytes, s, RmiGemvProblem{}, d_list, d_runs, tiles_per_wave);
            else
                hipLaunchKernelGGL((gemv_q8_0_x4_kernel<B, true, 512>), grid_group, block, lds_bytes, s, RmiGemvProblem{}, d_list, d_runs, tiles_per_wave);
            RMI_HIP_CHECK(hipGetLastError());
            return RMI_HIP_OK;
        }
    }
    // the grouped run table is padded to whole workgroups
    if (single && wpg == 1)
        hipLaunchKernelGGL((gemv_q8_0_kernel<B, false, 64>), grid_single, block, lds_bytes, s, *single, d_list, d_runs,
                           tiles_per_wave);
    else if (single)
        hipLaunchKernelGGL((gemv_q8_0_kernel<B, false, 512>), grid_single, block, lds_bytes, s, *single, d_list, d_runs,
                           tiles_per_wave);
    else if (wpg == 1)
        hipLaunchKernelGGL((gemv_q8_0_kernel<B, true, 64>), grid_group, block, lds_bytes, s, RmiGemvProblem{}, d_list, d_runs,
                           tiles_per_wave);
    else
        hipLaunchKernelGGL((gemv_q8_0_kernel<B, true, 512>), grid_group, block, lds_bytes, s, RmiGemvProblem{}, d_list, d_runs,
                           tiles_per_wave);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

// token_groups > 1 (single problems only): n_tokens is the tokens of one group, the launch covers token_groups of them
int dispatch_gemv(uint32_t n_tokens, const RmiGemvProblem *single, const RmiGemvProblem *d_list, const uint4 *d_runs,
                  uint32_t n_waves, uint32_t wpg, uint32_t tiles_per_wave, uint32_t max_n_oct, hipStream_t s,
                  uint32_t token_groups = 1) {
    if (n_waves == 0) return RMI_HIP_OK;
    switch (n_tokens) {
        case 1: return launch_gemv<1>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, s, token_groups);
        case 2: return launch_gemv<2>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, s, token_groups);
        case 3: return launch_gemv<3>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, s, token_groups);
        case 4: return launch_gemv<4>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, s, token_groups);
        case 5: return launch_gemv<5>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, s, token_groups);
        case 6: return launch_gemv<6>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, s, token_groups);
        case 7: return launch_gemv<7>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, s, token_groups);
        case 8: return launch_gemv<8>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, s, token_groups);
        default: return rmi_fail(RMI_HIP_E_INVALID, "gemv takes 1..8 tokens per launch, got %u", n_tokens);
    }
}

// ---- per-block integer dots from the repacked stream ----
__global__ __launch_bounds__(256) void block_dots_q8_0_kernel(const uint8_t *__restrict__ w,
                                                               const int8_t *__restrict__ x_q8,
                                                               int32_t *__restrict__ dots, uint32_t n_out, uint32_t nb,
                                                               uint32_t n_oct) {
    const uint64_t total = uint64_t(n_out) * nb;
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < total;
         i += uint64_t(gridDim.x) * blockDim.x) {
        const uint32_t row = uint32_t(i / nb), b = uint32_t(i % nb);
        const uint8_t *tile = w + size_t(row >> 3) * n_oct * kOctetBytes;
        const uint32_t *quad =
            reinterpret_cast<const uint32_t *>(tile + size_t(n_oct) * 128 + size_t(b >> 2) * 1024 + (row & 7) * 128);
        const uint32_t *xq = reinterpret_cast<const uint32_t *>(x_q8 + size_t(b) * 32);
        int acc = 0;
        for (uint32_t L = 0; L < 8; L++) acc = __builtin_amdgcn_sdot4(int(quad[L * 4 + (b & 3)]), int(xq[L]), acc, false);
        dots[i] = acc;
    }
}

// ---- quantize_q8_0_into on the device: 8 lanes per 32-element block ----
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float *__restrict__ x, int8_t *__restrict__ q8,
                                                             float *__restrict__ scales, uint32_t n_blocks,
                                                             int rounding) {
    const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t b = gid >> 3, l = gid & 7;
    if (b >= n_blocks) return;  // whole 8-lane groups leave together
    const float4 v = reinterpret_cast<const float4 *>(x)[size_t(b) * 8 + l];
    float scale;
    reinterpret_cast<uint32_t *>(q8)[size_t(b) * 8 + l] = rmi_quantize_block8(v, rounding, &scale);
    if (l == 0) scales[b] = scale;
}

// ---- ops::matmul_q8_0 with f32 activations, AVX2 order (avx2.rs:180-217):
// two 8-lane accumulators; elements 0-7 and 16-23 of a block feed acc0, 8-15
// and 24-31 feed acc1, each as fma(d*float(q), x, acc); y = hsum(acc0+acc1).
// Lane i of 8 holds acc0[i] and acc1[i]; one 8-lane group per row. ----
__global__ __launch_bounds__(64) void matmul_q8_0_f32_kernel(const uint8_t *__restrict__ w,
                                                              const float *__restrict__ x, float *__restrict__ y,
                                                              uint32_t n_out, uint32_t nb, uint32_t n_oct) {
    const uint32_t lane = threadIdx.x, r = lane >> 3, i = lane & 7;
    const uint32_t tile_idx = blockIdx.x;
    const uint8_t *tile = w + size_t(tile_idx) * n_oct * kOctetBytes;
    const uint8_t *quants = tile + size_t(n_oct) * 128;
    float acc0 = 0.0f, acc1 = 0.0f;
    for (uint32_t b = 0; b < nb; b++) {
        const float d = h2f(reinterpret_cast<const uint16_t *>(tile + size_t(b >> 3) * 128 + r * 16)[b & 7]);
        const uint8_t *quad = quants + size_t(b >> 2) * 1024 + r * 128 + (b & 3) * 4;
        // element e of the block sits in the slice of lane e/4 at byte e%4
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint32_t e = g * 8 + i;
            const float q = float(int(int8_t(quad[(e >> 2) * 16 + (e & 3)])));
            const float wq = d * q;
            const float xv = x[size_t(b) * 32 + e];
            if (g & 1) acc1 = __builtin_fmaf(wq, xv, acc1); else acc0 = __builtin_fmaf(wq, xv, acc0);
        }
    }
    const float s = hsum8_lanes(acc0 + acc1);
    const uint32_t row = tile_idx * kTileRows + r;
    if (i == 0 && row < n_out) y[row] = s;
}

// ---- matmul_q8_0_fallback_range (scalar.rs:3-29): the f32-activation product on hosts without AVX2.  Per row
// one chain: local = 0; local += float(q[k]) * x[k] for the 32 elements of a block in order (product and sum
// rounded separately); sum += d * local block after block.  The eight lanes of a row each make the four products
// of their slice; the adds are one dependent chain, so every lane of the row runs it on values read from the
// other lanes (only lane 0's copy is stored). ----
__global__ __launch_bounds__(64) void matmul_q8_0_f32_scalar_kernel(const uint8_t *__restrict__ w,
                                                                     const float *__restrict__ x, float *__restrict__ y,
                                                                     uint32_t row_start, uint32_t row_end, uint32_t nb,
                                                                     uint32_t n_oct, uint32_t tile0) {
    const uint32_t lane = threadIdx.x, r = lane >> 3, i = lane & 7;
    const uint32_t tile_idx = tile0 + blockIdx.x;
    const uint8_t *tile = w + size_t(tile_idx) * n_oct * kOctetBytes;
    const uint8_t *quants = tile + size_t(n_oct) * 128;
    float sum = 0.0f;
    for (uint32_t b = 0; b < nb; b++) {
        const float d = h2f(reinterpret_cast<const uint16_t *>(tile + size_t(b >> 3) * 128 + r * 16)[b & 7]);
        const uint32_t qw = *reinterpret_cast<const uint32_t *>(quants + size_t(b >> 2) * 1024 + r * 128 + i * 16 + (b & 3) * 4);
        const float4 xv = *reinterpret_cast<const float4 *>(x + size_t(b) * 32 + i * 4);
        float p[4];
        p[0] = float(int(int8_t(qw & 0xff))) * xv.x;
        p[1] = float(int(int8_t((qw >> 8) & 0xff))) * xv.y;
        p[2] = float(int(int8_t((qw >> 16) & 0xff))) * xv.z;
        p[3] = float(int(int8_t(qw >> 24))) * xv.w;
        float local = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; k++) {
#pragma unroll
            for (int j = 0; j < 4; j++) local = local + __shfl(p[j], k, 8);
        }
        sum = sum + d * local;
    }
    const uint32_t row = tile_idx * kTileRows + r;
    if (i == 0 && row >= row_start && row < row_end) y[row - row_start] = sum;
}

// plain streaming copy: the known-size kernel that HBM traffic counters are scaled against
__global__ __launch_bounds__(256) void copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n) {
    for (size_t i = blockIdx.x * size_t(blockDim.x) + threadIdx.x; i < n; i += size_t(gridDim.x) * blockDim.x)
        dst[i] = src[i];
}

}  // namespace

// Tiles a wave takes in one run: about 16 tile-octets (34 KiB of weights), whatever the batch, so that
// staging the activation stays small against the weights read while the launch keeps many more runs than the
// chip holds waves; fewer when the launch would otherwise have too few waves to fill the chip.  (Measured on
// the Qwen3-0.6B set: 8..32 octets within 2 % of each other at one token, 16 best at 4 and 8 tokens.)
uint32_t rmi_gemv_tiles_per_wave(uint32_t n_oct, uint32_t launch_tiles, uint32_t n_tokens) {
    (void)n_tokens;
    const uint32_t target = 16;
    uint32_t tpw = n_oct >= target ? 1 : target / (n_oct ? n_oct : 1);
    const uint32_t fill = uint32_t(rmi_device_cus()) * 8;
    while (tpw > 1 && launch_tiles / tpw < fill) tpw >>= 1;
    return tpw ? tpw : 1;
}

// Waves per workgroup.  Every workgroup stages the whole activation in LDS before its waves start on their
// runs of tiles.  More waves share one copy (a) when LDS would otherwise hold too few workgroups to keep about
// 16 waves on a compute unit, and (b) until the staged bytes are small (an eighth) against the weight bytes the
// workgroup streams.  Measured on MI355X: Q4_K rows of 6144 at one token 4.2 -> 4.7 TB/s with four waves,
// Q8_0 at eight tokens 1.5 -> 2.4 TB/s; more than needed costs again (barrier and tail).
uint32_t rmi_gemv_waves_per_group(size_t lds_bytes, size_t run_bytes) {
    const size_t fit = lds_bytes ? (160 * 1024) / lds_bytes : 64;
    uint32_t wpg = 1;
    while (wpg < 8 && (fit * wpg < 16 || run_bytes * wpg < 8 * lds_bytes)) wpg <<= 1;
    return wpg;
}

int rmi_launch_copy(const void *src, void *dst, size_t nbytes, hipStream_t s) {
    const size_t n = nbytes / 16;
    if (n == 0) return RMI_HIP_OK;
    hipLaunchKernelGGL(copy_kernel, dim3(uint32_t(rmi_device_cus()) * 8), dim3(256), 0, s,
                       static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), n);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

// token_groups groups of n_tokens tokens each (n_tokens <= 8), consecutive in x_q8, x_scales and y, in one launch
int rmi_launch_gemv_q8_0_single(const RmiGemvProblem &p, uint32_t n_tokens, hipStream_t s, uint32_t token_groups) {
    if (p.n_tiles == 0 || p.n_oct == 0 || token_groups == 0) return RMI_HIP_OK;
    if (n_tokens == 1 && token_groups == 1 && p.n_oct <= kDeepMaxOct && p.n_tiles <= kDeepMaxTiles) return dispatch_gemv_deep(p, s);
    const uint32_t tpw = rmi_gemv_tiles_per_wave(p.n_oct, p.n_tiles, n_tokens);
    const uint32_t n_waves = (p.n_tiles + tpw - 1) / tpw, cus = uint32_t(rmi_device_cus() > 0 ? rmi_device_cus() : 1);
    {
        // A matrix of a few MB at several tokens is a launch of a few hundred waves with a long instruction stream
        // each (the x86-64 order costs about 30 vector instructions a token and octet): its tokens are spread over
        // workgroups, two or four to each, which re-read the weight from L2 and finish in a half or a quarter of
        // the time (every token's result is that of any other grouping: a token has its own accumulators).
        uint32_t per_group = n_tokens, groups = token_groups;
        while (per_group > 2 && per_group % 2 == 0 && n_waves * groups < 4 * cus) {
            per_group >>= 1;
            groups <<= 1;
        }
        if (groups > 1) {
            // the waves of a workgroup share the staged tokens of their group: as many as leave every compute unit
            // two workgroups or more
            uint32_t wpg = rmi_gemv_waves_per_group(size_t(per_group) * p.n_oct * 288, size_t(tpw) * p.n_oct * kOctetBytes);
            if (per_group >= 4 && wpg > 4) wpg = 4;  // as in the grouped launch: four-wave workgroups turn over more evenly
            while (wpg > 1 && uint64_t(n_waves / wpg) * groups < 2ull * cus) wpg >>= 1;
            return dispatch_gemv(per_group, &p, nullptr, nullptr, n_waves, wpg, tpw, p.n_oct, s, groups);
        }
    }
    uint32_t wpg = rmi_gemv_waves_per_group(size_t(n_tokens) * p.n_oct * 288, size_t(tpw) * p.n_oct * kOctetBytes);
    if (n_tokens >= 4 && wpg > 4) wpg = 4;
    // a launch with fewer waves than would give every compute unit a workgroup of that size is bound by latency,
    // not by the staging it shares: smaller workgroups on more compute units
    while (wpg > 1 && n_waves / wpg < cus) wpg >>= 1;
    return dispatch_gemv(n_tokens, &p, nullptr, nullptr, n_waves, wpg, tpw, p.n_oct, s);
}

bool rmi_gemv_q8_0_norm_fusable(const rmi_hip_weight *w) {
    return w->n_in % 256 == 0 && w->n_units >= 1 && w->n_units <= 8 && w->n_tiles >= 1 && w->n_tiles <= kDeepMaxTiles;
}

int rmi_launch_gemv_q8_0_norm(const rmi_hip_weight *w, const float *x_in, const float *resid, const float *norm_weight,
                              float *x_out, float eps, int rounding, float *y, hipStream_t s) {
    if (!rmi_gemv_q8_0_norm_fusable(w)) return rmi_fail(RMI_HIP_E_INVALID, "shape %u x %u is not fusable", w->n_out, w->n_in);
    RmiGemvProblem p{};
    p.w = w->data;
    p.y = y;
    p.n_in = w->n_in;
    p.n_oct = w->n_units;
    p.y_stride = w->n_out;
    p.row_start = 0;
    p.row_end = w->n_out;
    p.tile0 = 0;
    p.n_tiles = w->n_tiles;
    const RmiNormArgs na{x_in, resid, norm_weight, x_out, eps, rounding};
    switch (p.n_oct) {
        case 1: return launch_gemv_norm_deep<1>(p, na, s);
        case 2: return launch_gemv_norm_deep<2>(p, na, s);
        case 3: return launch_gemv_norm_deep<3>(p, na, s);
        case 4: return launch_gemv_norm_deep<4>(p, na, s);
        case 5: return launch_gemv_norm_deep<5>(p, na, s);
        case 6: return launch_gemv_norm_deep<6>(p, na, s);
        case 7: return launch_gemv_norm_deep<7>(p, na, s);
        default: return launch_gemv_norm_deep<8>(p, na, s);
    }
}

bool rmi_gemv_q8_0_norm_silu_fusable(const rmi_hip_weight *w) {
    return w->n_in % 256 == 0 && w->n_units >= 1 && w->n_units <= 8 && w->n_out >= 64 && w->n_out % 64 == 0 &&
           w->n_out / 64 <= 65535;
}

int rmi_launch_gemv_q8_0_norm_silu(const rmi_hip_weight *w_gate_up, const float *x_in, const float *resid,
                                   const float *norm_weight, float *x_out, float eps, int rounding, int8_t *h_q8,
                                   float *h_scales, hipStream_t s) {
    if (!rmi_gemv_q8_0_norm_silu_fusable(w_gate_up))
        return rmi_fail(RMI_HIP_E_INVALID, "shape %u x %u is not fusable", w_gate_up->n_out, w_gate_up->n_in);
    const RmiNormArgs na{x_in, resid, norm_weight, x_out, eps, rounding};
    switch (w_gate_up->n_units) {
        case 1: return launch_gemv_norm_silu<1>(w_gate_up, na, h_q8, h_scales, s);
        case 2: return launch_gemv_norm_silu<2>(w_gate_up, na, h_q8, h_scales, s);
        case 3: return launch_gemv_norm_silu<3>(w_gate_up, na, h_q8, h_scales, s);
        case 4: return launch_gemv_norm_silu<4>(w_gate_up, na, h_q8, h_scales, s);
        case 5: return launch_gemv_norm_silu<5>(w_gate_up, na, h_q8, h_scales, s);
        case 6: return launch_gemv_norm_silu<6>(w_gate_up, na, h_q8, h_scales, s);
        case 7: return launch_gemv_norm_silu<7>(w_gate_up, na, h_q8, h_scales, s);
        default: return launch_gemv_norm_silu<8>(w_gate_up, na, h_q8, h_scales, s);
    }
}

bool rmi_gemv_q8_0_norm_rope_fusable(const rmi_hip_weight *w, uint32_t n_head, uint32_t n_head_kv, uint32_t head_dim_k,
                                     uint32_t head_dim_v) {
    return head_dim_k == 128 && head_dim_v == 128 && w->n_in % 256 == 0 && w->n_units >= 1 && w->n_units <= 4 &&
           w->n_out == (n_head + 2 * n_head_kv) * 128;
}

int rmi_launch_gemv_q8_0_norm_rope(const rmi_hip_weight *w_qkv, const float *x_in, const float *resid,
                                   const float *norm_weight, float *x_out, float eps, int rounding, const float *q_norm,
                                   const float *k_norm, const float *cos_row, const float *sin_row, uint16_t *q16,
                                   uint16_t *k_row, uint16_t *v_row, uint32_t n_head, uint32_t n_head_kv, hipStream_t s) {
    if (!rmi_gemv_q8_0_norm_rope_fusable(w_qkv, n_head, n_head_kv, 128, 128))
        return rmi_fail(RMI_HIP_E_INVALID, "shape %u x %u is not fusable", w_qkv->n_out, w_qkv->n_in);
    const RmiNormArgs na{x_in, resid, norm_weight, x_out, eps, rounding};
    const RmiRopeArgs ra{q_norm, k_norm, cos_row, sin_row, q16, k_row, v_row, n_head, n_head_kv, eps};
    switch (w_qkv->n_units) {
        case 1: return launch_gemv_norm_rope<1>(w_qkv, na, ra, s);
        case 2: return launch_gemv_norm_rope<2>(w_qkv, na, ra, s);
        case 3: return launch_gemv_norm_rope<3>(w_qkv, na, ra, s);
        default: return launch_gemv_norm_rope<4>(w_qkv, na, ra, s);
    }
}

int rmi_launch_gemv_q8_0_group(const RmiGemvProblem *d_list, const uint4 *d_runs, uint32_t n_runs, uint32_t wpg,
                               uint32_t max_n_oct, uint32_t n_tokens, hipStream_t s) {
    return dispatch_gemv(n_tokens, nullptr, d_list, d_runs, n_runs, wpg, 0, max_n_oct, s);
}

int rmi_launch_block_dots_q8_0(const rmi_hip_weight *w, const int8_t *x_q8, int32_t *dots, hipStream_t s) {
    const uint64_t total = uint64_t(w->n_out) * (w->n_in / 32);
    if (total == 0) return RMI_HIP_OK;
    const uint32_t grid = uint32_t(total / 256 + 1 < 65535 ? total / 256 + 1 : 65535);
    hipLaunchKernelGGL(block_dots_q8_0_kernel, dim3(grid), dim3(256), 0, s, w->data, x_q8, dots, w->n_out,
                       w->n_in / 32, w->n_units);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_launch_quantize_q8_0(const float *x, int8_t *q8, float *scales, uint32_t n_tokens, uint32_t n_in,
                             int rounding, hipStream_t s) {
    const uint64_t n_blocks = uint64_t(n_tokens) * (n_in / 32);
    if (rounding != RMI_HIP_ROUND_HALF_AWAY && rounding != RMI_HIP_ROUND_TIES_EVEN && rounding != RMI_HIP_ROUND_NEON)
        return rmi_fail(RMI_HIP_E_INVALID, "unknown activation rounding %d", rounding);
    if (n_blocks == 0) return RMI_HIP_OK;
    if (n_blocks * 8 > 0xffffffffull) return rmi_fail(RMI_HIP_E_INVALID, "activation too large for one launch");
    const uint32_t grid = uint32_t((n_blocks * 8 + 255) / 256);
    hipLaunchKernelGGL(quantize_q8_0_kernel, dim3(grid), dim3(256), 0, s, x, q8, scales, uint32_t(n_blocks), rounding);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_launch_matmul_q8_0_f32_scalar(const rmi_hip_weight *w, const float *x, float *y, uint32_t row_start,
                                      uint32_t row_end, hipStream_t s) {
    if (row_end <= row_start) return RMI_HIP_OK;
    const uint32_t tile0 = row_start / kTileRows, n_tiles = (row_end + kTileRows - 1) / kTileRows - tile0;
    hipLaunchKernelGGL(matmul_q8_0_f32_scalar_kernel, dim3(n_tiles), dim3(64), 0, s, w->data, x, y, row_start, row_end,
                       w->n_in / 32, w->n_units, tile0);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_launch_matmul_q8_0_f32(const rmi_hip_weight *w, const float *x, float *y, hipStream_t s) {
    if (w->n_tiles == 0) return RMI_HIP_OK;
    hipLaunchKernelGGL(matmul_q8_0_f32_kernel, dim3(w->n_tiles), dim3(64), 0, s, w->data, x, y, w->n_out,
                       w->n_in / 32, w->n_units);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
