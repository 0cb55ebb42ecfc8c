// Q4_K x Q8_K prefill GEMM on the matrix cores: Y[t][n] = vec_dot_q4k_q8k(W[n], Q8_K(X[t])) for many tokens
// (Kernel::forward_batched semantics, src/ops/kernel/trait_.rs:78-109, with the dot of
// src/ops/quant/mod.rs:210-289 / 701-799).
//
// Per super-block (256 elements) and 32-token x 32-row tile the reference needs
//   sumi = sum_j scale_j * dot_j   (eight 32-element sub-blocks, 6-bit scales)     acc   = fma(d * q8d, float(sumi), acc)
//   prod = sum_j min_j * bsum_j    (bsum_j = the two 16-element sums of sub-block j) acc_m = fma(-dmin * q8d, float(prod), acc_m)
// Scaling eight int32 dot tiles would cost the vector ALU one multiply-add per output and sub-block.  Instead the
// scale goes into the weights before the multiply: a 6-bit scale is 8 * s_hi + s_lo with both parts below 8, a
// nibble times such a part is at most 105 and still an int8, and one packed 16-bit multiply scales the four nibbles
// of a dword at once (no byte overflows into its neighbour).  Two chains of int8 MFMAs 32x32x32, one on nibble * s_hi
// and one on nibble * s_lo, run through the whole super-block with the matrix cores' own accumulation, and
// sumi = 8 * D_hi + D_lo: the same integer, exactly.  A chain mixes sub-blocks freely, so an MFMA call takes, from
// each weight row, one 16-byte piece of the GEMV tile stream as it lies there (the packed nibbles go through LDS
// untouched: the workgroup copies whole 1 KB tiles, a lane then reads the pieces of its row half), and the token
// quants are laid out in LDS to match (see kXRow).  A wave owns 32 rows and 32*TTW tokens; the four waves of a
// workgroup share the tokens, so the scaled weight operands of a call are built once per wave and used for TTW
// token tiles.
//   * the min term: one f16 MFMA 32x32x16 delivers float(prod) itself.  A pair sum of bsums (13 bits, |s| <= 4064)
//     is split into its even part and its lowest bit, both exact f16 values, in k = 0..7 and 8..15; the eight mins
//     (below 64) meet both.  Every product and the sum are integers below 2^24, exact in the f32 accumulator;
//   * d * q8d and -dmin * q8d for the tile: one f32 outer-product MFMA (two blocks per instruction).
// All integers are exact (sumi is the sum of the reference's eight lane integers, prod of its four), and the
// f32 scale products are the reference's; the f32 accumulation runs over super-blocks in one chain per output
// instead of the AVX2 kernel's 8 + 4 lane chains, so results agree with it to rounding, not bit for bit.
//
// LDS is double-buffered, one barrier per super-block; every load, store and barrier of the loop is unconditional
// (indices past the end are clamped) and two super-blocks are unrolled, so the loop body is one basic block.
// Every global load of the quants is a full-line, coalesced 16 bytes per lane (the vector memory path of a compute
// unit is the scarce resource: 9 KB per wave and super-block); a piece goes to LDS one super-block after it was
// requested and its registers take the piece of the super-block after at once.
//
// What bounds it, by the kernel's own clock stamps around the parts of a super-block (two waves a SIMD): a wave's
// MFMAs and the vector instructions behind them do not overlap; with TTW = 2 the eight calls (32 MFMAs) take about
// 2300 clocks for the two waves of a SIMD, which is their MFMAs back to back, the fold and the next scales 1200,
// which is their vector instructions back to back, the barrier 300: the matrix-core half and the vector half add
// up.  Putting the two waves of a SIMD into opposite halves (a late start of every second workgroup; an eight-wave
// workgroup whose second four waves fold a super-block at the start of the next) changed nothing.  Folding a
// super-block between the MFMAs of the next one needs the chains twice: 64 more registers, which TTW = 2 does not
// have at two waves a SIMD (it stands at 254) and which did not pay with TTW = 1.
#include <type_traits>

#include "rmi_internal.h"

#include "device_common.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef const uint8_t __attribute__((address_space(1))) *gptr_u8;

// Bytes between the LDS rows of two tokens.  A row holds the 256 quants of a super-block in call order: call
// m = 2T + e (T = which of the four 16-byte pieces of a weight row half, e = low / high nibbles) multiplies, in
// lane half h, the elements 16h + 4T .. + 3 of the sub-blocks 2g + e, g = 0..3; those 16 quants are the 16 bytes
// at m * 32 + h * 16.  272 = 68 dwords: the 16-byte reads of 8 consecutive tokens fall into 8 different bank groups.
constexpr int kXRow = 272;
// bytes between the LDS rows of two weight rows (128 bytes of nibbles each); 136, which would let a third workgroup
// of the 32-token kernel into the LDS, costs more in bank conflicts than the third workgroup brings
constexpr int kWRow = 144;
constexpr int kBRow = 32;  // per token: the even parts of the eight pair sums as f16, then their lowest bits

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

// A scalar (workgroup-uniform) HBM base that the compiler may not fold a per-thread offset into: the access
// becomes global_load v_off, s[base].
template <typename T>
__device__ __forceinline__ gptr_u8 sbase(const T *p) {
    gptr_u8 b = (gptr_u8)(uintptr_t)p;
    asm("" : "+s"(b));
    return b;
}

// A per-thread offset whose zero-extension happens where it is used.
__device__ __forceinline__ uint32_t voff(uint32_t &o) {
    asm volatile("" : "+v"(o));
    return o;
}

// byte K of a in the low half of the result, byte K of b in the high half
template <int K>
__device__ __forceinline__ uint32_t byte_pair(uint32_t a, uint32_t b) {
    return __builtin_amdgcn_perm(b, a, 0x0c000c00u | uint32_t(K) | (uint32_t(4 + K) << 16));
}

// bytes K and K + 1 of w (integers below 1024) as two f16 values: 0x6400 | n is the f16 1024 + n
template <int K>
__device__ __forceinline__ uint32_t bytes_to_f16_pair(uint32_t w) {
    const uint32_t biased = __builtin_amdgcn_perm(0u, w, 0x0c000c00u | uint32_t(K) | (uint32_t(K + 1) << 16)) | 0x64006400u;
    const v2h k1024 = {_Float16(1024.0f), _Float16(1024.0f)};
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(v2h, biased) - k1024);
}

// WAVES_PER_SIMD bounds the registers of a thread: that many waves are to share a SIMD.
// DUMP (parity only): instead of folding them, the kernel writes the integers of every super-block as they leave
// the matrix cores, sumi = 8 * D_hi + D_lo and prod (the min term's f16 MFMA result, an integer below 2^24), to
// reinterpret_cast<int32_t *>(y)[((t * n_out + n) * n_sb + sb) * 2 + {0, 1}].
// KS > 1: KS groups of four waves share the tile; group ks takes the super-blocks ks, ks + KS, ... (n_in / 256 must
// be a multiple of KS), stages them in LDS of its own and keeps its own f32 chains; at the end the groups' results
// are added in group order.  For launches with no more tiles than the chip has compute units (a long row, a few
// hundred tokens): eight waves a compute unit instead of four, and half as many super-blocks in sequence.
template <int TTW, int WAVES_PER_SIMD, bool DUMP, int KS = 1>
__global__ __launch_bounds__(256 * KS, WAVES_PER_SIMD) void gemm_q4_k_kernel(const uint8_t *__restrict__ w, const float *__restrict__ q8d,
                                                                         const int8_t *__restrict__ q8qs,
                                                                         const int16_t *__restrict__ q8bs, float *__restrict__ y,
                                                                         uint32_t n_out, uint32_t n_sb, uint32_t n_tiles,
                                                                         uint32_t n_tokens, uint32_t y_stride, uint32_t grid_n,
                                                                         uint32_t grid_t, uint32_t t_fastest, uint32_t xcd_split) {
    constexpr int kTileN = 128, kTileT = 32 * TTW;
    constexpr int kXPieces = kTileT * 16 / 256;  // 16-byte pieces of the token tile per thread and super-block
    constexpr int kXBuf = kTileT * kXRow, kBBuf = kTileT * kBRow, kWBuf = kTileN * kWRow;
    static_assert(kXPieces <= 4, "the token pieces move to LDS in the first four calls of a super-block");
    __shared__ __attribute__((aligned(16))) uint8_t sm_w_all[KS * 2 * kWBuf];
    __shared__ __attribute__((aligned(16))) uint8_t sm_x_all[KS * 2 * kXBuf];
    __shared__ __attribute__((aligned(16))) uint8_t sm_b_all[KS * 2 * kBBuf];
    static_assert(KS == 1 || (KS - 1) * kTileT * 4 <= KS * 2 * kWRow, "the groups' results meet in the weight buffers");

    // ks: this wave's group; tid, wave: position inside the group (the whole workgroup for KS = 1)
    const uint32_t ks = KS == 1 ? 0u : uint32_t(__builtin_amdgcn_readfirstlane(int(threadIdx.x >> 8)));
    uint8_t *const sm_w = sm_w_all + ks * 2 * kWBuf, *const sm_x = sm_x_all + ks * 2 * kXBuf, *const sm_b = sm_b_all + ks * 2 * kBBuf;
    const uint32_t tid = threadIdx.x & 255, lane = tid & 63, wave = uint32_t(__builtin_amdgcn_readfirstlane(int(tid >> 6)));
    const uint32_t c = lane & 31, h = lane >> 5;
    const uint32_t n_off = wave * 32;
    uint32_t n_tile, t_tile;  // one XCD's workgroups take neighbouring tiles
    rmi_gemm_tile_of(blockIdx.x, grid_n, grid_t, t_fastest, xcd_split, n_tile, t_tile);
    const uint32_t n0 = n_tile * kTileN, t0 = t_tile * kTileT;
    const uint32_t n_in = n_sb * 256;
    // super-blocks of this group: sb stands for super-block sb * KS + ks
    const uint32_t n_sb_group = n_sb / KS, sb_last = n_sb_group - 1;
    auto realsb = [&](uint32_t sb) __attribute__((always_inline)) { return KS == 1 ? sb : sb * KS + ks; };
    auto clampsb = [&](uint32_t sb) __attribute__((always_inline)) { return sb < sb_last ? sb : sb_last; };

    // ---- addresses: a workgroup-uniform base that moves with the super-block, plus a 32-bit offset per thread.
    // Rows past the padded stream and tokens past the input read the last one again; their results are not stored.
    const uint32_t tile_first = (n0 >> 3) < n_tiles ? (n0 >> 3) : n_tiles - 1;
    const uint8_t *w_base = w + size_t(tile_first) * n_sb * kQ4KSuperBytes;
    uint32_t hd_off;
    {
        const uint32_t row = n0 + n_off + c;
        uint32_t tile = row >> 3;
        if (tile >= n_tiles) tile = n_tiles - 1;
        hd_off = (tile - tile_first) * n_sb * kQ4KSuperBytes + (row & 7) * 16;
    }
    // Weight nibbles: wave w copies the tiles w, w + 4, w + 8, w + 12 of the workgroup's 16, one 16-byte piece a
    // lane (1 KB per instruction, as it lies in the stream); piece lane % 8 of row lane / 8 of the tile.
    uint32_t w_tile_off[4];  // wave-uniform
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t tile = (n0 >> 3) + wave + 4 * i;
        if (tile >= n_tiles) tile = n_tiles - 1;
        w_tile_off[i] = (tile - tile_first) * n_sb * kQ4KSuperBytes + 128;
    }
    uint32_t w_ld = lane * 16;
    const uint32_t w_dst = (8 * wave + (lane >> 3)) * kWRow + (lane & 7) * 16;
    const uint32_t last_tok = n_tokens - 1 - t0;
    const int8_t *x_base = q8qs + size_t(t0) * n_in;
    // Token quants: load i of a thread is piece tid % 16 of token tid / 16 + 16 i (16 lanes cover a token's 256
    // bytes).  Piece 2j + hq is half hq of sub-block j = 2g + e; its dword T belongs to call 2T + e, lane half hq,
    // dword g.
    uint32_t x_off, x_lim, x_dst;
    {
        const uint32_t piece = tid & 15, j = piece >> 1, hq = piece & 1, g = j >> 1, e = j & 1;
        x_off = (tid >> 4) * n_in + piece * 16;  // + 16 i tokens, clamped to the last token's piece
        x_lim = last_tok * n_in + piece * 16;
        x_dst = (tid >> 4) * kXRow + e * 32 + hq * 16 + g * 4;
    }
    // bsums: thread (token tid / 8, pair tid % 8) of each 32-token group
    const uint8_t *bs_base = reinterpret_cast<const uint8_t *>(q8bs + size_t(t0) * n_sb * 16);
    const uint8_t *d_base = reinterpret_cast<const uint8_t *>(q8d + size_t(t0) * n_sb);
    uint32_t bs_off[TTW], d_off[TTW];
#pragma unroll
    for (int tt = 0; tt < TTW; tt++) {
        const uint32_t tokb = tt * 32 + (tid >> 3), tokd = tt * 32 + c;
        bs_off[tt] = (tokb < last_tok ? tokb : last_tok) * n_sb * 32 + (tid & 7) * 4;
        d_off[tt] = (tokd < last_tok ? tokd : last_tok) * n_sb * 4;
    }
    const uint32_t b_dst = (tid >> 3) * kBRow + (tid & 7) * 2;

    // ---- what is in flight
    u32x4 wst[4];         // weight pieces on their way to LDS
    u32x4 raw[2];         // piece T of this lane's row half, out of LDS: dword g = nibbles of sub-blocks 2g, 2g+1
    u32x4 hdr_n;          // the next super-block's header of this lane's row: d, dmin, 12 bytes of scales and mins
    u32x4 xst[kXPieces];  // token pieces on their way to LDS
    uint32_t bst[TTW];    // two bsums on their way to LDS
    float xd[TTW], xd_n[TTW];
    // current super-block: s_hi (low half) and s_lo (high half) of its eight sub-blocks; the eight mins as f16;
    // d of this lane's row in lanes 0..31 and -dmin in lanes 32..63 (the scale MFMA's operand)
    uint32_t s_pair[8];
    u32x4 mins;
    float wd;

    auto load_w = [&](int i, uint32_t sb) __attribute__((always_inline)) {
        wst[i] = *(gptr_u4)(sbase(w_base + size_t(realsb(sb)) * kQ4KSuperBytes + w_tile_off[i]) + voff(w_ld));
    };
    auto store_w = [&](int i, int buf) __attribute__((always_inline)) {
        *reinterpret_cast<u32x4 *>(sm_w + buf * kWBuf + w_dst + i * 32 * kWRow) = wst[i];
    };
    auto load_hdr = [&](uint32_t sb) __attribute__((always_inline)) {
        hdr_n = *(gptr_u4)(sbase(w_base + size_t(realsb(sb)) * kQ4KSuperBytes) + voff(hd_off));
#pragma unroll
        for (int tt = 0; tt < TTW; tt++)
            xd_n[tt] = __builtin_bit_cast(float, *(gptr_u32)(sbase(d_base + size_t(realsb(sb)) * 4) + voff(d_off[tt])));
    };
    auto take_hdr = [&]() __attribute__((always_inline)) {
        const uint4 s8 = unpack_scales(hdr_n.y, hdr_n.z, hdr_n.w);
        const uint32_t hi_a = (s8.x >> 3) & 0x07070707u, hi_b = (s8.y >> 3) & 0x07070707u;
        const uint32_t lo_a = s8.x & 0x07070707u, lo_b = s8.y & 0x07070707u;
        s_pair[0] = byte_pair<0>(hi_a, lo_a), s_pair[1] = byte_pair<1>(hi_a, lo_a), s_pair[2] = byte_pair<2>(hi_a, lo_a), s_pair[3] = byte_pair<3>(hi_a, lo_a);
        s_pair[4] = byte_pair<0>(hi_b, lo_b), s_pair[5] = byte_pair<1>(hi_b, lo_b), s_pair[6] = byte_pair<2>(hi_b, lo_b), s_pair[7] = byte_pair<3>(hi_b, lo_b);
        mins = u32x4{bytes_to_f16_pair<0>(s8.z), bytes_to_f16_pair<2>(s8.z), bytes_to_f16_pair<0>(s8.w), bytes_to_f16_pair<2>(s8.w)};
        const float d = h2f(hdr_n.x & 0xffffu), dmin = h2f(hdr_n.x >> 16);
        wd = h == 0 ? d : -dmin;
#pragma unroll
        for (int tt = 0; tt < TTW; tt++) xd[tt] = xd_n[tt];
    };
    auto load_x = [&](int i, uint32_t sb) __attribute__((always_inline)) {
        uint32_t off = x_off + uint32_t(i) * 16 * n_in;
        off = off < x_lim ? off : x_lim;
        xst[i] = *(gptr_u4)(sbase(x_base + size_t(realsb(sb)) * 256) + voff(off));
    };
    auto store_x = [&](int i, int buf) __attribute__((always_inline)) {
        uint8_t *dst = sm_x + buf * kXBuf + x_dst + i * 16 * kXRow;
        *reinterpret_cast<uint32_t *>(dst) = xst[i].x;
        *reinterpret_cast<uint32_t *>(dst + 64) = xst[i].y;
        *reinterpret_cast<uint32_t *>(dst + 128) = xst[i].z;
        *reinterpret_cast<uint32_t *>(dst + 192) = xst[i].w;
    };
    auto load_bs = [&](uint32_t sb) __attribute__((always_inline)) {
#pragma unroll
        for (int tt = 0; tt < TTW; tt++) bst[tt] = *(gptr_u32)(sbase(bs_base + size_t(realsb(sb)) * 32) + voff(bs_off[tt]));
    };
    auto store_bs = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int tt = 0; tt < TTW; tt++) {  // pair sum of bsums: even part and lowest bit, both exact as f16
            const int s = int(int16_t(bst[tt] & 0xffffu)) + int(int16_t(bst[tt] >> 16));
            uint8_t *dst = sm_b + buf * kBBuf + tt * 32 * kBRow + b_dst;
            *reinterpret_cast<_Float16 *>(dst) = _Float16(float(s & ~1));
            *reinterpret_cast<_Float16 *>(dst + 16) = _Float16(float(s & 1));
        }
    };

    // Operands in flight: the token operands and the two scaled weight operands of the current and the next call.
    v4i xv[2][TTW], w_hi[2], w_lo[2];
    uint32_t x_rd = c * kXRow + h * 16, b_rd = c * kBRow + h * 16, w_rd = (n_off + c) * kWRow + h * 64;
    auto read_w = [&](int T, int buf) __attribute__((always_inline)) {
        raw[T & 1] = *reinterpret_cast<const u32x4 *>(sm_w + buf * kWBuf + w_rd + T * 16);
    };
    auto read_x = [&](int s, int buf, int m) __attribute__((always_inline)) {
#pragma unroll
        for (int tt = 0; tt < TTW; tt++) {
            const u32x4 u = *reinterpret_cast<const u32x4 *>(sm_x + buf * kXBuf + x_rd + tt * 32 * kXRow + m * 32);
            xv[s][tt] = v4i{int(u.x), int(u.y), int(u.z), int(u.w)};
        }
    };
    // the weight operands of call m = 2T + e: nibble * s_hi and nibble * s_lo, four elements per multiply (the
    // multiply takes either half of the scale pair for both of its lanes); dwords 2 * half and 2 * half + 1
    auto prep_w = [&](int s, int m, int half) __attribute__((always_inline)) {
        const int T = m >> 1, e = m & 1;
#pragma unroll
        for (int g = 2 * half; g < 2 * half + 2; g++) {
            const uint32_t r = raw[T & 1][g];
            const u16x2 nib = __builtin_bit_cast(u16x2, (e ? r >> 4 : r) & 0x0f0f0f0fu);
            const u16x2 sp = __builtin_bit_cast(u16x2, s_pair[2 * g + e]);
            w_hi[s][g] = int(__builtin_bit_cast(uint32_t, u16x2(nib * u16x2{sp.x, sp.x})));
            w_lo[s][g] = int(__builtin_bit_cast(uint32_t, u16x2(nib * u16x2{sp.y, sp.y})));
        }
    };

    float acc[TTW][16], acc_m[TTW][16];
#pragma unroll
    for (int tt = 0; tt < TTW; tt++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[tt][i] = acc_m[tt][i] = 0.0f;
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const v16f zero16f = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    v16i d_hi[TTW], d_lo[TTW];  // the two chains of the super-block in work
#pragma unroll
    for (int tt = 0; tt < TTW; tt++) d_hi[tt] = d_lo[tt] = zero16;

    // ---- before the loop: super-block 0 into LDS buffer 0, the pieces of super-block 1 into the registers
#pragma unroll
    for (int i = 0; i < 4; i++) load_w(i, 0);
    load_hdr(0);
#pragma unroll
    for (int i = 0; i < kXPieces; i++) load_x(i, 0);
    load_bs(0);
#pragma unroll
    for (int i = 0; i < kXPieces; i++) {
        store_x(i, 0);
        load_x(i, clampsb(1));
    }
    store_bs(0);
    load_bs(clampsb(1));
#pragma unroll
    for (int i = 0; i < 4; i++) {
        store_w(i, 0);
        load_w(i, clampsb(1));
    }
    take_hdr();
    __syncthreads();
    read_x(0, 0, 0);
    read_w(0, 0);
    read_w(1, 0);
    prep_w(0, 0, 0);
    prep_w(0, 0, 1);

    // One super-block out of LDS buffer BUF.  Between the MFMAs of a call sit the weight operands of the next call.
    auto stage = [&](uint32_t sb, auto buf_c) __attribute__((always_inline)) {
        constexpr int BUF = decltype(buf_c)::value;
        const uint32_t sb1 = clampsb(sb + 1), sb2 = clampsb(sb + 2);
        u32x4 xbv[TTW];
        v32f zero32;
#pragma unroll
        for (int i = 0; i < 32; i++) zero32[i] = 0.0f;
#pragma unroll
        for (int m = 0; m < 8; m++) {
            const int s = m & 1;
            // pin: this call's operands have arrived and nothing of this call starts before
#pragma unroll
            for (int tt = 0; tt < TTW; tt++) asm volatile("" : "+v"(xv[s][tt]), "+v"(d_hi[tt]), "+v"(d_lo[tt]));
            asm volatile("" : "+v"(w_hi[s]), "+v"(w_lo[s]), "+v"(x_rd), "+v"(w_rd));
            if (m + 1 < 8) read_x(s ^ 1, BUF, m + 1);
#pragma unroll
            for (int tt = 0; tt < TTW; tt++) {
                d_hi[tt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xv[s][tt], w_hi[s], m == 0 ? zero16 : d_hi[tt], 0, 0, 0);
                if (tt == 0 && m + 1 < 8) prep_w(s ^ 1, m + 1, 0);
                d_lo[tt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xv[s][tt], w_lo[s], m == 0 ? zero16 : d_lo[tt], 0, 0, 0);
                if (tt == TTW - 1 && m + 1 < 8) prep_w(s ^ 1, m + 1, 1);
            }
            // both nibbles of piece (m + 1) / 2 are used up: its registers take the piece after the next
            if (m + 1 < 8 && ((m + 1) & 1) && (m + 1) / 2 + 2 < 4) read_w((m + 1) / 2 + 2, BUF);
            if (m < kXPieces) {
                store_x(m, BUF ^ 1);
                load_x(m, sb2);
            }
            if (m >= 4) {
                store_w(m - 4, BUF ^ 1);
                load_w(m - 4, sb2);
            }
            if (m == 0) load_hdr(sb1);
            if (m == 4) {
                store_bs(BUF ^ 1);
                load_bs(sb2);
            }
            if (m == 6) {
#pragma unroll
                for (int tt = 0; tt < TTW; tt++)
                    xbv[tt] = *reinterpret_cast<const u32x4 *>(sm_b + BUF * kBBuf + b_rd + tt * 32 * kBRow);
            }
        }
        // The scale products and the min term of a token tile come from the matrix cores: block 0 (lanes 0-31)
        // q8d * d, block 1 (lanes 32-63) q8d * (-dmin); then two multiply-adds per output.
#pragma unroll
        for (int tt = 0; tt < TTW; tt++) {
            const v32f sc = __builtin_amdgcn_mfma_f32_32x32x1f32(xd[tt], wd, zero32, 0, 0, 0);
            const v16f pm = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, xbv[tt]), __builtin_bit_cast(v8h, mins), zero16f, 0, 0, 0);
            if constexpr (DUMP) {
                const uint32_t n = n0 + n_off + c;
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const uint32_t t = t0 + tt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                    if (n < n_out && t < n_tokens) {
                        int32_t *dst = reinterpret_cast<int32_t *>(y) + ((size_t(t) * n_out + n) * n_sb + realsb(sb)) * 2;
                        dst[0] = d_hi[tt][i] * 8 + d_lo[tt][i];
                        dst[1] = int32_t(pm[i]);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < 16; i++) {
                acc[tt][i] = __builtin_fmaf(sc[i], float(d_hi[tt][i] * 8 + d_lo[tt][i]), acc[tt][i]);
                acc_m[tt][i] = __builtin_fmaf(sc[16 + i], pm[i], acc_m[tt][i]);
            }
        }
        take_hdr();
        __syncthreads();  // super-block sb + 1 is in the other buffer; nobody reads this one any more
        read_x(0, BUF ^ 1, 0);
        read_w(0, BUF ^ 1);
        read_w(1, BUF ^ 1);
        prep_w(0, 0, 0);
        prep_w(0, 0, 1);
    };

    uint32_t sb = 0;
    for (; sb + 1 < n_sb_group; sb += 2) {
        stage(sb, std::integral_constant<int, 0>{});
        stage(sb + 1, std::integral_constant<int, 1>{});
    }
    if (sb < n_sb_group) stage(sb, std::integral_constant<int, 0>{});
    if constexpr (KS > 1) {
        // the groups' results (their two chains added): groups 1.. leave theirs in LDS, group 0 adds them in group
        // order and stores
        __syncthreads();  // the loop ends with reads ahead into the buffers; they are over before the results land there
        float *comb = reinterpret_cast<float *>(sm_w_all);
#pragma unroll
        for (int tt = 0; tt < TTW; tt++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[tt][i] += acc_m[tt][i];
        if (ks != 0) {
#pragma unroll
            for (int tt = 0; tt < TTW; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) comb[((((ks - 1) * 4 + wave) * TTW + tt) * 16 + i) * 64 + lane] = acc[tt][i];
        }
        __syncthreads();
        if (ks != 0) return;
#pragma unroll 1
        for (uint32_t g = 1; g < KS; g++)
#pragma unroll
            for (int tt = 0; tt < TTW; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    acc[tt][i] += comb[((((g - 1) * 4 + wave) * TTW + tt) * 16 + i) * 64 + lane];
                    acc_m[tt][i] = 0.0f;
                }
    }
    // ---- results: lane (c, h) holds row n = c of 16 tokens
    const uint32_t n = n0 + n_off + c;
    if (!DUMP && n < n_out) {
#pragma unroll
        for (int tt = 0; tt < TTW; tt++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint32_t t = t0 + tt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                if (t < n_tokens) y[size_t(t) * y_stride + n] = acc[tt][i] + acc_m[tt][i];
            }
    }
}

template <int TTW, int WAVES_PER_SIMD, bool DUMP = false, int KS = 1>
void launch(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bs, float *y, uint32_t n_tokens,
            uint32_t y_stride, hipStream_t s) {
    const uint32_t grid_n = (w->n_out + 127) / 128, grid_t = (n_tokens + 32 * TTW - 1) / (32 * TTW);
    const uint32_t xcd_split = rmi_gemm_xcd_split(grid_n, grid_t, double(w->n_out) * w->n_units * 144.0, double(n_tokens) * w->n_units * 292.0);
    hipLaunchKernelGGL((gemm_q4_k_kernel<TTW, WAVES_PER_SIMD, DUMP, KS>), dim3(grid_n * grid_t), dim3(256 * KS), 0, s, w->data, d, qs, bs, y,
                       w->n_out, w->n_units, w->n_tiles, n_tokens, y_stride, grid_n, grid_t, n_tokens < w->n_out ? 1u : 0u, xcd_split);
}

}  // namespace

// Two groups of waves per tile, on the even and the odd super-blocks: where the 32-token tiles are no more than the
// chip has compute units and each group still has eight super-blocks or more (measured at 2048 x 6144, 512 tokens:
// 29.5 -> 24.3 us).  RMI_Q4K_GEMM_GROUPS = 1 or 2 forces a count where the row allows it.
static int gemm_q4_k_groups(const rmi_hip_weight *w, uint32_t n_tokens) {
    const uint64_t groups32 = uint64_t((w->n_out + 127) / 128) * ((n_tokens + 31) / 32);
    const char *e = getenv("RMI_Q4K_GEMM_GROUPS");
    const int force = e ? atoi(e) : 0;
    if (w->n_units % 2 != 0 || force == 1) return 1;
    if (force == 2) return 2;
    return groups32 <= uint64_t(rmi_device_cus()) && w->n_units >= 16 ? 2 : 1;
}

// token tile width (in units of 32) the launcher takes for this problem; RMI_Q4K_GEMM_TTW = 1 or 2 forces one
static int gemm_q4_k_ttw(const rmi_hip_weight *w, uint32_t n_tokens) {
    const uint64_t groups64 = uint64_t((w->n_out + 127) / 128) * ((n_tokens + 63) / 64);
    const char *e = getenv("RMI_Q4K_GEMM_TTW");
    const int force = e ? atoi(e) : 0;
    return force == 2 || (force != 1 && groups64 >= 2 * uint64_t(rmi_device_cus())) ? 2 : 1;
}

// The same kernel, same tile width as the product would take, writing its per-super-block integers instead of y:
// ints[n_tokens][n_out][n_sb][2] = {sumi, prod} (parity entry point).
int rmi_launch_gemm_q4_k_block_ints(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums,
                                    int32_t *ints, uint32_t n_tokens, hipStream_t s) {
    if (n_tokens == 0 || w->n_out == 0 || w->n_units == 0) return RMI_HIP_OK;
    if (uint64_t((w->n_out + 127) / 128) * ((n_tokens + 31) / 32) > 0x7fffffffull)
        return rmi_fail(RMI_HIP_E_INVALID, "GEMM too large for one launch");
    if (gemm_q4_k_groups(w, n_tokens) == 2)
        launch<1, 2, true, 2>(w, d, qs, bsums, reinterpret_cast<float *>(ints), n_tokens, w->n_out, s);
    else if (gemm_q4_k_ttw(w, n_tokens) == 2)
        launch<2, 2, true>(w, d, qs, bsums, reinterpret_cast<float *>(ints), n_tokens, w->n_out, s);
    else
        launch<1, 2, true>(w, d, qs, bsums, reinterpret_cast<float *>(ints), n_tokens, w->n_out, s);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

int rmi_launch_gemm_q4_k(const rmi_hip_weight *w, const float *d, const int8_t *qs, const int16_t *bsums, float *y,
                         uint32_t n_tokens, uint32_t y_stride, hipStream_t s) {
    if (n_tokens == 0 || w->n_out == 0 || w->n_units == 0) return RMI_HIP_OK;
    const uint64_t groups32 = uint64_t((w->n_out + 127) / 128) * ((n_tokens + 31) / 32);
    if (groups32 > 0x7fffffffull) return rmi_fail(RMI_HIP_E_INVALID, "GEMM too large for one launch");
    // 64-token tiles halve the vector work per output but want two workgroups on every compute unit;
    // RMI_Q4K_GEMM_TTW = 1 or 2 forces a width (the parity tests run both)
    if (gemm_q4_k_groups(w, n_tokens) == 2)
        launch<1, 2, false, 2>(w, d, qs, bsums, y, n_tokens, y_stride, s);
    else if (gemm_q4_k_ttw(w, n_tokens) == 2)
        launch<2, 2>(w, d, qs, bsums, y, n_tokens, y_stride, s);
    else
        launch<1, 2>(w, d, qs, bsums, y, n_tokens, y_stride, s);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}
