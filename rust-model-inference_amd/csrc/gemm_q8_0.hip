// Q8_0 x Q8_0 prefill GEMM on the matrix cores: Y[t][n] = sum_b (f32(wd[n][b]) * xs[t][b]) * dot_b(W[n], X[t]).
//
// One 32x32x32 int8 MFMA is one Q8_0 block (K = 32) of a 32-token x 32-row tile, so its int32 result is the
// per-block dot and starts from zero every block.  The f32 scale products wd*xs of the same tile are a rank-1
// outer product and come from the matrix cores, too, in the accumulator layout of the int8 result.  The weight
// scale is an f16, and the token scale the reference's quantizers write is an f16 value held in an f32
// (src/ops/quant/q8_0.rs:63, 121, 207): the product of two f16 values has 22 significant bits, so
// v_mfma_f32_32x32x8_f16 with the two scales in one k slot and zeros against everything else delivers it
// exactly, and it overlaps with VALU work.  A quad of blocks in which some token scale is not a finite f16 value
// (a caller's own prequantized input) takes v_mfma_f32_32x32x2_f32 instead: one f32 product plus zero, correctly
// rounded, subnormals included.  What is left for the VALU is acc = fma(float(dot), scale, acc) with the blocks
// in sequence: the order of matmul_q8_0_vs_q8_0_neon (src/ops/kernel/q8_0/neon.rs:49-73), bit for bit.
//
// Workgroup = WN x WT waves; wave (wn, wt) owns NTW x TTW MFMA tiles, i.e. 32*NTW weight rows x 32*TTW tokens.
// Per quad (4 blocks, 128 k) the workgroup stages both int8 operands into LDS in the natural k order, 128 bytes
// a row, rows 144 bytes apart so that the 16-byte reads of 8 consecutive lanes fall into 8 different bank groups.
// Weights come from the GEMV tile stream, whose 16-byte pieces hold the 4-byte slice L of blocks 0..3: each piece
// is written back as four dwords, one into each block of the row.  LDS is double-buffered, one barrier per quad.
//
// The loop is software-pipelined by hand, because the VALU has 32 instructions to issue per tile and block
// (convert, fma) against two MFMAs, and nothing else may sit on its path:
//  * a step = one (block, sub-tile): it issues its two MFMAs, then folds the results of the step before, whose
//    MFMAs have had a whole step to finish; an empty asm statement between steps carries the registers a step
//    needs, which keeps the compiler from hoisting every MFMA of the quad to the front (and spilling) or
//    sinking every fold to the end;
//  * the LDS reads of an operand go out one step (weights) or one block (tokens) ahead, the barrier and the
//    first reads of the next quad sit in the last step of this one;
//  * one 16-byte piece of the next quad moves from its registers to LDS per step, and the same registers then
//    take the piece of the quad after: global loads have a whole quad to arrive;
//  * every load, store and barrier of the loop is unconditional (indices past the end are clamped), two quads
//    are unrolled so that the LDS buffer is a compile-time constant, global addresses are a scalar base that
//    moves with the quad plus a 32-bit per-thread offset: the loop body is one basic block with exact wait
//    counts and about 5 % of VALU instructions beside the 32 per step.
// This file is compiled with the machine scheduler's pre-allocation pass off (see the Makefile): that pass
// stretches live ranges up to the register budget and makes the allocator spill the pieces in flight.
#include <type_traits>

#include "rmi_internal.h"

#include "device_common.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef const uint8_t __attribute__((address_space(1))) *gptr_u8;

constexpr int kRowStride = 144;  // bytes between rows of the LDS tiles

// A scalar (workgroup-uniform) HBM base that the compiler may not fold a per-thread offset into: the access
// becomes global_load / global_store v_off, s[base].
template <typename T>
__device__ __forceinline__ gptr_u8 sbase(const T *p) {
    gptr_u8 b = (gptr_u8)(uintptr_t)p;
    asm("" : "+s"(b));
    return b;
}

// A per-thread offset whose zero-extension happens where it is used (hoisted out of the loop as a 64-bit value
// it would no longer fit the scalar-base form).
__device__ __forceinline__ uint32_t voff(uint32_t &o) {
    asm volatile("" : "+v"(o));
    return o;
}

// RAGGED: n_in / 32 is not a multiple of 4 (the last quad is partly padding) or the token scales are not
// 16-byte aligned; token scales are then read one by one and indices past the row end are clamped.
// PER_CU bounds the registers a thread may take: it is the number of waves that are to share a SIMD (the second
// argument of __launch_bounds__), which for these four-wave workgroups is also the workgroups per compute unit.
// KS > 1 (not the aarch64 order any more, see rmi_launch_gemm_q8_0_fast): KS groups of WN x WT waves share the tile;
// group ks takes the quads ks, ks + KS, ks + 2 KS, ... (n_in / 128 must be a multiple of KS), stages them in LDS of
// its own and keeps its own f32 chain per output; at the end the groups' sums are added in group order.  With a
// single workgroup per compute unit this puts two or four waves on every SIMD where the tile grid has only as many
// tiles as the chip has compute units, and a compute unit draws only so many bytes a microsecond: fewer, larger
// tiles per unit are what a product of a few hundred tokens needs.
template <int NTW, int TTW, int WN, int WT, int PER_CU, bool RAGGED, int KS = 1>
__global__ __launch_bounds__(64 * WN * WT * KS, PER_CU) void gemm_q8_0_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ x_q8,
                                                                 const float *__restrict__ x_scales, float *__restrict__ y,
                                                                 uint32_t n_out, uint32_t n_in, uint32_t n_oct,
                                                                 uint32_t n_tiles, uint32_t n_tokens, uint32_t y_stride,
                                                                 uint32_t grid_n, uint32_t grid_t, uint32_t t_fastest, uint32_t xcd_split) {
    constexpr int kThreads = 64 * WN * WT;
    constexpr int kTileN = 32 * NTW * WN, kTileT = 32 * TTW * WT;
    constexpr int kWPieces = kTileN * 8 / kThreads;  // 16-byte pieces of the weight tile per thread
    constexpr int kXPieces = kTileT * 8 / kThreads;  // 16-byte pieces of the token tile per thread
    static_assert(kWPieces * kThreads == kTileN * 8 && kXPieces * kThreads == kTileT * 8, "tile must split evenly");
    constexpr int kSub = NTW * TTW, kSteps = 4 * kSub;
    constexpr int kPieces = kWPieces + kXPieces;
    constexpr int kWBuf = kTileN * kRowStride, kXBuf = kTileT * kRowStride;
    static_assert(KS == 1 || !RAGGED, "the quads of a ragged row are not split");
    static_assert(KS == 1 || (KS - 1) * kTileT * 4 <= KS * 2 * kRowStride, "the groups' sums meet in the weight buffers");
    __shared__ __attribute__((aligned(16))) uint8_t sm_w_all[KS * 2 * kWBuf];
    __shared__ __attribute__((aligned(16))) uint8_t sm_x_all[KS * 2 * kXBuf];

    // ks: this wave's group; tid, wave: position inside the group (a group is what the whole workgroup is for KS = 1)
    const uint32_t ks = KS == 1 ? 0u : uint32_t(__builtin_amdgcn_readfirstlane(int(threadIdx.x / kThreads)));
    uint8_t *const sm_w = sm_w_all + ks * 2 * kWBuf, *const sm_x = sm_x_all + ks * 2 * kXBuf;
    const uint32_t tid = KS == 1 ? threadIdx.x : threadIdx.x % kThreads, lane = tid & 63,
                   wave = uint32_t(__builtin_amdgcn_readfirstlane(int(tid >> 6)));
    const uint32_t c = lane & 31, h = lane >> 5;
    const uint32_t n_off = (wave % WN) * 32 * NTW, t_off = (wave / WN) * 32 * TTW;
    uint32_t n_tile, t_tile;  // one XCD's workgroups take neighbouring tiles
    rmi_gemm_tile_of(blockIdx.x, grid_n, grid_t, t_fastest, xcd_split, n_tile, t_tile);
    const uint32_t n0 = n_tile * kTileN, t0 = t_tile * kTileT;
    const uint32_t nb = n_in >> 5, n_quads = ((nb + 3) >> 2) / KS;  // quads of this group: q stands for quad q * KS + ks
    auto realq = [&](uint32_t q) __attribute__((always_inline)) { return KS == 1 ? q : q * KS + ks; };
    const uint32_t t_last = n_tokens - 1 - t0;  // last token of the input, counted from this tile's first

    // ---- addresses: a workgroup-uniform base that moves with the quad, plus a 32-bit offset per thread.
    // Rows past the padded stream and tokens past the input read the last one again; their results are not stored.
    const uint32_t tile_first = (n0 >> 3) < n_tiles ? (n0 >> 3) : n_tiles - 1;
    const uint8_t *w_base = w + size_t(tile_first) * n_oct * kOctetBytes;
    const uint8_t *wq_base = w_base + size_t(n_oct) * 128;
    uint32_t w_off[kWPieces], w_dst[kWPieces];
#pragma unroll
    for (int i = 0; i < kWPieces; i++) {
        const uint32_t p = tid + kThreads * i, row = p >> 3, L = p & 7;
        uint32_t tile = (n0 + row) >> 3;
        if (tile >= n_tiles) tile = n_tiles - 1;
        w_off[i] = (tile - tile_first) * n_oct * kOctetBytes + ((n0 + row) & 7) * 128 + L * 16;
        w_dst[i] = row * kRowStride + L * 4;
    }
    const int8_t *x_base = x_q8 + size_t(t0) * n_in;
    // in the last quad of a ragged row, pieces past n_in meet zero weight quants; only their addresses matter
    const uint64_t x_room = uint64_t(n_tokens - t0) * n_in - 16;
    const uint32_t x_lim = x_room < 0xfffffff0ull ? uint32_t(x_room) : 0xfffffff0u;
    uint32_t x_off[kXPieces], x_dst[kXPieces];
#pragma unroll
    for (int i = 0; i < kXPieces; i++) {
        const uint32_t p = tid + kThreads * i, tok = p >> 3, piece = p & 7;
        x_off[i] = (tok < t_last ? tok : t_last) * n_in + piece * 16;
        x_dst[i] = tok * kRowStride + piece * 16;
    }
    uint32_t wd_off[NTW];
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
        const uint32_t row = n0 + n_off + nt * 32 + c;
        uint32_t tile = row >> 3;
        if (tile >= n_tiles) tile = n_tiles - 1;
        wd_off[nt] = (tile - tile_first) * n_oct * kOctetBytes + (row & 7) * 16;
    }
    const uint8_t *xs_base = reinterpret_cast<const uint8_t *>(x_scales + size_t(t0) * nb);
    uint32_t xs_off[TTW];
#pragma unroll
    for (int tt = 0; tt < TTW; tt++) {
        const uint32_t tok = t_off + tt * 32 + c;
        xs_off[tt] = (tok < t_last ? tok : t_last) * nb * 4;
    }

    struct Stage {  // the 16-byte pieces of one quad, as loaded
        u32x4 w[kWPieces], x[kXPieces];
    };
    struct Scales {  // as loaded: the four f16 weight scales of the quad, the four f32 token scales
        u32x2 wd[NTW];
        u32x4 xs[TTW];
    };
    auto load_piece = [&](Stage &g, int pc, uint32_t q) __attribute__((always_inline)) {
        if (pc < kWPieces) {
            g.w[pc] = *(gptr_u4)(sbase(wq_base + size_t(realq(q)) * 1024) + voff(w_off[pc]));
        } else {
            const int i = pc - kWPieces;
            if (RAGGED) {
                const uint32_t off = x_off[i] + q * 128;
                g.x[i] = *reinterpret_cast<const u32x4 *>(x_base + (off < x_lim ? off : x_lim));
            } else {
                g.x[i] = *(gptr_u4)(sbase(x_base + size_t(realq(q)) * 128) + voff(x_off[i]));
            }
        }
    };
    auto store_piece = [&](const Stage &g, int pc, int buf) __attribute__((always_inline)) {
        if (pc < kWPieces) {
            uint8_t *dst = sm_w + buf * kWBuf + w_dst[pc];
            *reinterpret_cast<uint32_t *>(dst) = g.w[pc].x;
            *reinterpret_cast<uint32_t *>(dst + 32) = g.w[pc].y;
            *reinterpret_cast<uint32_t *>(dst + 64) = g.w[pc].z;
            *reinterpret_cast<uint32_t *>(dst + 96) = g.w[pc].w;
        } else {
            const int i = pc - kWPieces;
            *reinterpret_cast<u32x4 *>(sm_x + buf * kXBuf + x_dst[i]) = g.x[i];
        }
    };
    auto load_scales = [&](Scales &sc, uint32_t q_group) __attribute__((always_inline)) {
        const uint32_t q = realq(q_group);
        // weight scales of padded blocks are zero in the stream; token scales past n_in/32 are not there
        const gptr_u8 wb = sbase(w_base + ((q >> 1) * 128 + (q & 1) * 8));
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) sc.wd[nt] = *(gptr_u2)(wb + voff(wd_off[nt]));
        if (RAGGED) {
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const uint32_t b = q * 4 + p;  // past the row end the last scale is read; the consumer replaces it by zero
                const gptr_u8 xb = sbase(xs_base + size_t(b < nb ? b : nb - 1) * 4);
#pragma unroll
                for (int tt = 0; tt < TTW; tt++) sc.xs[tt][p] = *(gptr_u32)(xb + voff(xs_off[tt]));
            }
        } else {
            const gptr_u8 xb = sbase(xs_base + size_t(q) * 16);
#pragma unroll
            for (int tt = 0; tt < TTW; tt++) sc.xs[tt] = *(gptr_u4)(xb + voff(xs_off[tt]));
        }
    };

    Stage st;
    Scales sc[2];
    const uint32_t q_last = n_quads - 1;
    auto clampq = [&](uint32_t q) __attribute__((always_inline)) { return q < q_last ? q : q_last; };
#pragma unroll
    for (int pc = 0; pc < kPieces; pc++) load_piece(st, pc, 0);
    load_scales(sc[0], 0);

    v16f acc[NTW][TTW];
    const v16f zero16f = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int nt = 0; nt < NTW; nt++)
#pragma unroll
        for (int tt = 0; tt < TTW; tt++) acc[nt][tt] = zero16f;

    // Operands of the scale MFMA (v_mfma_f32_32x32x8_f16: k slots 0..3 in lanes 0..31, 4..7 in lanes 32..63).
    // Tokens: the f16 scales of blocks 2p and 2p+1 in k slots 0 and 1, in every lane (finite values; what they
    // meet in lanes 32..63 and in the other block's slot is zero).  Weights: the scale of the one block in its
    // slot, zero in the other slot and in lanes 32..63.  Slots 2 and 3 are the second register of each pair:
    // zero, set once here and hidden from the compiler, which would otherwise copy a zero next to every value;
    // the loop writes the first registers only.
    u32x2 wdp[NTW], xsp[TTW][2];
#pragma unroll
    for (int nt = 0; nt < NTW; nt++) {
        wdp[nt] = u32x2{0u, 0u};
        asm volatile("" : "+v"(wdp[nt]));
    }
#pragma unroll
    for (int tt = 0; tt < TTW; tt++)
#pragma unroll
        for (int p = 0; p < 2; p++) {
            xsp[tt][p] = u32x2{0u, 0u};
            asm volatile("" : "+v"(xsp[tt][p]));
        }
    const uint32_t mask_lo = h ? 0u : 0xffffu, mask_hi = h ? 0u : 0xffff0000u;

    // LDS read addresses; they pass through the pins below, which is what keeps a read from moving up
    uint32_t w_rd = (n_off + c) * kRowStride + h * 16, x_rd = (t_off + c) * kRowStride + h * 16;
    // Operands in flight: the token operands of the current and the next block, the weight operand of the
    // current and the next step.  MFMA lane (c, h) holds bytes 16h..16h+15 of the block of its row / token.
    v4i wv[2], xv[2][TTW];
    auto read_w = [&](int slot_, int buf, int blk, int nt) __attribute__((always_inline)) {
        const u32x4 u = *reinterpret_cast<const u32x4 *>(sm_w + buf * kWBuf + w_rd + nt * 32 * kRowStride + blk * 32);
        wv[slot_] = v4i{int(u.x), int(u.y), int(u.z), int(u.w)};
    };
    auto read_x = [&](int slot_, int buf, int blk) __attribute__((always_inline)) {
#pragma unroll
        for (int tt = 0; tt < TTW; tt++) {
            const u32x4 u = *reinterpret_cast<const u32x4 *>(sm_x + buf * kXBuf + x_rd + tt * 32 * kRowStride + blk * 32);
            xv[slot_][tt] = v4i{int(u.x), int(u.y), int(u.z), int(u.w)};
        }
    };

#pragma unroll
    for (int pc = 0; pc < kPieces; pc++) store_piece(st, pc, 0);
#pragma unroll
    for (int pc = 0; pc < kPieces; pc++) load_piece(st, pc, clampq(1));
    __syncthreads();
    read_x(0, 0, 0);
    read_w(0, 0, 0, 0);
    // the results of the step before; the first fold adds fma(0, 0, +0)
    v16i d_prev = zero16;
    v16f s_prev = zero16f;
    constexpr int kScaleStep = kPieces < kSteps - 1 ? kPieces : kSteps - 1;

    // Nonzero once a token scale of this wave was not a finite f16 value: the scale MFMA's products are then not
    // the f32 products, and the wave redoes its tiles the slow way after the loop.
    uint32_t not_f16 = 0;

    // One quad out of LDS buffer BUF.
    auto stage = [&](uint32_t q, auto buf_c) __attribute__((always_inline)) {
        constexpr int BUF = decltype(buf_c)::value;
        Scales &scq = sc[BUF];
#pragma unroll
        for (int tt = 0; tt < TTW; tt++) {
            _Float16 hx[4];
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const uint32_t xbits = scq.xs[tt][p];  // (a bit_cast of the vector element itself reads element 0)
                // a scale past n_in/32 must be a true zero: its block's dot is zero and the product must not be NaN
                const float x = (!RAGGED || q * 4 + p < nb) ? __builtin_bit_cast(float, xbits) : 0.0f;
                hx[p] = _Float16(x);
                // x - f32(f16(x)) is +-0 exactly when x is a finite f16 value (inf - inf and NaN are not)
                not_f16 |= __builtin_bit_cast(uint32_t, x - float(hx[p])) & 0x7fffffffu;
            }
            xsp[tt][0].x = __builtin_bit_cast(uint32_t, v2h{hx[0], hx[1]});
            xsp[tt][1].x = __builtin_bit_cast(uint32_t, v2h{hx[2], hx[3]});
        }
        const uint32_t q_ld = clampq(q + 2);
#pragma unroll
        for (int k = 0; k < kSteps; k++) {
            const int blk = k / kSub, nt = (k % kSub) / TTW, tt = k % TTW;
            const int pn = k == 0 ? NTW - 1 : ((k - 1) % kSub) / TTW, pt = k == 0 ? TTW - 1 : (k - 1) % TTW;
            const int ws = (k / TTW) & 1;
            // pin: what the previous step folded is done, this step's operands have arrived, and nothing of this
            // step starts before
            asm volatile("" : "+v"(acc[nt][tt]), "+v"(xv[blk & 1][tt]), "+v"(wv[ws]), "+v"(w_rd), "+v"(x_rd));
            if (k % kSub == 0 && blk + 1 < 4) read_x((blk + 1) & 1, BUF, blk + 1);
            if (k == kSteps - 1) {
                __syncthreads();  // quad q + 1 is in the other buffer; nobody reads this one any more
                read_x(0, BUF ^ 1, 0);
                read_w(0, BUF ^ 1, 0, 0);
            } else if ((k + 1) % TTW == 0) {
                read_w(ws ^ 1, BUF, (k + 1) / kSub, ((k + 1) % kSub) / TTW);
            }
            // blocks past n_in/32 in the last quad are zero on both sides (scale 0, quants 0):
            // fma(float(0), 0, acc) leaves acc unchanged, so they are multiplied like the rest
            const v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(xv[blk & 1][tt], wv[ws], zero16, 0, 0, 0);
            wdp[nt].x = (blk < 2 ? scq.wd[nt].x : scq.wd[nt].y) & (blk & 1 ? mask_hi : mask_lo);
            const v16f s = __builtin_amdgcn_mfma_f32_32x32x8f16(__builtin_bit_cast(v4h, xsp[tt][blk >> 1]),
                                                                __builtin_bit_cast(v4h, wdp[nt]), zero16f, 0, 0, 0);
            // one piece of the next quad moves to LDS per step, and its registers take the piece of the quad after
#pragma unroll
            for (int pc = k; k < kSteps - 1 && pc < kPieces; pc += kSteps - 1) {
                store_piece(st, pc, BUF ^ 1);
                load_piece(st, pc, q_ld);
            }
            if (k == kScaleStep) load_scales(sc[BUF ^ 1], clampq(q + 1));
#pragma unroll
            for (int i = 0; i < 16; i++) acc[pn][pt][i] = __builtin_fmaf(float(d_prev[i]), s_prev[i], acc[pn][pt][i]);
            d_prev = d;
            s_prev = s;
        }
    };

    uint32_t q = 0;
    for (; q + 1 < n_quads; q += 2) {
        stage(q, std::integral_constant<int, 0>{});
        stage(q + 1, std::integral_constant<int, 1>{});
    }
    if (q < n_quads) stage(q, std::integral_constant<int, 0>{});
#pragma unroll
    for (int i = 0; i < 16; i++)
        acc[NTW - 1][TTW - 1][i] = __builtin_fmaf(float(d_prev[i]), s_prev[i], acc[NTW - 1][TTW - 1][i]);

    if (__builtin_amdgcn_ballot_w64(not_f16 != 0) != 0) {
        // Token scales that are not f16 values: the wave's tiles again, block by block straight from HBM, with the
        // scale product from v_mfma_f32_32x32x2_f32 (k slot 0 in lanes 0..31, slot 1, zero on both sides, in lanes
        // 32..63).  Slow, and only a caller's own scales get here.
#pragma unroll 1
        for (int sub = 0; sub < kSub; sub++) {
            const uint32_t nt = uint32_t(sub) / TTW, tt = uint32_t(sub) % TTW;
            const uint32_t row = n0 + n_off + nt * 32 + c, tok = t_off + tt * 32 + c;
            uint32_t tile = row >> 3;
            if (tile >= n_tiles) tile = n_tiles - 1;
            const uint8_t *w_tile = w + size_t(tile) * n_oct * kOctetBytes;
            const uint8_t *w_row = w_tile + size_t(n_oct) * 128 + (row & 7) * 128 + h * 64;
            const size_t tok_c = size_t(t0) + (tok < t_last ? tok : t_last);
            const int8_t *x_row = x_q8 + tok_c * n_in + h * 16;
            v16f a = zero16f;
#pragma unroll 1
            for (uint32_t b = 0; b < nb; b++) {
                if (KS > 1 && (b >> 2) % KS != ks) continue;  // another group's quad
                const uint8_t *wp = w_row + size_t(b >> 2) * 1024 + (b & 3) * 4;
                const v4i wo = {int(*reinterpret_cast<const uint32_t *>(wp)), int(*reinterpret_cast<const uint32_t *>(wp + 16)),
                                int(*reinterpret_cast<const uint32_t *>(wp + 32)), int(*reinterpret_cast<const uint32_t *>(wp + 48))};
                const u32x4 xu = *reinterpret_cast<const u32x4 *>(x_row + size_t(b) * 32);
                const v4i xo = {int(xu.x), int(xu.y), int(xu.z), int(xu.w)};
                const uint32_t wd_bits = *reinterpret_cast<const uint16_t *>(w_tile + size_t(b >> 3) * 128 + (row & 7) * 16 + (b & 7) * 2);
                const float wd_f = h ? 0.0f : h2f(wd_bits);
                const float xs_f = h ? 0.0f : x_scales[tok_c * nb + b];
                const v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(xo, wo, zero16, 0, 0, 0);
                const v16f sp = __builtin_amdgcn_mfma_f32_32x32x2f32(xs_f, wd_f, zero16f, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 16; i++) a[i] = __builtin_fmaf(float(d[i]), sp[i], a[i]);
            }
            // sub is a loop counter, not a constant: the tile is handed over through a compare per candidate
#pragma unroll
            for (int n2 = 0; n2 < NTW; n2++)
#pragma unroll
                for (int t2 = 0; t2 < TTW; t2++)
                    if (n2 * TTW + t2 == sub) acc[n2][t2] = a;
        }
    }

    if constexpr (KS > 1) {
        // the groups' sums: groups 1.. leave theirs in LDS, group 0 adds them in group order and stores
        __syncthreads();  // nobody reads a staging buffer any more
        float *comb = reinterpret_cast<float *>(sm_w_all);
        if (ks != 0) {
#pragma unroll
            for (int nt = 0; nt < NTW; nt++)
#pragma unroll
                for (int tt = 0; tt < TTW; tt++)
#pragma unroll
                    for (int i = 0; i < 16; i++)
                        comb[((((ks - 1) * WN * WT + wave) * kSub + nt * TTW + tt) * 16 + i) * 64 + lane] = acc[nt][tt][i];
        }
        __syncthreads();
        if (ks != 0) return;
#pragma unroll 1
        for (uint32_t g = 1; g < KS; g++)
#pragma unroll
            for (int nt = 0; nt < NTW; nt++)
#pragma unroll
                for (int tt = 0; tt < TTW; tt++)
#pragma unroll
                    for (int i = 0; i < 16; i++)
                        acc[nt][tt][i] += comb[((((g - 1) * WN * WT + wave) * kSub + nt * TTW + tt) * 16 + i) * 64 + lane];
    }
    // ---- results: lane (c, h) holds row n = c of 16 tokens
    const uint32_t t_w = t0 + t_off, n_w = n0 + n_off;
    if (t_w + 32 * TTW <= n_tokens && n_w + 32 * NTW <= n_out) {
        // a scalar base per store, one offset per lane
        uint32_t v_off = (4 * h * y_stride + c) * 4;
#pragma unroll
        for (int nt = 0; nt < NTW; nt++)
#pragma unroll
            for (int tt = 0; tt < TTW; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const uint32_t t = t_w + tt * 32 + 8 * (i >> 2) + (i & 3);
                    const gptr_u8 base = sbase(y + size_t(t) * y_stride + n_w + nt * 32);
                    *(gptr_f32_w)(uintptr_t)(base + voff(v_off)) = acc[nt][tt][i];
                }
    } else {
#pragma unroll
        for (int nt = 0; nt < NTW; nt++) {
            const uint32_t n = n_w + nt * 32 + c;
            if (n < n_out) {
#pragma unroll
                for (int tt = 0; tt < TTW; tt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const uint32_t t = t_w + tt * 32 + 8 * (i >> 2) + 4 * h + (i & 3);
                        if (t < n_tokens) y[size_t(t) * y_stride + n] = acc[nt][tt][i];
                    }
            }
        }
    }
}

typedef void (*GemmLaunch)(const rmi_hip_weight *, const int8_t *, const float *, float *, uint32_t, uint32_t, bool,
                           hipStream_t);

template <int NTW, int TTW, int WN, int WT, int PER_CU, int KS>
void launch_gemm(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y, uint32_t n_tokens,
                 uint32_t y_stride, bool ragged, hipStream_t s) {
    constexpr uint32_t tile_n = 32 * NTW * WN, tile_t = 32 * TTW * WT;
    const uint32_t grid_n = (w->n_out + tile_n - 1) / tile_n, grid_t = (n_tokens + tile_t - 1) / tile_t;
    const uint32_t xcd_split = rmi_gemm_xcd_split(grid_n, grid_t, double(w->n_out) * w->n_in * (34.0 / 32.0), double(n_tokens) * w->n_in * (36.0 / 32.0));
    if constexpr (KS == 1) {
        if (ragged) {
            hipLaunchKernelGGL((gemm_q8_0_kernel<NTW, TTW, WN, WT, PER_CU, true>), dim3(grid_n * grid_t), dim3(64 * WN * WT), 0, s,
                               w->data, x_q8, x_scales, y, w->n_out, w->n_in, w->n_units, w->n_tiles, n_tokens, y_stride,
                               grid_n, grid_t, n_tokens < w->n_out ? 1u : 0u, xcd_split);
            return;
        }
    }
    hipLaunchKernelGGL((gemm_q8_0_kernel<NTW, TTW, WN, WT, PER_CU, false, KS>), dim3(grid_n * grid_t), dim3(64 * WN * WT * KS), 0, s,
                       w->data, x_q8, x_scales, y, w->n_out, w->n_in, w->n_units, w->n_tiles, n_tokens, y_stride,
                       grid_n, grid_t, n_tokens < w->n_out ? 1u : 0u, xcd_split);
}

// A tile shape: rows x tokens of a workgroup, sub-tiles per wave, waves of a group, groups that split the quads, how
// many workgroups a compute unit holds at once (asked of the runtime once: it knows the registers and the LDS the
// compiled kernel takes).
struct GemmShape {
    uint32_t tile_n, tile_t, sub, waves, ks;
    int per_cu;
    GemmLaunch launch;
};

template <int NTW, int TTW, int WN, int WT, int PER_CU, int KS = 1>
GemmShape make_shape() {
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, gemm_q8_0_kernel<NTW, TTW, WN, WT, PER_CU, false, KS>, 64 * WN * WT * KS, 0) !=
            hipSuccess ||
        per_cu < 1) {
        (void)hipGetLastError();
        per_cu = 1;
    }
    return GemmShape{32u * NTW * WN, 32u * TTW * WT, uint32_t(NTW * TTW), uint32_t(WN * WT), uint32_t(KS), per_cu,
                     launch_gemm<NTW, TTW, WN, WT, PER_CU, KS>};
}

}  // namespace

namespace {

struct GemmPlan {
    const GemmShape *shape;
    double cost_us;
};

// Every wave spends about the same time per sub-tile and block (the rescale on the VALU) and the waves of a SIMD
// share it, so a launch takes about (waves on the busiest SIMD) x (sub-tiles per wave) steps per block, round
// after round of workgroups, plus a fixed cost per round (first loads, last stores).  Measured on MI355X, a
// step: 90 ns with three or more waves on the SIMD or several sub-tiles per wave, 105 ns with two waves of one
// sub-tile, 125 ns for a wave alone; a round: about 3.5 us.  A compute unit also draws only about 40 KB a
// microsecond from L2 and memory, whatever its waves do, so a round takes at least its workgroups' operand bytes at
// that rate.  The shape with the smallest estimate is taken, the larger tile on a tie (less traffic): 96x128
// (4 waves x 3 sub-tiles, two workgroups a compute unit) for large products, 64x128 and 64x64 where those would
// leave compute units idle.  single_chain: only the shapes that keep one f32 chain per output.
GemmPlan plan_gemm(const rmi_hip_weight *w, uint32_t n_tokens, bool single_chain) {
    static const GemmShape shapes[] = {make_shape<3, 1, 1, 4, 2>(),    make_shape<2, 1, 1, 4, 2>(),    make_shape<1, 1, 2, 2, 3>(),
                                       make_shape<3, 1, 1, 4, 2, 2>(), make_shape<2, 1, 1, 4, 2, 2>(), make_shape<1, 1, 2, 2, 2, 2>(),
                                       make_shape<1, 1, 2, 1, 2, 4>()};
    constexpr int kShapes = int(sizeof(shapes) / sizeof(shapes[0]));
    const uint64_t cus = uint64_t(rmi_device_cus() > 0 ? rmi_device_cus() : 1);
    const uint32_t n_quads = (w->n_in / 32 + 3) / 4;
    const bool whole_quads = (w->n_in / 32) % 4 == 0;
    GemmPlan best{nullptr, 0.0};
    static const int forced = [] {  // measurements only: RMI_GEMM_SHAPE = index into the table above
        const char *e = getenv("RMI_GEMM_SHAPE");
        return e ? atoi(e) : -1;
    }();
    for (const GemmShape &g : shapes) {
        if (forced >= 0 && !single_chain && &g != &shapes[forced % kShapes]) continue;
        // groups pay off on long rows only (measured: 1024 x 3072 gains 10-15 % from 768 tokens on, 3072 x 1024 loses
        // 3-10 %: a group needs about eight quads to make up for its own first loads and the last add; four groups
        // of a 64 x 32 tile, one workgroup of eight waves a compute unit, with six quads each: 1024 x 3072 at 512
        // tokens 11.2 us against 12.7 for the k-split kernel and 17.6 for the single chain)
        if (g.ks > 1 && (single_chain || !whole_quads || n_quads % g.ks != 0 || (forced < 0 && n_quads / g.ks < (g.ks == 4 ? 6 : 8)))) continue;
        const uint64_t groups = uint64_t((w->n_out + g.tile_n - 1) / g.tile_n) * ((n_tokens + g.tile_t - 1) / g.tile_t);
        if (groups > 0x7fffffffull) continue;
        const double nb = double(w->n_in / 32) / double(g.ks);
        const uint64_t at_once = cus * uint64_t(g.per_cu);
        const uint64_t full = groups / at_once, rest = groups % at_once;
        const uint64_t per_simd = (g.waves * g.ks + 3) / 4;  // a workgroup's waves spread over the four SIMDs of its compute unit
        const double wg_kb = double(g.tile_n + g.tile_t) * double(w->n_in) * (35.0 / 32.0) * 1e-3;
        auto round_us = [&](uint64_t groups_per_cu) __attribute__((always_inline)) {
            const uint64_t wps = groups_per_cu * per_simd;
            const double step_ns = wps == 1 ? 125.0 : (wps >= 3 || g.sub >= 2) ? 90.0 : 105.0;
            const double valu = double(wps * g.sub) * nb * step_ns * 1e-3;
            const double mem = single_chain ? 0.0 : double(groups_per_cu) * wg_kb / 40.0;
            return (valu > mem ? valu : mem) + 3.5 + (g.ks > 1 ? 0.5 : 0.0);
        };
        double cost = double(full) * round_us(uint64_t(g.per_cu));
        if (rest) cost += round_us((rest + cus - 1) / cus);
        if (!best.shape || cost < best.cost_us * 0.999) best = GemmPlan{&g, cost};
    }
    return best;
}

}  // namespace

// the launch time the tile chooser expects for this product, in microseconds (a negative value: no shape fits), and
// the number of groups that split the quads in the shape it takes
bool rmi_gemm_q8_0_shape_forced() { return getenv("RMI_GEMM_SHAPE") != nullptr; }

double rmi_gemm_q8_0_cost_us(const rmi_hip_weight *w, uint32_t n_tokens, bool single_chain, uint32_t *groups) {
    if (groups) *groups = 1;
    if (n_tokens == 0 || w->n_out == 0 || w->n_in < 32) return 0.0;
    const GemmPlan plan = plan_gemm(w, n_tokens, single_chain);
    if (plan.shape && groups) *groups = plan.shape->ks;
    return plan.shape ? plan.cost_us : -1.0;
}

static int launch_planned(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y, uint32_t n_tokens,
                          uint32_t y_stride, bool single_chain, hipStream_t s) {
    if (n_tokens == 0 || w->n_out == 0) return RMI_HIP_OK;
    if (w->n_in < 32) return rmi_fail(RMI_HIP_E_INVALID, "GEMM needs at least one block per row");
    const GemmPlan plan = plan_gemm(w, n_tokens, single_chain);
    if (!plan.shape) return rmi_fail(RMI_HIP_E_INVALID, "GEMM too large for one launch");
    const bool ragged = (w->n_in / 32) % 4 != 0 || (reinterpret_cast<uintptr_t>(x_scales) & 15) != 0;
    if (ragged && plan.shape->ks > 1) return launch_planned(w, x_q8, x_scales, y, n_tokens, y_stride, true, s);  // unaligned scales
    plan.shape->launch(w, x_q8, x_scales, y, n_tokens, y_stride, ragged, s);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

// one f32 chain per output in block order: the aarch64 kernel's result bit for bit
int rmi_launch_gemm_q8_0(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                         uint32_t n_tokens, uint32_t y_stride, hipStream_t s) {
    return launch_planned(w, x_q8, x_scales, y, n_tokens, y_stride, true, s);
}

// the tiled kernel with the quads of a row split over two or four groups of waves where the chooser expects that to
// be faster: a chain per group, the groups' sums added in group order (within rounding of the single chain)
int rmi_launch_gemm_q8_0_grouped(const rmi_hip_weight *w, const int8_t *x_q8, const float *x_scales, float *y,
                                 uint32_t n_tokens, uint32_t y_stride, hipStream_t s) {
    return launch_planned(w, x_q8, x_scales, y, n_tokens, y_stride, false, s);
}
