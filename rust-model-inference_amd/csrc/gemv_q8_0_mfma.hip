// Q8_0 x Q8_0 for a small batch of tokens (1..64) on the matrix cores, weights streamed once:
//   y[t][n] = sum over blocks b, in sequence, of fma(float(dot_b(W[n], X[t])), f32(wd[n][b]) * xs[t][b], sum)
// which is the order of matmul_q8_0_vs_q8_0_neon (src/ops/kernel/q8_0/neon.rs:49-73), bit for bit, applied to
// every token as Kernel::forward_batched does (src/ops/kernel/trait_.rs:78-109).
//
// Why a second small-batch kernel: the AVX2-order GEMV (gemv_q8_0.hip) converts eight partial sums per row and
// block and is bound by the vector ALU from four tokens on; in the NEON order one int32 dot per row, block and
// token is converted, and v_mfma_i32_16x16x32_i8 delivers sixteen rows x sixteen tokens of them at once, so the
// kernel stays bound by HBM up to a few dozen tokens.
//
// A wave owns a run of consecutive tiles of one matrix, as in the GEMV, and takes them two at a time (16 rows).
// The weight bytes arrive in the GEMV tile stream's layout (lane 8r + L holds the 4-byte slice L of blocks of
// row r); the MFMA wants lane 16g + m to hold bytes 8g..8g+7 of a block of row m.  Two ds_permute per block
// (the LDS crossbar, no memory) turn one into the other: source lanes with even L send tile A's slice and
// those with odd L tile B's, then the other way round, and each destination lane sorts the two arrivals into
// low and high dword.  The activations sit in LDS in natural order, one row per token (rows 32 bytes apart from
// a multiple of 256, which spreads the 8-byte reads of a quarter wave over all banks), with their block scales.
// Lane 16g + m receives the dots of rows 4g..4g+3 of the pair for token m.  Those rows' f16 scales (64 bytes an
// octet, the same for the 16 lanes of a g) are loaded a dword a lane and shared by DPP row broadcasts.  A lane's
// four rows are neighbours in y and leave as one 16-byte store, two pairs of tiles at a time.
#include "rmi_internal.h"

#include "device_common.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef f32x4 __attribute__((address_space(1))) *gptr_f32x4_w;

constexpr uint32_t kRowPadBytes = 32;   // added to a token's row of quants in LDS
constexpr uint32_t kScalePadFloats = 4; // added to a token's row of block scales in LDS
// Results of this many pairs of tiles are kept before they are stored: a token's 32 rows then leave together and
// fill a 128-byte line of y.  (Stores that reach HBM are dear next to the weight stream: with 8 tokens they are 3 %
// of the bytes and cost 10 % of the time; 4-byte stores, one row a lane, cost 15 %.)
constexpr int kHoldPairs = 2;

__host__ __device__ inline size_t mfma_lds_bytes(uint32_t n_tokens, uint32_t n_oct) {
    return size_t(n_tokens) * (size_t(n_oct) * 256 + kRowPadBytes) +
           size_t(n_tokens) * (size_t(n_oct) * 8 + kScalePadFloats) * 4;
}

// Lane K of every sixteen lanes, to all of the sixteen (DPP row_newbcast).
template <int K>
__device__ __forceinline__ uint32_t row_bcast(uint32_t x) {
    return uint32_t(__builtin_amdgcn_update_dpp(0, int(x), 0x150 + K, 0xf, 0xf, false));
}

struct PairRegs {        // one octet of two tiles
    u32x4 qa[2], qb[2];  // [tile]: blocks 8o..8o+3 and 8o+4..8o+7, bytes 4L..4L+3 of each, of row r
    // Block scales of rows 4g..4g+3 of the pair: 64 bytes that all sixteen lanes of a g need.  Each lane loads one
    // dword of them, lane 16g + m the f16 scales of blocks 2(m&3), 2(m&3)+1 of row 4g + (m>>2), and the sixteen
    // share them by row broadcasts when they are used: one load instruction an octet instead of four, 1 register
    // instead of 16.
    uint32_t sc1;
};

// The activations of the n_tokens tokens into LDS: quants in natural order, a row per token, then the block
// scales; zeros for blocks from nb on.  Loads are unconditional (clamped); the first eight 16-byte pieces and the
// first four scales of every thread are in flight together, so that a workgroup usually stages its tokens in one
// memory round trip.
__device__ __forceinline__ void stage_tokens(uint8_t *lds_q, float *lds_s, const int8_t *x_q8, const float *x_scales,
                                             uint32_t n_tokens, uint32_t n_oct, uint32_t nb, uint32_t tid,
                                             uint32_t n_threads) {
    constexpr int kQ = 8, kS = 4;
    gptr_u4 xq = as_global<gptr_u4>(x_q8);
    gptr_f32 xs = as_global<gptr_f32>(x_scales);
    const uint32_t row_u4 = n_oct * 16, src_u4 = nb * 2, total = n_tokens * row_u4;
    const uint32_t stride_u4 = row_u4 + kRowPadBytes / 16;
    const uint32_t row_s = n_oct * 8, total_s = n_tokens * row_s, stride_s = row_s + kScalePadFloats;
    uint4 *dq = reinterpret_cast<uint4 *>(lds_q);
    u32x4 v[kQ];
    uint32_t qd[kQ];  // LDS index of the piece, ~0u for none
    bool qlive[kQ];
    float sv[kS];
    uint32_t sd[kS];
    bool slive[kS];
    // piece i = (token t, piece c of its row); from one piece of a thread to its next both move by the same
    // amounts, so one division per call does
    const uint32_t q_dt = n_threads / row_u4, q_dc = n_threads - q_dt * row_u4;
    const uint32_t s_dt = n_threads / row_s, s_dc = n_threads - s_dt * row_s;
    auto load_q = [&](uint32_t base) {
        uint32_t t = base / row_u4, c = base - t * row_u4;
#pragma unroll
        for (int j = 0; j < kQ; j++) {
            const uint32_t i = base + j * n_threads;
            qlive[j] = i < total && c < src_u4;
            qd[j] = i < total ? t * stride_u4 + c : ~0u;
            v[j] = xq[qlive[j] ? t * src_u4 + c : 0];
            c += q_dc;
            t += q_dt + (c >= row_u4 ? 1u : 0u);
            c -= c >= row_u4 ? row_u4 : 0u;
        }
    };
    auto load_s = [&](uint32_t base) {
        uint32_t t = base / row_s, c = base - t * row_s;
#pragma unroll
        for (int j = 0; j < kS; j++) {
            const uint32_t i = base + j * n_threads;
            slive[j] = i < total_s && c < nb;
            sd[j] = i < total_s ? t * stride_s + c : ~0u;
            sv[j] = xs[slive[j] ? t * nb + c : 0];
            c += s_dc;
            t += s_dt + (c >= row_s ? 1u : 0u);
            c -= c >= row_s ? row_s : 0u;
        }
    };
    // the empty asm statements keep the compiler from moving a load into the guarded store that uses it, where it
    // would wait for itself
    auto store_q = [&]() {
#pragma unroll
        for (int j = 0; j < kQ; j++) asm volatile("" : "+v"(v[j]));
#pragma unroll
        for (int j = 0; j < kQ; j++) {
            if (qd[j] != ~0u) {
                const u32x4 z = {0u, 0u, 0u, 0u};
                const u32x4 o = qlive[j] ? v[j] : z;
                dq[qd[j]] = make_uint4(o.x, o.y, o.z, o.w);
            }
        }
    };
    auto store_s = [&]() {
#pragma unroll
        for (int j = 0; j < kS; j++) asm volatile("" : "+v"(sv[j]));
#pragma unroll
        for (int j = 0; j < kS; j++)
            if (sd[j] != ~0u) lds_s[sd[j]] = slive[j] ? sv[j] : 0.0f;
    };
    load_q(tid);
    load_s(tid);
    store_q();
    store_s();
    for (uint32_t base = tid + n_threads * kQ; base < total; base += n_threads * kQ) {
        load_q(base);
        store_q();
    }
    for (uint32_t base = tid + n_threads * kS; base < total_s; base += n_threads * kS) {
        load_s(base);
        store_s();
    }
}

// TT = sixteens of tokens (1..4).  GROUPED and the run table as in gemv_q8_0_kernel; a run pairs its tiles from
// its own first tile on and may hold an odd count (the last pair then has one tile).
template <int TT, bool GROUPED>
__global__ __launch_bounds__(512) void gemv_q8_0_mfma_kernel(RmiGemvProblem single,
                                                             const RmiGemvProblem *__restrict__ list,
                                                             const uint4 *__restrict__ runs, uint32_t tiles_per_wave,
                                                             uint32_t n_tokens) {
    extern __shared__ uint4 lds[];
    const uint32_t lane = threadIdx.x & 63, r = lane >> 3, L = lane & 7, m = lane & 15, g = lane >> 4;
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
    const uint32_t n_oct = p.n_oct, run_tiles = k_end - k;
    const uint32_t n_units = ((run_tiles + 1) >> 1) * n_oct;  // one octet of one pair of tiles
    const uint32_t tile_u4 = n_oct * (kOctetBytes / 16);

    struct Cursor {
        gptr_u4 tile_a;  // the same for all lanes
        uint32_t o, pair, n_oct, run_tiles, tile_u4, lane, g;
        __device__ __forceinline__ void load(PairRegs &R) const {
            // a pair's second tile that is not part of the run is read from the first: in bounds, never stored
            gptr_u4 tile_b = 2 * pair + 1 < run_tiles ? tile_a + tile_u4 : tile_a;
            gptr_u4 qa = tile_a + n_oct * 8 + (2 * o) * 64 + lane, qb = tile_b + n_oct * 8 + (2 * o) * 64 + lane;
            R.qa[0] = __builtin_nontemporal_load(qa);
            R.qb[0] = __builtin_nontemporal_load(qa + 64);
            R.qa[1] = __builtin_nontemporal_load(qb);
            R.qb[1] = __builtin_nontemporal_load(qb + 64);
            gptr_u4 sc = (g >> 1 ? tile_b : tile_a) + o * 8 + 4 * (g & 1);
            R.sc1 = reinterpret_cast<gptr_u32>(sc)[lane & 15];
        }
        __device__ __forceinline__ void step() {
            if (++o == n_oct) {
                o = 0;
                pair++;
                tile_a += 2 * size_t(tile_u4);
            }
        }
    } cur;
    // a wave without tiles (padding of the last workgroup) reads the matrix's first tile: in bounds, unused
    cur = Cursor{as_global<gptr_u4>(p.w + size_t(p.tile0 + (n_units ? k : 0)) * n_oct * kOctetBytes), 0, 0, n_oct,
                 run_tiles, tile_u4, lane, g};
    // Two units in flight: the one being multiplied and the next.  After the run's last unit the loads read it
    // again (in bounds, unused).
    uint32_t next_unit = 0;
    auto fetch = [&](PairRegs &R) {
        if (next_unit > 0 && next_unit < n_units) cur.step();
        cur.load(R);
        next_unit++;
    };
    PairRegs R0, R1;
    fetch(R0);

    const uint32_t row_stride = n_oct * 256 + kRowPadBytes, scale_stride = n_oct * 8 + kScalePadFloats;
    uint8_t *lds_q = reinterpret_cast<uint8_t *>(lds);
    float *lds_s = reinterpret_cast<float *>(lds_q + size_t(n_tokens) * row_stride);
    stage_tokens(lds_q, lds_s, p.x_q8, p.x_scales, n_tokens, n_oct, p.n_in >> 5, threadIdx.x, blockDim.x);
    __syncthreads();
    // this lane's token of each sixteen; a lane past the last token reads token 0's row (its column of the
    // product is independent of the others and never stored)
    uint32_t q_row[TT], s_row[TT];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        const uint32_t token = tt * 16 + m < n_tokens ? tt * 16 + m : 0;
        q_row[tt] = token * row_stride + g * 8;
        s_row[tt] = token * scale_stride;
    }

    // where this lane's two slices go: even L sends tile A's to lane (row r, g' = L / 2) and odd L tile B's to
    // lane (row 8 + r, g' = L / 2); the second permute swaps the tiles
    const bool l_even = (L & 1) == 0, low_rows = m < 8;
    const int dst_a = int((r + 16 * (L >> 1)) * 4), dst_b = int((8 + r + 16 * (L >> 1)) * 4);
    const int addr1 = l_even ? dst_a : dst_b, addr2 = l_even ? dst_b : dst_a;

    float acc[TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int v = 0; v < 4; v++) acc[tt][v] = 0.0f;
    uint32_t o = 0, pair = 0;
    gptr_f32_w yp = as_global<gptr_f32_w>(p.y);
    const bool vec_ok = (reinterpret_cast<uintptr_t>(p.y) & 15) == 0 && (p.y_stride & 3) == 0;

    // finished pairs wait here (consecutive pairs of the run: rows first_row0 + 16 j) and are stored together; only
    // the run's last pair can lack its second tile
    float hold[TT][kHoldPairs][4];
    uint32_t held = 0, first_row0 = 0;
    bool last_has_b = true;
    auto flush = [&]() {
#pragma unroll
        for (int j = 0; j < kHoldPairs; j++) {
            if (uint32_t(j) < held) {
                const uint32_t row0 = first_row0 + 16 * j;
                const bool has_b = uint32_t(j) + 1 < held || last_has_b;
                const bool whole = vec_ok && row0 >= p.row_start && row0 + 4 <= p.row_end;
#pragma unroll
                for (int tt = 0; tt < TT; tt++) {
                    const uint32_t token = tt * 16 + m;
                    if (token < n_tokens && (g < 2 || has_b)) {
                        if (whole) {
                            const f32x4 out = {hold[tt][j][0], hold[tt][j][1], hold[tt][j][2], hold[tt][j][3]};
                            *reinterpret_cast<gptr_f32x4_w>(yp + size_t(token) * p.y_stride + row0) = out;
                        } else {
#pragma unroll
                            for (int v = 0; v < 4; v++)
                                if (row0 + v >= p.row_start && row0 + v < p.row_end)
                                    yp[size_t(token) * p.y_stride + row0 + v] = hold[tt][j][v];
                        }
                    }
                }
            }
        }
        held = 0;
    };
    auto consume = [&](const PairRegs &R) {
        float4 xs[TT][2];  // this lane's token's eight block scales of the octet
#pragma unroll
        for (int tt = 0; tt < TT; tt++) {
            const float4 *s4 = reinterpret_cast<const float4 *>(lds_s + s_row[tt] + o * 8);
            xs[tt][0] = s4[0];
            xs[tt][1] = s4[1];
        }
        const uint32_t wq[2][8] = {{R.qa[0].x, R.qa[0].y, R.qa[0].z, R.qa[0].w, R.qb[0].x, R.qb[0].y, R.qb[0].z, R.qb[0].w},
                                   {R.qa[1].x, R.qa[1].y, R.qa[1].z, R.qa[1].w, R.qb[1].x, R.qb[1].y, R.qb[1].z, R.qb[1].w}};
        // [row v][block pair]: lane 4v + pair of this lane's sixteen holds it
        const uint32_t scw[4][4] = {{row_bcast<0>(R.sc1), row_bcast<1>(R.sc1), row_bcast<2>(R.sc1), row_bcast<3>(R.sc1)},
                                    {row_bcast<4>(R.sc1), row_bcast<5>(R.sc1), row_bcast<6>(R.sc1), row_bcast<7>(R.sc1)},
                                    {row_bcast<8>(R.sc1), row_bcast<9>(R.sc1), row_bcast<10>(R.sc1), row_bcast<11>(R.sc1)},
                                    {row_bcast<12>(R.sc1), row_bcast<13>(R.sc1), row_bcast<14>(R.sc1), row_bcast<15>(R.sc1)}};
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const int first = int(l_even ? wq[0][b] : wq[1][b]), second = int(l_even ? wq[1][b] : wq[0][b]);
            const uint32_t p1 = uint32_t(__builtin_amdgcn_ds_permute(addr1, first));
            const uint32_t p2 = uint32_t(__builtin_amdgcn_ds_permute(addr2, second));
            const uint64_t a64 = uint64_t(low_rows ? p1 : p2) | (uint64_t(low_rows ? p2 : p1) << 32);
#pragma unroll
            for (int tt = 0; tt < TT; tt++) {
                const uint64_t b64 = *reinterpret_cast<const uint64_t *>(lds_q + q_row[tt] + (o * 8 + b) * 32);
                const v4i zero = {0, 0, 0, 0};
                const v4i d = __builtin_amdgcn_mfma_i32_16x16x32_i8(long(a64), long(b64), zero, 0, 0, 0);
                const float xsb = b < 4 ? (b == 0 ? xs[tt][0].x : b == 1 ? xs[tt][0].y : b == 2 ? xs[tt][0].z : xs[tt][0].w)
                                        : (b == 4 ? xs[tt][1].x : b == 5 ? xs[tt][1].y : b == 6 ? xs[tt][1].z : xs[tt][1].w);
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const uint32_t wd16 = (b & 1) ? scw[v][b >> 1] >> 16 : scw[v][b >> 1] & 0xffffu;
                    acc[tt][v] = __builtin_fmaf(float(d[v]), h2f_times<true>(wd16, xsb), acc[tt][v]);
                }
            }
        }
        if (++o == n_oct) {  // the pair is done: rows 4g..4g+3 of it, token m of each sixteen
            if (held == 0) first_row0 = (p.tile0 + k + 2 * pair) * kTileRows + 4 * g;
#pragma unroll
            for (int tt = 0; tt < TT; tt++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
#pragma unroll
                    for (int j = 0; j < kHoldPairs; j++)
                        if (held == uint32_t(j)) hold[tt][j][v] = acc[tt][v];
                    acc[tt][v] = 0.0f;
                }
            last_has_b = 2 * pair + 1 < run_tiles;
            held++;
            if (held == kHoldPairs) flush();
            o = 0;
            pair++;
        }
    };
    for (uint32_t u = 0; u < n_units; u += 2) {
        fetch(R1);
        consume(R0);
        fetch(R0);
        if (u + 1 < n_units) consume(R1);
    }
    if (held) flush();
}

size_t mfma_lds_limit();

template <int TT>
int launch_mfma(const RmiGemvProblem *single, const RmiGemvProblem *d_list, const uint4 *d_runs, uint32_t n_waves,
                uint32_t wpg, uint32_t tiles_per_wave, uint32_t max_n_oct, uint32_t n_tokens, hipStream_t s) {
    const size_t lds_bytes = mfma_lds_bytes(n_tokens, max_n_oct);
    if (lds_bytes > mfma_lds_limit())
        return rmi_fail(RMI_HIP_E_INVALID, "%u tokens x %u elements do not fit the LDS staging", n_tokens, max_n_oct * 256);
    const dim3 block(64 * wpg);
    if (single)
        hipLaunchKernelGGL((gemv_q8_0_mfma_kernel<TT, false>), dim3((n_waves + wpg - 1) / wpg), block, lds_bytes, s, *single,
                           d_list, d_runs, tiles_per_wave, n_tokens);
    else
        hipLaunchKernelGGL((gemv_q8_0_mfma_kernel<TT, true>), dim3(n_waves / wpg), block, lds_bytes, s, RmiGemvProblem{},
                           d_list, d_runs, tiles_per_wave, n_tokens);
    RMI_HIP_CHECK(hipGetLastError());
    return RMI_HIP_OK;
}

// more than 64 KiB of dynamic LDS has to be asked for, once, per kernel
size_t mfma_lds_limit() {
    static const size_t limit = [] {
        constexpr size_t kWant = 159 * 1024;
        const void *kernels[] = {reinterpret_cast<const void *>(gemv_q8_0_mfma_kernel<1, false>),
                                 reinterpret_cast<const void *>(gemv_q8_0_mfma_kernel<2, false>),
                                 reinterpret_cast<const void *>(gemv_q8_0_mfma_kernel<3, false>),
                                 reinterpret_cast<const void *>(gemv_q8_0_mfma_kernel<4, false>),
                                 reinterpret_cast<const void *>(gemv_q8_0_mfma_kernel<1, true>),
                                 reinterpret_cast<const void *>(gemv_q8_0_mfma_kernel<2, true>),
                                 reinterpret_cast<const void *>(gemv_q8_0_mfma_kernel<3, true>),
                                 reinterpret_cast<const void *>(gemv_q8_0_mfma_kernel<4, true>)};
        bool ok = true;
        for (const void *f : kernels)
            ok = ok && hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, int(kWant)) == hipSuccess;
        if (!ok) (void)hipGetLastError();
        return ok ? kWant : size_t(64 * 1024);
    }();
    return limit;
}

}  // namespace

bool rmi_gemv_q8_0_mfma_fits(uint32_t n_tokens, uint32_t max_n_oct) {
    return n_tokens >= 1 && n_tokens <= kMfmaMaxTokens && mfma_lds_bytes(n_tokens, max_n_oct) <= mfma_lds_limit();
}

size_t rmi_gemv_q8_0_mfma_lds_bytes(uint32_t n_tokens, uint32_t max_n_oct) {
    return mfma_lds_bytes(n_tokens, max_n_oct);
}

int rmi_launch_gemv_q8_0_mfma(const RmiGemvProblem *single, const RmiGemvProblem *d_list, const uint4 *d_runs,
                              uint32_t n_waves, uint32_t wpg, uint32_t tiles_per_wave, uint32_t max_n_oct,
                              uint32_t n_tokens, hipStream_t s) {
    if (n_waves == 0) return RMI_HIP_OK;
    if (wpg == 0 || wpg > 8) return rmi_fail(RMI_HIP_E_INVALID, "%u waves per workgroup", wpg);
    if (single && tiles_per_wave == 0) return rmi_fail(RMI_HIP_E_INVALID, "runs of no tiles");
    switch ((n_tokens + 15) / 16) {
        case 1: return launch_mfma<1>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, n_tokens, s);
        case 2: return launch_mfma<2>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, n_tokens, s);
        case 3: return launch_mfma<3>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, n_tokens, s);
        case 4: return launch_mfma<4>(single, d_list, d_runs, n_waves, wpg, tiles_per_wave, max_n_oct, n_tokens, s);
        default: return rmi_fail(RMI_HIP_E_INVALID, "the small-batch kernel takes 1..%u tokens, got %u", kMfmaMaxTokens, n_tokens);
    }
}
