// How a wave of a GEMV kernel walks its run of the weight stream, shared by the Q8_0, Q4_0, Q4_K and Q6_K kernels.
//
// A run is a contiguous piece of a matrix's tile stream: n_units units (one octet or one super-block of one
// 8-row tile), tile after tile.  Four units are in flight per wave, in four register sets taken in turn.  Every
// load of the steady loop is unconditional and no store sits between a load and its use, so the compiler's
// s_waitcnt leaves the three younger units in flight while the oldest is multiplied; a load or a store under
// a branch in that window makes the same wait drain the whole queue (it must hold on the path that skipped the
// instruction, too).  For the same reason the results of finished tiles do not leave from inside the loop:
// they wait in registers (RmiRunResults) and are stored eight tiles at a time.
#ifndef RMI_DEVICE_RUN_RING_H
#define RMI_DEVICE_RUN_RING_H

#include <hip/hip_runtime.h>
#include <stdint.h>

template <typename Regs>
struct RmiRing {
    Regs r0, r1, r2, r3;
};

// A cursor names the next unit to load: `cur.load(regs)` issues that unit's loads, `cur.step()` moves on by
// one unit.  Its address is the same for all lanes (the lane adds a fixed offset), so a step is scalar work.
//
// Units 0..3 of the run; a run of fewer units loads its last unit again (in bounds, never used).  Call this
// before the activation is staged: the two round trips then overlap.
template <typename Regs, typename Cursor>
__device__ __forceinline__ void rmi_ring_fill(RmiRing<Regs> &ring, uint32_t n_units, Cursor &cur) {
    cur.load(ring.r0);
    if (n_units > 1) cur.step();
    cur.load(ring.r1);
    if (n_units > 2) cur.step();
    cur.load(ring.r2);
    if (n_units > 3) cur.step();
    cur.load(ring.r3);
    if (n_units > 4) cur.step();
}

// `consume(regs)` multiplies one unit (and finishes a tile after its last unit); units are consumed in
// ascending order.  On entry the cursor is where rmi_ring_fill left it: at unit 4, if the run has one.
template <typename Regs, typename Cursor, typename Consume>
__device__ __forceinline__ void rmi_ring_walk(RmiRing<Regs> &ring, uint32_t n_units, Cursor &cur, Consume consume) {
    uint32_t u = 0;
    for (; u + 8 <= n_units; u += 4) {  // units u+4 .. u+7 exist
        consume(ring.r0);
        cur.load(ring.r0);
        cur.step();
        consume(ring.r1);
        cur.load(ring.r1);
        cur.step();
        consume(ring.r2);
        cur.load(ring.r2);
        cur.step();
        consume(ring.r3);
        cur.load(ring.r3);
        cur.step();
    }
    // the ring holds units u .. u+3 (those that exist); at most three more follow, the cursor is at the first
    const uint32_t rest = n_units - u;
    if (rest > 0) consume(ring.r0);
    if (rest > 1) consume(ring.r1);
    if (rest > 2) consume(ring.r2);
    if (rest > 3) consume(ring.r3);
    if (rest > 4) {
        cur.load(ring.r0);
        if (rest > 5) {
            cur.step();
            cur.load(ring.r1);
        }
        if (rest > 6) {
            cur.step();
            cur.load(ring.r2);
        }
        consume(ring.r0);
        if (rest > 5) consume(ring.r1);
        if (rest > 6) consume(ring.r2);
    }
}

// Results of the tiles a wave has finished.  The eight lanes of a row all hold the row's sum after the
// horizontal add; lane t8 (0..7) keeps the one of tile t8 of the current group of eight tiles, per token.  A
// group leaves with one 256-byte store per token.
template <int B>
struct RmiRunResults {
    float res[B];
    uint32_t tiles_done = 0, flushed = 0;

    __device__ __forceinline__ void keep(const float (&y)[B], uint32_t t8) {
#pragma unroll
        for (int t = 0; t < B; t++) res[t] = t8 == (tiles_done & 7) ? y[t] : res[t];
        tiles_done++;
    }
    __device__ __forceinline__ bool group_full() const { return (tiles_done & 7) == 0; }
    __device__ __forceinline__ bool pending() const { return flushed < tiles_done; }
    // first_tile: index of the run's first tile in the matrix; rows outside [row_start, row_end) are not stored
    template <typename YPtr>
    __device__ __forceinline__ void flush(YPtr y, uint32_t y_stride, uint32_t first_tile, uint32_t r, uint32_t t8,
                                          uint32_t row_start, uint32_t row_end) {
        const uint32_t row = (first_tile + flushed + t8) * 8 + r;
#pragma unroll
        for (int t = 0; t < B; t++)
            if (flushed + t8 < tiles_done && row >= row_start && row < row_end) y[size_t(t) * y_stride + row] = res[t];
        flushed = tiles_done;
    }
};

#endif  // RMI_DEVICE_RUN_RING_H
