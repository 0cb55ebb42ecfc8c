// Small device helpers every kernel file uses: f16 bits -> f32, the 4 x int8 dot, the horizontal add of the
// reference's hsum_ps over the eight lanes of a row, and pointer types that say "HBM" to the compiler.
#ifndef RMI_DEVICE_COMMON_H
#define RMI_DEVICE_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// Pointers that arrive inside a struct are generic; these casts tell the compiler they are HBM addresses, so
// that it emits global_load / global_store.
typedef const u32x4 __attribute__((address_space(1))) *gptr_u4;
typedef const u32x2 __attribute__((address_space(1))) *gptr_u2;
typedef const uint32_t __attribute__((address_space(1))) *gptr_u32;
typedef const uint16_t __attribute__((address_space(1))) *gptr_u16;
typedef const int16_t __attribute__((address_space(1))) *gptr_i16;
typedef const float __attribute__((address_space(1))) *gptr_f32;
typedef float __attribute__((address_space(1))) *gptr_f32_w;
template <typename T, typename U>
__device__ __forceinline__ T as_global(U *p) {
    return (T)(uintptr_t)p;
}

__device__ __forceinline__ float h2f(uint32_t bits16) {
    return float(__builtin_bit_cast(_Float16, uint16_t(bits16)));
}

// f32(h) * x with one rounding, h an f16 sitting in either half of a 32-bit register.  MIX: written as
// fma(h, x, -0.0), which is the product in every case (signed zeros included), with the -0.0 opaque to the
// compiler, so that it becomes one v_fma_mix_f32 that reads the f16 half in place; otherwise a conversion and a
// multiply.  The mixed form saves the shift, mask and conversion where they are not shared by several tokens.
template <bool MIX>
__device__ __forceinline__ float h2f_times(uint32_t bits16, float x) {
    if (MIX) {
        float neg_zero = -0.0f;
        asm("" : "+v"(neg_zero));  // opaque, or the fma is folded back into a multiply
        return __builtin_fmaf(h2f(bits16), x, neg_zero);
    }
    return h2f(bits16) * x;
}

// ---- which tile of a GEMM a workgroup takes.  Workgroups are handed to the 8 XCDs round-robin, each XCD with its
// own L2, so the tiles are renumbered per XCD.  split_n = 0: an XCD's workgroups are consecutive tiles, running
// fastest along the smaller operand; every XCD then fetches that operand whole and its own eighth of the larger one.
// split_n = 2 or 4 (the tile grid divides evenly): the XCDs form a split_n x (8 / split_n) grid over the tile grid,
// so every XCD fetches 1 / split_n of the weights and split_n / 8 of the tokens.
__device__ __forceinline__ void rmi_gemm_tile_of(uint32_t lin, uint32_t grid_n, uint32_t grid_t, uint32_t t_fastest,
                                                 uint32_t split_n, uint32_t &n_tile, uint32_t &t_tile) {
    const uint32_t xcd = lin & 7, slot = lin >> 3;
    if (split_n == 0) {
        const uint32_t n_groups = grid_n * grid_t;
        const uint32_t tile_id = xcd * (n_groups >> 3) + (xcd < (n_groups & 7) ? xcd : (n_groups & 7)) + slot;
        n_tile = t_fastest ? tile_id / grid_t : tile_id % grid_n;
        t_tile = t_fastest ? tile_id % grid_t : tile_id / grid_n;
    } else {
        const uint32_t sub_n = grid_n / split_n, sub_t = grid_t / (8 / split_n);
        n_tile = (xcd % split_n) * sub_n + (t_fastest ? slot / sub_t : slot % sub_n);
        t_tile = (xcd / split_n) * sub_t + (t_fastest ? slot % sub_t : slot / sub_n);
    }
}

// Between LDS accesses by which the lanes of ONE wave hand values to each other: every lane arrives, and the compiler
// moves no memory access across (the barrier emits no instruction; it is a point in the program that accesses stay on
// their side of).  The hardware carries a wave's LDS instructions out in order, which is all the hand-over needs; but
// to the compiler lanes that talk through memory without this are a race, and it has been seen to move one lane
// group's later writes in front of another's reads.  (Fences of wavefront scope around it would do the same and
// wait for every global load in flight as well: 7 % on a kernel that prefetches across the point.)
__device__ __forceinline__ void rmi_wave_lds_fence() { __builtin_amdgcn_wave_barrier(); }

// signed 4 x int8 dot from zero (the build turns v_dot4c off, so this is one v_dot4_i32_i8 with a literal 0)
__device__ __forceinline__ int dot4_i8(int a, int b) {
    return __builtin_amdgcn_sdot4(a, b, 0, false);
}

// ---- values of other lanes without an address register: DPP where the pattern exists, else the LDS crossbar
// with a constant pattern (ds_swizzle).  All 64 lanes must be active wherever these are used.
constexpr int kDppQuadXor1 = 1 | (0 << 2) | (3 << 4) | (2 << 6);  // quad_perm [1,0,3,2]: lane ^ 1
constexpr int kDppQuadXor2 = 2 | (3 << 2) | (0 << 4) | (1 << 6);  // quad_perm [2,3,0,1]: lane ^ 2
constexpr int kDppRowHalfMirror = 0x141;                          // lane i <-> 7 - i of each 8 lanes
constexpr int kDppRowMirror = 0x140;                              // lane i <-> 15 - i of each 16 lanes
constexpr int kDppRowBcast15 = 0x142;                             // lane 15 of a row to the whole next row
constexpr int kDppRowBcast31 = 0x143;                             // lane 31 to rows 2 and 3
constexpr int kSwizzleFirstOf8 = 0x18;                            // bit-mask mode: lane & ~7

template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {  // rows outside ROW_MASK read 0
    return uint32_t(__builtin_amdgcn_update_dpp(0, int(v), CTRL, ROW_MASK, 0xf, ROW_MASK == 0xf));
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(float, dpp_u32<CTRL, ROW_MASK>(__builtin_bit_cast(uint32_t, v)));
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ double dpp_f64(double v) {
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const uint64_t lo = dpp_u32<CTRL, ROW_MASK>(uint32_t(b)), hi = dpp_u32<CTRL, ROW_MASK>(uint32_t(b >> 32));
    return __builtin_bit_cast(double, lo | (hi << 32));
}

// The value of lane ^ 4 without the LDS crossbar: lanes 0..3 and 8..11 of a row of sixteen (banks 0 and 2) read four
// lanes up (row_shl:4), the others four lanes down (row_shr:4); two vector moves instead of a ds_swizzle, whose
// round trip a lone wave waits out.
constexpr int kDppRowShl4 = 0x104, kDppRowShr4 = 0x114;
__device__ __forceinline__ float dpp_xor4_f32(float v) {
    const int b = __builtin_bit_cast(int, v);
    int r = __builtin_amdgcn_update_dpp(0, b, kDppRowShl4, 0xf, 0x5, false);
    r = __builtin_amdgcn_update_dpp(r, b, kDppRowShr4, 0xf, 0xa, false);
    return __builtin_bit_cast(float, r);
}

// ((l0+l4)+(l1+l5))+((l2+l6)+(l3+l7)) of the eight lanes of a row (src/ops/dot.rs:447-456); every lane of the
// row ends up with the sum (a + b and b + a are the same bits).
__device__ __forceinline__ float hsum8_lanes(float a) {
    a = a + dpp_xor4_f32(a);
    a = a + dpp_f32<kDppQuadXor1>(a);
    a = a + dpp_f32<kDppQuadXor2>(a);
    return a;
}

// the largest of the eight lanes' values, in all eight
__device__ __forceinline__ float max8_lanes(float a) {
    a = fmaxf(a, dpp_f32<kDppQuadXor1>(a));
    a = fmaxf(a, dpp_f32<kDppQuadXor2>(a));
    return fmaxf(a, dpp_f32<kDppRowHalfMirror>(a));
}

// Sum of the wave's 64 values, the same in every lane (it comes back through a scalar register): quads, halves
// of eight, rows of sixteen, then row to row; the total forms in lane 63.  For f64 sums of exact terms, where
// the order of the additions is free.
__device__ __forceinline__ double wave_sum_f64(double v) {
    v += dpp_f64<kDppQuadXor1>(v);
    v += dpp_f64<kDppQuadXor2>(v);
    v += dpp_f64<kDppRowHalfMirror>(v);
    v += dpp_f64<kDppRowMirror>(v);
    v += dpp_f64<kDppRowBcast15, 0xa>(v);
    v += dpp_f64<kDppRowBcast31, 0xc>(v);
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    const uint64_t lo = uint32_t(__builtin_amdgcn_readlane(int(uint32_t(b)), 63));
    const uint64_t hi = uint32_t(__builtin_amdgcn_readlane(int(uint32_t(b >> 32)), 63));
    return __builtin_bit_cast(double, lo | (hi << 32));
}

// Largest of the wave's 64 values, the same in every lane (rows a broadcast does not write keep their own value).
__device__ __forceinline__ float wave_max_f32(float v) {
    v = fmaxf(v, dpp_f32<kDppQuadXor1>(v));
    v = fmaxf(v, dpp_f32<kDppQuadXor2>(v));
    v = fmaxf(v, dpp_f32<kDppRowHalfMirror>(v));
    v = fmaxf(v, dpp_f32<kDppRowMirror>(v));
    // row to row with the old value kept where the broadcast does not write
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v),
                                                                       kDppRowBcast15, 0xa, 0xf, false)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v),
                                                                       kDppRowBcast31, 0xc, 0xf, false)));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

#endif  // RMI_DEVICE_COMMON_H
