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

// signed 4 x int8 dot from zero (the build turns v_dot4c off, so this is one v_dot4_i32_i8 with a literal 0)
__device__ __forceinline__ int dot4_i8(int a, int b) {
    return __builtin_amdgcn_sdot4(a, b, 0, false);
}

// ((l0+l4)+(l1+l5))+((l2+l6)+(l3+l7)) of the eight lanes of a row (src/ops/dot.rs:447-456); every lane of the
// row ends up with the sum (a + b and b + a are the same bits)
__device__ __forceinline__ float hsum8_lanes(float a) {
    a = a + __shfl_xor(a, 4, 64);
    a = a + __shfl_xor(a, 1, 64);
    a = a + __shfl_xor(a, 2, 64);
    return a;
}

#endif  // RMI_DEVICE_COMMON_H
