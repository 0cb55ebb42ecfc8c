// f32 exponential with the bits of the platform libm's expf, which is what the
// reference's f32::exp (softmax, src/ops/attention.rs:28-38; SiLU,
// src/ops/activation/mod.rs:137-151) resolves to on x86-64 Linux.  glibc's
// algorithm (2.27 and later, the FMA build that AVX2 hosts select): reduce in
// f64 to x*32/ln2 = k + r, 2^(k/32) from a 32-entry table, a cubic in r, with
// the reduction and the three polynomial steps each one fused multiply-add.
// The same formula in plain C equals the host's expf on all 2^32 inputs; the
// tests hold the C twin to the host libm and this function to the twin.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

// 2^(i/32) as f64 bits, minus i << 47 so that adding k << 47 yields 2^(k/32)
__device__ static constexpr uint64_t kRmiExp2fTab[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull,
};

// `tab` is kRmiExp2fTab or a copy of it in LDS (a kernel that calls this in a latency-bound phase copies it first)
__device__ __forceinline__ float rmi_expf_tab(float x, const uint64_t *tab) {
    const uint32_t ux = __float_as_uint(x);
    const uint32_t abstop = (ux >> 20) & 0x7ff;
    if (abstop >= (0x42b00000u >> 20)) {  // |x| >= 88 or NaN
        if (ux == 0xff800000u) return 0.0f;
        if (abstop >= (0x7f800000u >> 20)) return x + x;
        if (x > 0x1.62e42ep6f) return __uint_as_float(0x7f800000u);  // overflow
        if (x < -0x1.9fe368p6f) return 0.0f;                         // underflow
    }
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32, shift = 0x1.8p+52;
    const double c0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32, c1 = 0x1.ebfce50fac4f3p-3 / 32 / 32,
                 c2 = 0x1.62e42ff0c52d6p-1 / 32;
    const double xd = double(x);
    const double z = inv_ln2_n * xd;
    double kd = z + shift;
    const uint64_t ki = uint64_t(__double_as_longlong(kd));
    kd -= shift;
    const double r = __builtin_fma(inv_ln2_n, xd, -kd);
    const uint64_t t = tab[ki & 31] + (ki << 47);
    const double s = __longlong_as_double((long long)t);
    const double p = __builtin_fma(c0, r, c1);
    const double r2 = r * r;
    double y = __builtin_fma(c2, r, 1.0);
    y = __builtin_fma(p, r2, y);
    y = y * s;
    return float(y);
}

__device__ __forceinline__ float rmi_expf(float x) { return rmi_expf_tab(x, kRmiExp2fTab); }

// f32 -> f16 of a value that has already been rounded to f32.  The empty asm keeps the compiler from folding
// a preceding fma into v_fma_mixlo_f16, which rounds the exact result once; the reference rounds twice.
__device__ __forceinline__ uint16_t rmi_f2h(float v) {
    asm volatile("" : "+v"(v));
    return __builtin_bit_cast(uint16_t, _Float16(v));
}
