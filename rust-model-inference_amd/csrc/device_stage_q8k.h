// Staging of a Q8_K activation in LDS for the K-quant GEMVs (Q4_K, Q6_K), shared by both kernels.
// Per token and super-block 76 dwords: 64 dwords of quants ordered [T][g] (dword T*8+g = elements 32g+4T..),
// 8 dwords derived from bsums, 1 dword d (+3 pad).  The loads are 16 bytes wide and UNROLL of them go out
// before the first LDS write waits: a load per dword inside the loop costs one memory round trip per iteration.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

constexpr uint32_t kQ8kSbDwords = 76;

// PAIR_SUMS: dword 64+j = bsums[2j] + bsums[2j+1] wrapped to int16 (what _mm_hadd_epi16 yields), sign-extended;
// otherwise dword 64+j = the raw pair bsums[2j] | bsums[2j+1] << 16.
template <bool PAIR_SUMS, int UNROLL>
__device__ __forceinline__ void rmi_stage_q8k_token(uint32_t *dst, const int8_t *qs, const int16_t *bsums, const float *d,
                                                    uint32_t n_sb, uint32_t tid, uint32_t n_threads) {
    typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
    typedef const u32x4_t __attribute__((address_space(1))) *gp_u4;
    typedef const uint32_t __attribute__((address_space(1))) *gp_u32;
    typedef const float __attribute__((address_space(1))) *gp_f32;
    gp_u4 xq = (gp_u4)(uintptr_t)qs;
    gp_u32 bs = (gp_u32)(uintptr_t)bsums;
    gp_f32 dp = (gp_f32)(uintptr_t)d;
    const uint32_t n_u4 = n_sb * 16;
    // the first bsums pair and d of this thread travel with the quants
    const uint32_t b0 = tid < n_sb * 8 ? tid : 0, d0 = tid < n_sb ? tid : 0;
    const uint32_t bv0 = bs[b0];
    const float dv0 = dp[d0];
    for (uint32_t base = tid; base < n_u4; base += n_threads * UNROLL) {
        u32x4_t v[UNROLL];
#pragma unroll
        for (int j = 0; j < UNROLL; j++) {
            const uint32_t i = base + j * n_threads;
            v[j] = xq[i < n_u4 ? i : n_u4 - 1];
        }
#pragma unroll
        for (int j = 0; j < UNROLL; j++) {
            const uint32_t i = base + j * n_threads;
            if (i < n_u4) {
                // source dwords e = 4*(i%16) .. +3 of super-block i/16: g = e/8, T = e%8
                const uint32_t sb = i >> 4, e = (i & 15) * 4;
                uint32_t *p = dst + sb * kQ8kSbDwords + (e & 7) * 8 + (e >> 3);
                p[0] = v[j].x;
                p[8] = v[j].y;
                p[16] = v[j].z;
                p[24] = v[j].w;
            }
        }
    }
    auto put_bs = [&](uint32_t i, uint32_t raw) {
        uint32_t val = raw;
        if (PAIR_SUMS) val = uint32_t(int32_t(int16_t(int16_t(raw & 0xffffu) + int16_t(raw >> 16))));
        dst[(i >> 3) * kQ8kSbDwords + 64 + (i & 7)] = val;
    };
    if (tid < n_sb * 8) put_bs(tid, bv0);
    for (uint32_t i = tid + n_threads; i < n_sb * 8; i += n_threads) put_bs(i, bs[i]);
    if (tid < n_sb) dst[tid * kQ8kSbDwords + 72] = __float_as_uint(dv0);
    for (uint32_t i = tid + n_threads; i < n_sb; i += n_threads) dst[i * kQ8kSbDwords + 72] = __float_as_uint(dp[i]);
}
