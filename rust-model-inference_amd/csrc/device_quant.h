// Device-side pieces shared by the activation quantizer and the kernels that
// quantize their own output (norm, attention, SiLU): quantize_q8_0_into
// (src/ops/quant/q8_0.rs:49-71 scalar, :176-230 AVX2, :75-164 NEON) for 8 consecutive lanes
// that hold one 32-element block, 4 consecutive elements each.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/rmi_hip.h"
#include "device_common.h"

// Returns the four quants packed little-endian; *scale is f32(f16(amax/127)), valid in all 8 lanes.
// The 8 lanes of a block must be consecutive lanes of one wave, aligned to 8, and all active.
__device__ __forceinline__ uint32_t rmi_quantize_block8(float4 v, int rounding, float *scale) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = max8_lanes(amax);
    if (rounding == RMI_HIP_ROUND_NEON) {
        // the aarch64 host: vmaxq / vmaxvq hand a NaN on (fmaxf drops it), scale = amax / 127 with no zero test,
        // 1 / scale, clamp to [-127, 127] before and after vcvtnq (nearest, ties to even; NaN gives 0)
        const bool nan_here = v.x != v.x || v.y != v.y || v.z != v.z || v.w != v.w;
        if (max8_lanes(nan_here ? 1.0f : 0.0f) != 0.0f) amax = __builtin_nanf("");
        const float d = amax / 127.0f;
        const float inv = d > 0.0f ? 1.0f / d : 0.0f;
        const float t[4] = {v.x * inv, v.y * inv, v.z * inv, v.w * inv};
        uint32_t packed = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int q = t[k] != t[k] ? 0 : int(rintf(fminf(fmaxf(t[k], -127.0f), 127.0f)));
            packed |= uint32_t(q & 0xff) << (8 * k);
        }
        *scale = float(_Float16(d));
        return packed;
    }
    const float d = amax == 0.0f ? 0.0f : amax / 127.0f;
    float r0, r1, r2, r3;
    if (rounding == RMI_HIP_ROUND_TIES_EVEN) {
        const float id = amax == 0.0f ? 0.0f : 127.0f / amax;
        r0 = rintf(v.x * id);
        r1 = rintf(v.y * id);
        r2 = rintf(v.z * id);
        r3 = rintf(v.w * id);
    } else {
        const float inv = d == 0.0f ? 0.0f : 1.0f / d;
        r0 = roundf(v.x * inv);
        r1 = roundf(v.y * inv);
        r2 = roundf(v.z * inv);
        r3 = roundf(v.w * inv);
    }
    // NaN: the AVX2 clamp max_ps(r,-128) yields -128, Rust's clamp + `as i8` yields 0
    const bool even = rounding == RMI_HIP_ROUND_TIES_EVEN;
    const int i0 = (r0 != r0 && !even) ? 0 : int(fminf(fmaxf(r0, -128.0f), 127.0f));
    const int i1 = (r1 != r1 && !even) ? 0 : int(fminf(fmaxf(r1, -128.0f), 127.0f));
    const int i2 = (r2 != r2 && !even) ? 0 : int(fminf(fmaxf(r2, -128.0f), 127.0f));
    const int i3 = (r3 != r3 && !even) ? 0 : int(fminf(fmaxf(r3, -128.0f), 127.0f));
    *scale = float(_Float16(d));
    return uint32_t(i0 & 0xff) | (uint32_t(i1 & 0xff) << 8) | (uint32_t(i2 & 0xff) << 16) | (uint32_t(i3 & 0xff) << 24);
}
