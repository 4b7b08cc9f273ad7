// Device-side pieces of the reference's activation quantiser (src/nvfp4.c:12-130) shared by the NVFP4 kernels:
// closed-form round-to-nearest-even encoders in place of the reference's argmin scans (equality is proven on the
// host by the tests) and the quantiser of one 16-column block.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {
namespace {

// Closed-form round-to-nearest-even E4M3FN encode of a finite, non-negative
// value already clamped to 448.
__device__ __forceinline__ uint32_t e4m3_encode_positive(float m) {
    if (m < 0.015625f) return (uint32_t)__builtin_rintf(m * 512.0f);
    uint32_t bits = __float_as_uint(m);
    bits += 0x7FFFFu + ((bits >> 20) & 1u);
    return (bits >> 20) - ((127u - 7u) << 3);
}

__device__ __forceinline__ uint32_t e2m1_encode(float v) {
    const float m = __builtin_fabsf(v);
    const uint32_t code = (uint32_t)(m > 0.25f) + (uint32_t)(m >= 0.75f) + (uint32_t)(m > 1.25f) +
                          (uint32_t)(m >= 1.75f) + (uint32_t)(m > 2.5f) + (uint32_t)(m >= 3.5f) +
                          (uint32_t)(m > 5.0f);
    return code | ((__float_as_uint(v) >> 28) & 8u);
}

__device__ __forceinline__ float e2m1_decode(uint32_t code) {
    const uint32_t m = code & 7u;
    // 0, .5, 1, 1.5, 2, 3, 4, 6; magnitude zero is +0 whatever the sign bit
    const float mag = m == 0 ? 0.0f : m == 1 ? 0.5f : (1.0f + 0.5f * (float)(m & 1u)) * (float)(1u << ((m >> 1) - 1u));
    return (code & 8u) && m != 0 ? -mag : mag;
}

// One 16-element block of the reference's group-16 quantiser (nvfp4.c:82-130) for consumers that multiply codes:
// codes[0..1] receive the sixteen E2M1 codes (low nibble = even element), from_code the factor scale / g that turns
// a code value into the dequantised activation.  Returns false when an element is not finite (the reference rejects
// the call).
__device__ __forceinline__ bool fp4_quantise_block(const float (&v)[16], float g, uint32_t (&codes)[2], float &from_code) {
    float top = 0.0f;
    bool finite = true;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float m = __builtin_fabsf(v[i]);
        finite = finite && (m < __builtin_inff());           // false for inf and NaN
        if (m > top) top = m;
    }
    if (!finite) return false;
    const float sixth = top * (1.0f / 6.0f);
    float raw = g * sixth;
    if (raw > 448.0f) raw = 448.0f;
    const uint32_t scale_code = e4m3_encode_positive(raw);
    const float scale = __builtin_amdgcn_cvt_f32_fp8((int)scale_code, 0);
    const float to_code = scale == 0.0f ? 0.0f : g / scale;
    from_code = scale / g;
    codes[0] = 0u; codes[1] = 0u;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        float s = v[i] * to_code;
        if (s > 6.0f) s = 6.0f;
        if (s < -6.0f) s = -6.0f;
        codes[i >> 3] |= e2m1_encode(s) << (4 * (i & 7));
    }
    return true;
}

}  // namespace
}  // namespace mi355
