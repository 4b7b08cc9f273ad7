// Device restatement of SALT's deterministic transcendentals.
//
// The engine's softmax weights and GELU gate go through its own exp/tanh
// (reference src/bitmath.c:44-63, 144-153; models/gemma4-26b-a4b/src/gemma4.c:80-83)
// so that every platform produces the same bits.  The same operation sequence
// is written here for gfx950: fp64 range reduction, a degree-8 fp32 Horner
// chain with separately rounded multiplies and adds, and an exact ldexp.
// Compile with -ffp-contract=off: a fused multiply-add anywhere in this file
// changes results.
#pragma once

#include <hip/hip_runtime.h>

namespace mi355 {

__device__ __forceinline__ float det_expf(float x) {
    if (x != x) return x;
    if (x > 88.722839f) return 3.402823466e+38f;
    if (x < -87.336548f) return 0.0f;
    const double n = round((double)x * 1.442695040888963407359924681001892137426645954152985934135449406931);
    const double r = (double)x - n * 0.693147180559945309417232121458176568075500134360255254120680009;
    const float rf = (float)r;
    float p = 2.48015873015873e-05f;
    p = p * rf; p = p + 1.98412698412698e-04f;
    p = p * rf; p = p + 1.38888888888889e-03f;
    p = p * rf; p = p + 8.33333333333333e-03f;
    p = p * rf; p = p + 4.16666666666667e-02f;
    p = p * rf; p = p + 1.66666666666667e-01f;
    p = p * rf; p = p + 5.0e-01f;
    p = p * rf; p = p + 1.0f;
    p = p * rf; p = p + 1.0f;
    return ldexpf(p, (int)n);
}

__device__ __forceinline__ float det_tanhf(float x) {
    if (x != x) return x;
    if (x >= 10.0f) return 1.0f;
    if (x <= -10.0f) return -1.0f;
    const float m = x < 0.0f ? -x : x;
    const float e = det_expf(2.0f * m);
    const float t = (e - 1.0f) / (e + 1.0f);
    return x < 0.0f ? -t : t;
}

// gelu_tanh(x) = (0.5*x) * (1 + tanh(k*(x + ((0.044715*x)*x)*x)))
__device__ __forceinline__ float det_gelu_tanh(float x) {
    const float k = 0.7978845608028654f;
    float cube = 0.044715f * x;
    cube = cube * x;
    cube = cube * x;
    const float inner = x + cube;
    const float t = det_tanhf(k * inner);
    const float half = 0.5f * x;
    return half * (1.0f + t);
}

}  // namespace mi355
