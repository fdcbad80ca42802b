// GELU-tanh value and slope, shared by the activation kernels and the fused
// bias + GELU pair.  Operation order is the reference CPU kernel's (each multiply
// / add rounds separately): backend.py:376-414 with the constants of
// backend.py:18-20.
#pragma once
#include <hip/hip_runtime.h>

namespace agrad {

constexpr float kGeluC = 0.7978845608028654f;
constexpr float kGeluA = 0.044715f;
constexpr float kGeluA3 = 0.134145f;

// z = C (x + A x^3)
__device__ __forceinline__ float gelu_inner(float x) {
    float z = x * x;
    z = z * x;
    z = z * kGeluA;
    z = x + z;
    return z * kGeluC;
}

// GELU(x) = (x (tanh z + 1)) / 2
__device__ __forceinline__ float gelu_value(float x) {
    float b = tanhf(gelu_inner(x));
    b = b + 1.0f;
    b = x * b;
    return b * 0.5f;
}

// d GELU / dx = (1 + t)/2 + (1 - t^2) * (x/2) * C (1 + A3 x^2), t = tanh z.  The
// reference forms 1 - t*t and (t + 1) from the rounded t (backend.py:398-411),
// which loses every significant bit once |t| is within a few ulp of 1; here both
// factors come from w = exp(-2|z|) with no cancellation, so the device value is
// the accurate one and differs from the CPU value by the CPU's own rounding
// noise only.
__device__ __forceinline__ float gelu_slope(float x) {
    const float z = gelu_inner(x);
    const float w = expf(-2.0f * fabsf(z));
    const float inv = 1.0f / (1.0f + w);
    const float half_one_plus_t = z >= 0.0f ? inv : w * inv;   // (1 + tanh z) / 2
    const float sech2 = (4.0f * w) * (inv * inv);              // 1 - tanh^2 z
    const float d_inner = kGeluC * (1.0f + (kGeluA3 * x) * x);
    const float a = sech2 * ((0.5f * x) * d_inner);
    return half_one_plus_t + a;
}

}  // namespace agrad
