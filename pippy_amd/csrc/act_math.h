// GELU (exact-erf and tanh forms) and their derivatives, shared by the GEMM epilogues and the
// stand-alone activation-gradient kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

namespace pp {

// The exact (erf) form of GELU through the complementary error function of |x| / sqrt(2) in the rational-
// exponential form of Abramowitz & Stegun 7.1.26,
//   erfc(u) = (a1 t + a2 t^2 + a3 t^3 + a4 t^4 + a5 t^5) e^(-u^2),  t = 1 / (1 + p u),  u >= 0,
// whose absolute error is below 1.5e-7 (far below half a unit of bf16 at every magnitude the product with
// x can have), with one hardware exp2 and one reciprocal instead of the library's erff.  The negative side
// uses erfc itself, 0.5 x erfc(u), not 1 - (1 - erfc(u)): small values of GELU keep their relative accuracy.
struct ErfcParts {
    float q;  // erfc(|x| / sqrt(2))
    float e;  // e^(-x^2 / 2)
};
__device__ __forceinline__ ErfcParts erfc_half_square(float x) {
    const float u = fabsf(x) * 0.70710678118654752440f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, u, 1.0f));
    const float e = __builtin_amdgcn_exp2f(-1.44269504088896340736f * u * u);
    const float poly = t * fmaf(t, fmaf(t, fmaf(t, fmaf(t, 1.061405429f, -1.453152027f), 1.421413741f),
                                        -0.284496736f), 0.254829592f);
    return {poly * e, e};
}
__device__ __forceinline__ float gelu_erf(float x) {
    const float q = erfc_half_square(x).q;
    return x >= 0.f ? x * fmaf(-0.5f, q, 1.0f) : 0.5f * x * q;
}
// The tanh form of GELU written through the logistic function: with u = k (x + c x^3),
//   0.5 x (1 + tanh(u)) = x * s,   s = 1 / (1 + e^(-2u)),
// so one hardware exp2 and one reciprocal do the transcendental work.  e^(-2u) = inf gives s = 0
// and e^(-2u) = 0 gives s = 1 exactly; the absolute error of s is a few 1e-8.
constexpr float kGeluK = 0.79788456080286535588f, kGeluC = 0.044715f;
constexpr float kGeluA = -2.0f * 1.44269504088896340736f * kGeluK;  // exponent of 2 per unit of x
constexpr float kGeluB = kGeluA * kGeluC;                          // ... per unit of x^3
__device__ __forceinline__ float gelu_tanh(float x) {
    const float x2 = x * x;
    const float e = __builtin_amdgcn_exp2f(x * fmaf(x2, kGeluB, kGeluA));
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}
// d/dx [x Phi(x)] = Phi(x) + x phi(x), with the same two pieces: Phi from erfc, phi from its exponential
__device__ __forceinline__ float dgelu_erf(float x) {
    const ErfcParts p = erfc_half_square(x);
    const float cdf = x >= 0.f ? fmaf(-0.5f, p.q, 1.0f) : 0.5f * p.q;
    return fmaf(x, 0.39894228040143267794f * p.e, cdf);
}
// d/dx [x s] = s + x s (1 - s) 2 u',  u' = k (1 + 3 c x^2).
__device__ __forceinline__ float dgelu_tanh(float x) {
    const float x2 = x * x;
    const float e = __builtin_amdgcn_exp2f(x * fmaf(x2, kGeluB, kGeluA));
    const float s = __builtin_amdgcn_rcpf(1.0f + e);
    const float du2 = fmaf(x2, 6.0f * kGeluK * kGeluC, 2.0f * kGeluK);
    return s * fmaf(x * du2, 1.0f - s, 1.0f);
}

// logistic function through the hardware exp2 and reciprocal
__device__ __forceinline__ float sigmoid_fast(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896340736f * x));
}
// SwiGLU on values already rounded to the storage type: h = silu(g) u, and its two gradients
// dg = dh u silu'(g), du = dh silu(g) with silu'(g) = s (1 + g (1 - s)), s = sigmoid(g).  The stand-alone
// kernels and the GEMM epilogues share these, so that both leave the same bits.
__device__ __forceinline__ float swiglu_value(float g, float u) { return g * sigmoid_fast(g) * u; }
__device__ __forceinline__ void swiglu_grads(float g, float u, float dh, float* dg, float* du) {
    const float s = sigmoid_fast(g);
    *dg = dh * u * (s * fmaf(g, 1.0f - s, 1.0f));
    *du = dh * (g * s);
}

}  // namespace pp
