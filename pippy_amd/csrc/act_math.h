// GELU (exact-erf and tanh forms) and their derivatives, shared by the GEMM epilogues and the
// stand-alone activation-gradient kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

namespace pp {

__device__ __forceinline__ float gelu_erf(float x) {
    return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
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
__device__ __forceinline__ float dgelu_erf(float x) {
    const float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752440f));
    const float pdf = 0.39894228040143267794f * __expf(-0.5f * x * x);
    return cdf + x * pdf;
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
