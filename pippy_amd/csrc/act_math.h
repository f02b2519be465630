// GELU (exact-erf and tanh forms) and their derivatives, shared by the GEMM epilogues and the
// stand-alone activation-gradient kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

namespace pp {

__device__ __forceinline__ float gelu_erf(float x) {
    return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
// tanh through the hardware exp2 and reciprocal: 1 - 2 / (e^(2u) + 1).  The absolute error is a few
// 1e-7 everywhere (e^(2u) = inf gives exactly 1, e^(2u) = 0 exactly -1), which is what the GELU
// forms below need: they multiply tanh by values of order one.
__device__ __forceinline__ float fast_tanh(float u) {
    const float e = __builtin_amdgcn_exp2f(u * 2.88539008177792681472f);
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}
__device__ __forceinline__ float gelu_tanh(float x) {
    const float u = 0.79788456080286535588f * (x + 0.044715f * x * x * x);
    return 0.5f * x * (1.0f + fast_tanh(u));
}
__device__ __forceinline__ float dgelu_erf(float x) {
    const float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752440f));
    const float pdf = 0.39894228040143267794f * __expf(-0.5f * x * x);
    return cdf + x * pdf;
}
__device__ __forceinline__ float dgelu_tanh(float x) {
    const float k = 0.79788456080286535588f, c = 0.044715f;
    const float u = k * (x + c * x * x * x);
    const float t = fast_tanh(u);
    return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * k * (1.0f + 3.0f * c * x * x);
}

}  // namespace pp
