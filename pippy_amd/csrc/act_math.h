// GELU (exact-erf and tanh forms) and their derivatives, shared by the GEMM epilogues and the
// stand-alone activation-gradient kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

namespace pp {

__device__ __forceinline__ float gelu_erf(float x) {
    return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
__device__ __forceinline__ float gelu_tanh(float x) {
    const float u = 0.79788456080286535588f * (x + 0.044715f * x * x * x);
    return 0.5f * x * (1.0f + tanhf(u));
}
__device__ __forceinline__ float dgelu_erf(float x) {
    const float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752440f));
    const float pdf = 0.39894228040143267794f * __expf(-0.5f * x * x);
    return cdf + x * pdf;
}
__device__ __forceinline__ float dgelu_tanh(float x) {
    const float k = 0.79788456080286535588f, c = 0.044715f;
    const float u = k * (x + c * x * x * x);
    const float t = tanhf(u);
    return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * k * (1.0f + 3.0f * c * x * x);
}

}  // namespace pp
