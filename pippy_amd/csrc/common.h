// Shared helpers for the gfx950 kernels: status reporting, bf16 bit conversions, wave utilities.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/pippy_amd.h"

namespace pp {

// Thread-local message returned by pp_last_error().
char* error_buffer();

inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(PP_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return PP_OK;
}

__host__ __device__ inline bool aligned(const void* p, size_t a) {
    return (reinterpret_cast<uintptr_t>(p) % a) == 0;
}

// bf16 <-> fp32 on raw bits.  Round-to-nearest-even with NaN quieting, the rule torch uses
// (c10::BFloat16 round_to_nearest_even).
__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
typedef __bf16 pp_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float pp_f32x2_t __attribute__((ext_vector_type(2)));
// fp32 -> bf16, round-to-nearest-even, through the hardware conversion (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const pp_f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, pp_bf16x2_t));
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    return static_cast<uint16_t>(pack_bf16(f, 0.f) & 0xffffu);
}
__device__ __forceinline__ float bf16lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// Sum / max over the 64 lanes of a wave (every lane gets the result).
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

}  // namespace pp
