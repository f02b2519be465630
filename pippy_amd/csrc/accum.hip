// fp32 gradient accumulation across microbatches (HBM-bound, bit-exact).
//   acc[i] = init ? (float)g[i] : acc[i] + (float)g[i]
// One IEEE fp32 add per element, so a sequence of calls in microbatch order reproduces
// torch `acc.add_(g.float())` bit for bit.  Traffic per element: 2 B (bf16 g) + 4 B read +
// 4 B write of acc = 10 B (6 B when init).
#include "common.h"

namespace pp {

constexpr int kAccThreads = 256;
constexpr int kAccUnroll = 2;  // 16-byte bf16 chunks per thread

template <bool INIT>
__global__ __launch_bounds__(kAccThreads) void accum_bf16_kernel(float* __restrict__ acc,
                                                                  const uint16_t* __restrict__ g,
                                                                  int64_t n8) {
    // n8 = number of 8-element groups; all pointers 16-byte aligned
    const int64_t base = ((int64_t)blockIdx.x * kAccUnroll) * kAccThreads + threadIdx.x;
    uint4 gv[kAccUnroll];
    float4 a0[kAccUnroll], a1[kAccUnroll];
#pragma unroll
    for (int u = 0; u < kAccUnroll; ++u) {
        const int64_t i = base + (int64_t)u * kAccThreads;
        if (i < n8) {
            gv[u] = reinterpret_cast<const uint4*>(g)[i];
            if (!INIT) {
                a0[u] = reinterpret_cast<const float4*>(acc)[2 * i];
                a1[u] = reinterpret_cast<const float4*>(acc)[2 * i + 1];
            }
        }
    }
#pragma unroll
    for (int u = 0; u < kAccUnroll; ++u) {
        const int64_t i = base + (int64_t)u * kAccThreads;
        if (i < n8) {
            float4 r0, r1;
            if (INIT) {
                // -0.0f is the exact identity of IEEE addition, so init is a pure conversion
                r0 = make_float4(-0.f, -0.f, -0.f, -0.f);
                r1 = r0;
            } else {
                r0 = a0[u];
                r1 = a1[u];
            }
            r0.x += bf16lo(gv[u].x); r0.y += bf16hi(gv[u].x);
            r0.z += bf16lo(gv[u].y); r0.w += bf16hi(gv[u].y);
            r1.x += bf16lo(gv[u].z); r1.y += bf16hi(gv[u].z);
            r1.z += bf16lo(gv[u].w); r1.w += bf16hi(gv[u].w);
            reinterpret_cast<float4*>(acc)[2 * i] = r0;
            reinterpret_cast<float4*>(acc)[2 * i + 1] = r1;
        }
    }
}

template <bool INIT>
__global__ __launch_bounds__(kAccThreads) void accum_bf16_tail_kernel(float* acc, const uint16_t* g,
                                                                       int64_t begin, int64_t n) {
    const int64_t i = begin + (int64_t)blockIdx.x * kAccThreads + threadIdx.x;
    if (i < n) acc[i] = (INIT ? -0.f : acc[i]) + bf16_to_f32(g[i]);
}

template <bool INIT>
__global__ __launch_bounds__(kAccThreads) void accum_f32_kernel(float* __restrict__ acc,
                                                                 const float* __restrict__ g,
                                                                 int64_t n4) {
    const int64_t base = ((int64_t)blockIdx.x * kAccUnroll) * kAccThreads + threadIdx.x;
    float4 gv[kAccUnroll], av[kAccUnroll];
#pragma unroll
    for (int u = 0; u < kAccUnroll; ++u) {
        const int64_t i = base + (int64_t)u * kAccThreads;
        if (i < n4) {
            gv[u] = reinterpret_cast<const float4*>(g)[i];
            if (!INIT) av[u] = reinterpret_cast<const float4*>(acc)[i];
        }
    }
#pragma unroll
    for (int u = 0; u < kAccUnroll; ++u) {
        const int64_t i = base + (int64_t)u * kAccThreads;
        if (i < n4) {
            float4 r = INIT ? make_float4(-0.f, -0.f, -0.f, -0.f) : av[u];
            r.x += gv[u].x; r.y += gv[u].y; r.z += gv[u].z; r.w += gv[u].w;
            reinterpret_cast<float4*>(acc)[i] = r;
        }
    }
}

template <bool INIT>
__global__ __launch_bounds__(kAccThreads) void accum_f32_tail_kernel(float* acc, const float* g,
                                                                      int64_t begin, int64_t n) {
    const int64_t i = begin + (int64_t)blockIdx.x * kAccThreads + threadIdx.x;
    if (i < n) acc[i] = (INIT ? -0.f : acc[i]) + g[i];
}

__global__ __launch_bounds__(256) void fill_kernel(uint4* dst, uint32_t w, int64_t n16) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) dst[i] = make_uint4(w, w, w, w);
}
__global__ __launch_bounds__(256) void fill_tail_kernel(uint8_t* dst, uint8_t v, int64_t begin,
                                                        int64_t n) {
    const int64_t i = begin + (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = v;
}

}  // namespace pp

using namespace pp;

extern "C" int pp_grad_accum_f32_bf16(float* acc, const uint16_t* g, int64_t n, int init,
                                      pp_stream stream) {
    if (n < 0) return fail(PP_ERR_INVALID, "pp_grad_accum_f32_bf16: n < 0");
    if (n == 0) return PP_OK;
    if (!acc || !g) return fail(PP_ERR_INVALID, "pp_grad_accum_f32_bf16: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    int64_t body = 0;
    if (aligned(acc, 16) && aligned(g, 16)) {
        const int64_t n8 = n / 8;
        body = n8 * 8;
        if (n8 > 0) {
            const int64_t per_block = (int64_t)kAccThreads * kAccUnroll;
            const uint32_t nb = (uint32_t)((n8 + per_block - 1) / per_block);
            if (init) hipLaunchKernelGGL(accum_bf16_kernel<true>, dim3(nb), dim3(kAccThreads), 0, st, acc, g, n8);
            else hipLaunchKernelGGL(accum_bf16_kernel<false>, dim3(nb), dim3(kAccThreads), 0, st, acc, g, n8);
        }
    }
    if (body < n) {
        const uint32_t nb = (uint32_t)((n - body + kAccThreads - 1) / kAccThreads);
        if (init) hipLaunchKernelGGL(accum_bf16_tail_kernel<true>, dim3(nb), dim3(kAccThreads), 0, st, acc, g, body, n);
        else hipLaunchKernelGGL(accum_bf16_tail_kernel<false>, dim3(nb), dim3(kAccThreads), 0, st, acc, g, body, n);
    }
    return check_launch("accum_bf16_kernel");
}

extern "C" int pp_grad_accum_f32_f32(float* acc, const float* g, int64_t n, int init,
                                     pp_stream stream) {
    if (n < 0) return fail(PP_ERR_INVALID, "pp_grad_accum_f32_f32: n < 0");
    if (n == 0) return PP_OK;
    if (!acc || !g) return fail(PP_ERR_INVALID, "pp_grad_accum_f32_f32: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    int64_t body = 0;
    if (aligned(acc, 16) && aligned(g, 16)) {
        const int64_t n4 = n / 4;
        body = n4 * 4;
        if (n4 > 0) {
            const int64_t per_block = (int64_t)kAccThreads * kAccUnroll;
            const uint32_t nb = (uint32_t)((n4 + per_block - 1) / per_block);
            if (init) hipLaunchKernelGGL(accum_f32_kernel<true>, dim3(nb), dim3(kAccThreads), 0, st, acc, g, n4);
            else hipLaunchKernelGGL(accum_f32_kernel<false>, dim3(nb), dim3(kAccThreads), 0, st, acc, g, n4);
        }
    }
    if (body < n) {
        const uint32_t nb = (uint32_t)((n - body + kAccThreads - 1) / kAccThreads);
        if (init) hipLaunchKernelGGL(accum_f32_tail_kernel<true>, dim3(nb), dim3(kAccThreads), 0, st, acc, g, body, n);
        else hipLaunchKernelGGL(accum_f32_tail_kernel<false>, dim3(nb), dim3(kAccThreads), 0, st, acc, g, body, n);
    }
    return check_launch("accum_f32_kernel");
}

extern "C" int pp_fill_bytes(void* dst, int value, int64_t n_bytes, pp_stream stream) {
    if (n_bytes < 0) return fail(PP_ERR_INVALID, "pp_fill_bytes: n < 0");
    if (n_bytes == 0) return PP_OK;
    if (!dst) return fail(PP_ERR_INVALID, "pp_fill_bytes: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint8_t v = (uint8_t)value;
    int64_t body = 0;
    if (aligned(dst, 16)) {
        const int64_t n16 = n_bytes / 16;
        body = n16 * 16;
        if (n16 > 0) {
            const uint32_t w = 0x01010101u * v;
            hipLaunchKernelGGL(fill_kernel, dim3((uint32_t)((n16 + 255) / 256)), dim3(256), 0, st,
                               static_cast<uint4*>(dst), w, n16);
        }
    }
    if (body < n_bytes)
        hipLaunchKernelGGL(fill_tail_kernel, dim3((uint32_t)((n_bytes - body + 255) / 256)), dim3(256),
                           0, st, static_cast<uint8_t*>(dst), v, body, n_bytes);
    return check_launch("fill_kernel");
}
