// SwiGLU gate and rotary position embedding: the element-wise pieces of a Llama-style layer
// (HBM-bound; 8 bf16 elements = 16 bytes per lane and access).
#include "common.h"
#include "act_math.h"

namespace pp {

__device__ __forceinline__ void unpack8(const uint4& w, float (&f)[8]) {
    f[0] = bf16lo(w.x); f[1] = bf16hi(w.x); f[2] = bf16lo(w.y); f[3] = bf16hi(w.y);
    f[4] = bf16lo(w.z); f[5] = bf16hi(w.z); f[6] = bf16lo(w.w); f[7] = bf16hi(w.w);
}
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
    return make_uint4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7]));
}

// h = silu(g) * u
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const uint4* __restrict__ g, const uint4* __restrict__ u,
                                                         uint4* __restrict__ h, int64_t n8) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
        float gf[8], uf[8], o[8];
        unpack8(g[i], gf);
        unpack8(u[i], uf);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = swiglu_value(gf[e], uf[e]);
        h[i] = pack8(o);
    }
}

// dg = dh * u * silu'(g),  du = dh * silu(g);  silu'(g) = s (1 + g (1 - s)),  s = sigmoid(g)
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const uint4* __restrict__ g, const uint4* __restrict__ u,
                                                         const uint4* __restrict__ dh, uint4* __restrict__ dg,
                                                         uint4* __restrict__ du, int64_t n8) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
        float gf[8], uf[8], df[8], og[8], ou[8];
        unpack8(g[i], gf);
        unpack8(u[i], uf);
        unpack8(dh[i], df);
#pragma unroll
        for (int e = 0; e < 8; ++e) swiglu_grads(gf[e], uf[e], df[e], &og[e], &ou[e]);
        dg[i] = pack8(og);
        du[i] = pack8(ou);
    }
}

// In-place rotation of `n_heads` heads of width D at the start of every row of x [n_tok, ld]:
// (a, b) = (x[i], x[i + D/2]) -> (a cos - b sin, b cos + a sin) with the angle of position
// t % seq and frequency i taken from tables cos/sin [seq, D/2] (fp32).  sign = -1 applies the
// transposed rotation, which is the backward pass.
__global__ __launch_bounds__(256) void rope_kernel(uint16_t* __restrict__ x, const float* __restrict__ cos_t,
                                                   const float* __restrict__ sin_t, int64_t n_tok, int64_t seq,
                                                   int n_heads, int D, int64_t ld, float sign) {
    const int half8 = D >> 4;  // 16-byte chunks in half a head
    const int64_t total = n_tok * n_heads * half8;
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int c = (int)(idx % half8);
        const int64_t th = idx / half8;
        const int hd = (int)(th % n_heads);
        const int64_t t = th / n_heads;
        uint16_t* p = x + t * ld + (int64_t)hd * D + c * 8;
        const float* cp = cos_t + (t % seq) * (D >> 1) + c * 8;
        const float* sp = sin_t + (t % seq) * (D >> 1) + c * 8;
        float a[8], b[8], oa[8], ob[8];
        unpack8(*reinterpret_cast<const uint4*>(p), a);
        unpack8(*reinterpret_cast<const uint4*>(p + (D >> 1)), b);
        const float4 c0 = *reinterpret_cast<const float4*>(cp), c1 = *reinterpret_cast<const float4*>(cp + 4);
        const float4 s0 = *reinterpret_cast<const float4*>(sp), s1 = *reinterpret_cast<const float4*>(sp + 4);
        const float cs[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
        const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float s = sign * sn[e];
            oa[e] = a[e] * cs[e] - b[e] * s;
            ob[e] = b[e] * cs[e] + a[e] * s;
        }
        *reinterpret_cast<uint4*>(p) = pack8(oa);
        *reinterpret_cast<uint4*>(p + (D >> 1)) = pack8(ob);
    }
}

static uint32_t grid_for(int64_t items) {
    int64_t nb = (items + 255) / 256;
    if (nb > (1 << 20)) nb = 1 << 20;
    return (uint32_t)(nb > 0 ? nb : 1);
}

}  // namespace pp

using namespace pp;

extern "C" int pp_swiglu_fwd(const void* g, const void* u, void* h, int64_t n, pp_stream stream) {
    if (n < 0 || (n & 7)) return fail(PP_ERR_INVALID, "pp_swiglu_fwd: n must be a non-negative multiple of 8");
    if (n == 0) return PP_OK;
    if (!g || !u || !h) return fail(PP_ERR_INVALID, "pp_swiglu_fwd: null pointer");
    if (!aligned(g, 16) || !aligned(u, 16) || !aligned(h, 16)) return fail(PP_ERR_INVALID, "pp_swiglu_fwd: pointers must be 16-byte aligned");
    hipLaunchKernelGGL(swiglu_fwd_kernel, dim3(grid_for(n / 8)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       (const uint4*)g, (const uint4*)u, (uint4*)h, n / 8);
    return check_launch("swiglu_fwd_kernel");
}

extern "C" int pp_swiglu_bwd(const void* g, const void* u, const void* dh, void* dg, void* du, int64_t n,
                             pp_stream stream) {
    if (n < 0 || (n & 7)) return fail(PP_ERR_INVALID, "pp_swiglu_bwd: n must be a non-negative multiple of 8");
    if (n == 0) return PP_OK;
    if (!g || !u || !dh || !dg || !du) return fail(PP_ERR_INVALID, "pp_swiglu_bwd: null pointer");
    if (!aligned(g, 16) || !aligned(u, 16) || !aligned(dh, 16) || !aligned(dg, 16) || !aligned(du, 16))
        return fail(PP_ERR_INVALID, "pp_swiglu_bwd: pointers must be 16-byte aligned");
    hipLaunchKernelGGL(swiglu_bwd_kernel, dim3(grid_for(n / 8)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       (const uint4*)g, (const uint4*)u, (const uint4*)dh, (uint4*)dg, (uint4*)du, n / 8);
    return check_launch("swiglu_bwd_kernel");
}

extern "C" int pp_rope(void* x, const float* cos_table, const float* sin_table, int64_t n_tok, int64_t seq,
                       int64_t n_heads, int64_t D, int64_t ld, int inverse, pp_stream stream) {
    if (n_tok < 0 || seq <= 0 || n_heads < 0 || D <= 0) return fail(PP_ERR_INVALID, "pp_rope: bad shape");
    if (D % 16) return fail(PP_ERR_UNSUPPORTED, "pp_rope: head width %lld is not a multiple of 16", (long long)D);
    if (ld < n_heads * D || (ld & 7)) return fail(PP_ERR_INVALID, "pp_rope: ld too small or not a multiple of 8");
    if (n_tok == 0 || n_heads == 0) return PP_OK;
    if (!x || !cos_table || !sin_table) return fail(PP_ERR_INVALID, "pp_rope: null pointer");
    if (!aligned(x, 16) || !aligned(cos_table, 16) || !aligned(sin_table, 16))
        return fail(PP_ERR_INVALID, "pp_rope: pointers must be 16-byte aligned");
    hipLaunchKernelGGL(rope_kernel, dim3(grid_for(n_tok * n_heads * (D / 16))), dim3(256), 0,
                       static_cast<hipStream_t>(stream), (uint16_t*)x, cos_table, sin_table, n_tok, seq,
                       (int)n_heads, (int)D, ld, inverse ? -1.0f : 1.0f);
    return check_launch("rope_kernel");
}
