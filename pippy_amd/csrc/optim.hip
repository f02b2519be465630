// Optimizer step on the fp32 gradient accumulators (HBM-bound): SGD with momentum and AdamW over a
// flat parameter range, one launch per stage arena.
//
// Parameters are bf16 or fp32; gradients are the fp32 accumulators of the weight-gradient passes;
// optimizer state is fp32.  An optional fp32 master copy of bf16 parameters takes the update and the
// bf16 parameter becomes its rounding, so that updates smaller than half a bf16 ulp are not lost.
// All arithmetic is fp32, one rounding per operation in the order torch.optim's single-tensor
// kernels apply them (written out below), so fp32 parameters follow torch to the last bits that
// fused multiply-adds allow.
//
// Traffic per parameter (bf16, no master copy): SGD+momentum 4 (g) + 4 + 4 (buffer) + 2 + 2 (p) =
// 16 B, AdamW 4 + 8 + 8 + 2 + 2 = 24 B; a master copy adds 8 B, fp32 parameters 4 B.
#include "common.h"

namespace pp {

constexpr int kOptThreads = 256;

struct SgdArgs {
    void* p; float* master; const float* g; float* buf;
    int64_t n;
    float lr, momentum, dampening, weight_decay;
    int nesterov, first, maximize;
};
struct AdamwArgs {
    void* p; float* master; const float* g; float* m; float* v;
    int64_t n;
    float lr, beta1, beta2, eps, weight_decay, bias1, bias2_sqrt;
    int maximize;
};

template <bool BF16>
__device__ __forceinline__ void load4(const void* p, const float* master, int64_t i, float (&x)[4]) {
    if (master) {
        const float4 w = *reinterpret_cast<const float4*>(master + i);
        x[0] = w.x; x[1] = w.y; x[2] = w.z; x[3] = w.w;
    } else if (BF16) {
        const uint2 w = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(p) + i);
        x[0] = bf16lo(w.x); x[1] = bf16hi(w.x); x[2] = bf16lo(w.y); x[3] = bf16hi(w.y);
    } else {
        const float4 w = *reinterpret_cast<const float4*>(static_cast<const float*>(p) + i);
        x[0] = w.x; x[1] = w.y; x[2] = w.z; x[3] = w.w;
    }
}
template <bool BF16>
__device__ __forceinline__ void store4(void* p, float* master, int64_t i, const float (&x)[4]) {
    if (master) *reinterpret_cast<float4*>(master + i) = make_float4(x[0], x[1], x[2], x[3]);
    if (BF16)
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(p) + i) = make_uint2(pack_bf16(x[0], x[1]), pack_bf16(x[2], x[3]));
    else
        *reinterpret_cast<float4*>(static_cast<float*>(p) + i) = make_float4(x[0], x[1], x[2], x[3]);
}

// torch.optim.SGD (_single_tensor_sgd): g' = g + wd p;  buf = first ? g' : momentum buf + (1 - dampening) g';
// g'' = nesterov ? g' + momentum buf : buf;  p = p - lr g''.
template <bool BF16>
__global__ __launch_bounds__(kOptThreads) void sgd_kernel(const SgdArgs a) {
    const int64_t i = ((int64_t)blockIdx.x * kOptThreads + threadIdx.x) * 4;
    if (i >= a.n) return;  // n is a multiple of 4
    float x[4];
    load4<BF16>(a.p, a.master, i, x);
    const float4 gw = *reinterpret_cast<const float4*>(a.g + i);
    float g[4] = {gw.x, gw.y, gw.z, gw.w};
    float b[4] = {0.f, 0.f, 0.f, 0.f};
    if (a.momentum != 0.f && !a.first) {
        const float4 bw = *reinterpret_cast<const float4*>(a.buf + i);
        b[0] = bw.x; b[1] = bw.y; b[2] = bw.z; b[3] = bw.w;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float d = a.maximize ? -g[e] : g[e];
        if (a.weight_decay != 0.f) d = d + a.weight_decay * x[e];
        if (a.momentum != 0.f) {
            b[e] = a.first ? d : a.momentum * b[e] + (1.0f - a.dampening) * d;
            d = a.nesterov ? d + a.momentum * b[e] : b[e];
        }
        x[e] = x[e] - a.lr * d;
    }
    if (a.momentum != 0.f) *reinterpret_cast<float4*>(a.buf + i) = make_float4(b[0], b[1], b[2], b[3]);
    store4<BF16>(a.p, a.master, i, x);
}

// torch.optim.AdamW (_single_tensor_adamw): p = p (1 - lr wd);  m = m + (1 - beta1)(g - m);
// v = beta2 v + (1 - beta2) g g;  denom = sqrt(v) / sqrt(1 - beta2^t) + eps;
// p = p - (lr / (1 - beta1^t)) m / denom.
template <bool BF16>
__global__ __launch_bounds__(kOptThreads) void adamw_kernel(const AdamwArgs a) {
    const int64_t i = ((int64_t)blockIdx.x * kOptThreads + threadIdx.x) * 4;
    if (i >= a.n) return;
    float x[4];
    load4<BF16>(a.p, a.master, i, x);
    const float4 gw = *reinterpret_cast<const float4*>(a.g + i);
    const float4 mw = *reinterpret_cast<const float4*>(a.m + i);
    const float4 vw = *reinterpret_cast<const float4*>(a.v + i);
    float g[4] = {gw.x, gw.y, gw.z, gw.w}, m[4] = {mw.x, mw.y, mw.z, mw.w}, v[4] = {vw.x, vw.y, vw.z, vw.w};
    const float step_size = a.lr / a.bias1;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float d = a.maximize ? -g[e] : g[e];
        x[e] = x[e] * (1.0f - a.lr * a.weight_decay);
        m[e] = m[e] + (1.0f - a.beta1) * (d - m[e]);
        v[e] = a.beta2 * v[e] + (1.0f - a.beta2) * d * d;
        const float denom = sqrtf(v[e]) / a.bias2_sqrt + a.eps;
        x[e] = x[e] - step_size * (m[e] / denom);
    }
    *reinterpret_cast<float4*>(a.m + i) = make_float4(m[0], m[1], m[2], m[3]);
    *reinterpret_cast<float4*>(a.v + i) = make_float4(v[0], v[1], v[2], v[3]);
    store4<BF16>(a.p, a.master, i, x);
}

static int check_common(const char* who, const void* p, const float* g, int64_t n, int dtype, const float* master) {
    if (n < 0) return fail(PP_ERR_INVALID, "%s: negative size", who);
    if (n == 0) return PP_OK;
    if (!p || !g) return fail(PP_ERR_INVALID, "%s: null pointer", who);
    if (dtype != PP_BF16 && dtype != PP_F32) return fail(PP_ERR_INVALID, "%s: parameter dtype %d", who, dtype);
    if (n & 3) return fail(PP_ERR_INVALID, "%s: n must be a multiple of 4 (n=%lld)", who, (long long)n);
    if (master && dtype != PP_BF16) return fail(PP_ERR_INVALID, "%s: a master copy goes with bf16 parameters", who);
    if (!aligned(p, dtype == PP_BF16 ? 8 : 16) || !aligned(g, 16) || !aligned(master, 16))
        return fail(PP_ERR_INVALID, "%s: pointers must be aligned to 4 elements", who);
    if ((n + 3) / 4 / kOptThreads > 0x7fffff00ll) return fail(PP_ERR_UNSUPPORTED, "%s: too many elements", who);
    return PP_OK;
}

}  // namespace pp

using namespace pp;

extern "C" int pp_sgd_step(void* param, int param_dtype, float* master, const float* grad, float* momentum_buf,
                           int64_t n, float lr, float momentum, float dampening, float weight_decay,
                           int nesterov, int first_step, int maximize, pp_stream stream) {
    int rc = check_common("pp_sgd_step", param, grad, n, param_dtype, master);
    if (rc || n == 0) return rc;
    if (momentum != 0.f && (!momentum_buf || !aligned(momentum_buf, 16)))
        return fail(PP_ERR_INVALID, "pp_sgd_step: momentum needs a 16-byte aligned buffer");
    if (nesterov && (momentum <= 0.f || dampening != 0.f))
        return fail(PP_ERR_INVALID, "pp_sgd_step: Nesterov momentum requires a momentum and zero dampening");
    SgdArgs a{param, master, grad, momentum_buf, n, lr, momentum, dampening, weight_decay, nesterov, first_step, maximize};
    const uint32_t grid = (uint32_t)((n / 4 + kOptThreads - 1) / kOptThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (param_dtype == PP_BF16) hipLaunchKernelGGL(sgd_kernel<true>, dim3(grid), dim3(kOptThreads), 0, st, a);
    else hipLaunchKernelGGL(sgd_kernel<false>, dim3(grid), dim3(kOptThreads), 0, st, a);
    return check_launch("sgd_kernel");
}

extern "C" int pp_adamw_step(void* param, int param_dtype, float* master, const float* grad, float* exp_avg,
                             float* exp_avg_sq, int64_t n, float lr, float beta1, float beta2, float eps,
                             float weight_decay, float bias_correction1, float bias_correction2_sqrt,
                             int maximize, pp_stream stream) {
    int rc = check_common("pp_adamw_step", param, grad, n, param_dtype, master);
    if (rc || n == 0) return rc;
    if (!exp_avg || !exp_avg_sq || !aligned(exp_avg, 16) || !aligned(exp_avg_sq, 16))
        return fail(PP_ERR_INVALID, "pp_adamw_step: moment buffers must be 16-byte aligned");
    if (!(bias_correction1 > 0.f) || !(bias_correction2_sqrt > 0.f))
        return fail(PP_ERR_INVALID, "pp_adamw_step: bias corrections must be positive");
    AdamwArgs a{param, master, grad, exp_avg, exp_avg_sq, n, lr, beta1, beta2, eps, weight_decay,
                bias_correction1, bias_correction2_sqrt, maximize};
    const uint32_t grid = (uint32_t)((n / 4 + kOptThreads - 1) / kOptThreads);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (param_dtype == PP_BF16) hipLaunchKernelGGL(adamw_kernel<true>, dim3(grid), dim3(kOptThreads), 0, st, a);
    else hipLaunchKernelGGL(adamw_kernel<false>, dim3(grid), dim3(kOptThreads), 0, st, a);
    return check_launch("adamw_kernel");
}
