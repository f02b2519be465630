// Stand-alone activation gradient dz = dy * act'(aux) (HBM-bound).  Transformer stages fold this
// into GEMM epilogues; small MLP stages, whose activations sit between separately lowered
// linears, use this kernel.
#include "common.h"
#include "act_math.h"

namespace pp {

template <int ACT>
__device__ __forceinline__ float act_grad(float dy, float aux) {
    if (ACT == 0) return aux > 0.f ? dy : 0.f;
    if (ACT == 1) return dy * dgelu_erf(aux);
    return dy * dgelu_tanh(aux);
}

template <int ACT>
__global__ __launch_bounds__(256) void act_bwd_bf16_kernel(const uint16_t* __restrict__ dy,
                                                           const uint16_t* __restrict__ aux,
                                                           uint16_t* __restrict__ dz, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        dz[i] = f32_to_bf16(act_grad<ACT>(bf16_to_f32(dy[i]), bf16_to_f32(aux[i])));
}
template <int ACT>
__global__ __launch_bounds__(256) void act_bwd_f32_kernel(const float* __restrict__ dy,
                                                          const float* __restrict__ aux,
                                                          float* __restrict__ dz, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        dz[i] = act_grad<ACT>(dy[i], aux[i]);
}

}  // namespace pp

using namespace pp;

extern "C" int pp_activation_bwd(const void* dy, const void* aux, void* dz, int64_t n, int act,
                                 int dtype, pp_stream stream) {
    if (n < 0) return fail(PP_ERR_INVALID, "pp_activation_bwd: n < 0");
    if (n == 0) return PP_OK;
    if (!dy || !aux || !dz) return fail(PP_ERR_INVALID, "pp_activation_bwd: null pointer");
    if (act < 0 || act > 2) return fail(PP_ERR_INVALID, "pp_activation_bwd: unknown activation %d", act);
    hipStream_t st = static_cast<hipStream_t>(stream);
    int64_t nb = (n + 255) / 256;
    if (nb > 1 << 20) nb = 1 << 20;
    const dim3 grid((uint32_t)nb), block(256);
#define PP_ACT_LAUNCH(K, T, ACT) \
    hipLaunchKernelGGL(K<ACT>, grid, block, 0, st, (const T*)dy, (const T*)aux, (T*)dz, n)
    if (dtype == PP_F32) {
        if (act == 0) PP_ACT_LAUNCH(act_bwd_f32_kernel, float, 0);
        else if (act == 1) PP_ACT_LAUNCH(act_bwd_f32_kernel, float, 1);
        else PP_ACT_LAUNCH(act_bwd_f32_kernel, float, 2);
    } else {
        if (act == 0) PP_ACT_LAUNCH(act_bwd_bf16_kernel, uint16_t, 0);
        else if (act == 1) PP_ACT_LAUNCH(act_bwd_bf16_kernel, uint16_t, 1);
        else PP_ACT_LAUNCH(act_bwd_bf16_kernel, uint16_t, 2);
    }
#undef PP_ACT_LAUNCH
    return check_launch("activation_bwd");
}
