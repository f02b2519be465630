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

// dst[c][r] = src[r][c] for 2-byte elements, 64 x 64 tiles through LDS (both sides coalesced).
__global__ __launch_bounds__(256) void transpose16_kernel(const uint16_t* __restrict__ src, int64_t rows,
                                                          int64_t cols, int64_t ld_src,
                                                          uint16_t* __restrict__ dst, int64_t ld_dst) {
    __shared__ uint16_t tile[64][64 + 2];
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {
        const int64_t r = r0 + i, c = c0 + tx;
        tile[i][tx] = (r < rows && c < cols) ? src[r * ld_src + c] : (uint16_t)0;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const int64_t c = c0 + i, r = r0 + tx;
        if (c < cols && r < rows) dst[c * ld_dst + r] = tile[tx][i];
    }
}

}  // namespace pp

using namespace pp;

extern "C" int pp_transpose_bf16(const void* src, int64_t rows, int64_t cols, int64_t ld_src, void* dst,
                                 int64_t ld_dst, pp_stream stream) {
    if (rows < 0 || cols < 0 || ld_src < cols || ld_dst < rows) return fail(PP_ERR_INVALID, "pp_transpose_bf16: bad shape");
    if (rows == 0 || cols == 0) return PP_OK;
    if (!src || !dst) return fail(PP_ERR_INVALID, "pp_transpose_bf16: null pointer");
    const dim3 grid((uint32_t)((cols + 63) / 64), (uint32_t)((rows + 63) / 64));
    if (grid.y > 65535) return fail(PP_ERR_UNSUPPORTED, "pp_transpose_bf16: too many rows");
    hipLaunchKernelGGL(transpose16_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                       (const uint16_t*)src, rows, cols, ld_src, (uint16_t*)dst, ld_dst);
    return check_launch("transpose16_kernel");
}

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
