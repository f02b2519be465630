// fp32 GEMM (SIMT, LDS-tiled) for the small fp32 MLP configuration.  Same descriptor and operand
// conventions as the bf16 MFMA GEMM: C[M,N] = epilogue( sum_k A(m,k) * B(n,k) ).
#include "common.h"

namespace pp {

struct GemmF32Args {
    const float* A;
    const float* B;
    float* C;
    int64_t M, N, K, lda, ldb, ldc;
    const float* bias;
    const float* aux_in;
    int64_t ld_aux;
    int beta;
    int a_trans, b_trans;
};

constexpr int FT = 64;   // output tile edge
constexpr int FK = 16;   // k step

template <int EPI>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const GemmF32Args g) {
    __shared__ float As[FK][FT + 1];
    __shared__ float Bs[FK][FT + 1];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;  // 16 x 16 lanes, 4 x 4 outputs each
    const int64_t m0 = (int64_t)blockIdx.x * FT, n0 = (int64_t)blockIdx.y * FT;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int64_t k0 = 0; k0 < g.K; k0 += FK) {
        // 64 x 16 elements per operand, 4 per lane
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int id = tid + 256 * i;
            int r, k;
            if (g.a_trans) { r = id & 63; k = id >> 6; } else { k = id & 15; r = id >> 4; }
            const int64_t gm = m0 + r, gk = k0 + k;
            float v = 0.f;
            if (gm < g.M && gk < g.K) v = g.a_trans ? g.A[gk * g.lda + gm] : g.A[gm * g.lda + gk];
            As[k][r] = v;
            if (g.b_trans) { r = id & 63; k = id >> 6; } else { k = id & 15; r = id >> 4; }
            const int64_t gn = n0 + r, gk2 = k0 + k;
            v = 0.f;
            if (gn < g.N && gk2 < g.K) v = g.b_trans ? g.B[gk2 * g.ldb + gn] : g.B[gn * g.ldb + gk2];
            Bs[k][r] = v;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < FK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t m = m0 + ty * 4 + i;
        if (m >= g.M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t n = n0 + tx * 4 + j;
            if (n >= g.N) continue;
            float v = acc[i][j];
            if ((EPI == PP_EPI_BIAS || EPI == PP_EPI_BIAS_RELU) && g.bias) v += g.bias[n];
            if (EPI == PP_EPI_BIAS_RELU) v = fmaxf(v, 0.f);
            if (EPI == PP_EPI_DRELU) v = g.aux_in[m * g.ld_aux + n] > 0.f ? v : 0.f;
            float* cp = g.C + m * g.ldc + n;
            if (EPI == PP_EPI_ACCUM_F32 && g.beta) v += *cp;
            *cp = v;
        }
    }
}

template <int EPI>
static int launch_f32(const GemmF32Args& g, hipStream_t st) {
    dim3 grid((uint32_t)((g.M + FT - 1) / FT), (uint32_t)((g.N + FT - 1) / FT));
    hipLaunchKernelGGL(gemm_f32_kernel<EPI>, grid, dim3(256), 0, st, g);
    return check_launch("gemm_f32_kernel");
}

}  // namespace pp

using namespace pp;

extern "C" int pp_gemm_f32(const pp_gemm_desc* d, pp_stream stream) {
    if (!d) return fail(PP_ERR_INVALID, "pp_gemm_f32: null descriptor");
    if (d->M < 0 || d->N < 0 || d->K < 0) return fail(PP_ERR_INVALID, "pp_gemm_f32: negative size");
    if (d->M == 0 || d->N == 0) return PP_OK;
    if (!d->A || !d->B || !d->C) return fail(PP_ERR_INVALID, "pp_gemm_f32: null operand");
    if (d->c_dtype != PP_F32) return fail(PP_ERR_INVALID, "pp_gemm_f32: C must be fp32");
    if (d->lda < (d->a_trans ? d->M : d->K) || d->ldb < (d->b_trans ? d->N : d->K) || d->ldc < d->N)
        return fail(PP_ERR_INVALID, "pp_gemm_f32: leading dimension too small");
    if (d->epilogue == PP_EPI_DRELU && (!d->aux_in || d->ld_aux < d->N))
        return fail(PP_ERR_INVALID, "pp_gemm_f32: PP_EPI_DRELU needs aux_in");
    GemmF32Args g;
    g.A = static_cast<const float*>(d->A);
    g.B = static_cast<const float*>(d->B);
    g.C = static_cast<float*>(d->C);
    g.M = d->M; g.N = d->N; g.K = d->K;
    g.lda = d->lda; g.ldb = d->ldb; g.ldc = d->ldc;
    g.bias = static_cast<const float*>(d->bias);
    g.aux_in = static_cast<const float*>(d->aux_in);
    g.ld_aux = d->ld_aux;
    g.beta = d->beta;
    g.a_trans = d->a_trans ? 1 : 0;
    g.b_trans = d->b_trans ? 1 : 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (d->epilogue) {
        case PP_EPI_NONE: return launch_f32<PP_EPI_NONE>(g, st);
        case PP_EPI_BIAS: return launch_f32<PP_EPI_BIAS>(g, st);
        case PP_EPI_BIAS_RELU: return launch_f32<PP_EPI_BIAS_RELU>(g, st);
        case PP_EPI_DRELU: return launch_f32<PP_EPI_DRELU>(g, st);
        case PP_EPI_ACCUM_F32: return launch_f32<PP_EPI_ACCUM_F32>(g, st);
        default: return fail(PP_ERR_UNSUPPORTED, "pp_gemm_f32: epilogue %d", d->epilogue);
    }
}
