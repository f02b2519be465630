// fp32 GEMM on the fp32 matrix cores for the small fp32 MLP configuration.  Same descriptor and operand
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

typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int FT = 32;       // output tile edge: one 32 x 32 MFMA tile per work-group
constexpr int FW = 8;        // waves per work-group; each takes every 8th k-chunk
constexpr int FC = 8;        // k values per chunk (4 MFMA steps of k = 2)
constexpr int FU = 8;        // chunks whose loads a wave has in flight at a time

// The four k values that lane (row, h) feeds to the 4 MFMA steps of a chunk starting at k0:
// k0 + 4h + {0,1,2,3}.  A and B use the same assignment, so step e of a chunk multiplies
// k = k0 + e (lanes 0-31) and k0 + 4 + e (lanes 32-63) on both sides.
__device__ __forceinline__ float4 load_chunk(const float* X, int64_t ld, bool trans, int64_t row, bool row_ok,
                                             int64_t k, int64_t K, bool vec_ok) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!row_ok || k >= K) return v;
    if (!trans) {
        const float* p = X + row * ld + k;
        if (vec_ok && k + 3 < K) return *reinterpret_cast<const float4*>(p);
        v.x = p[0];
        if (k + 1 < K) v.y = p[1];
        if (k + 2 < K) v.z = p[2];
        if (k + 3 < K) v.w = p[3];
    } else {
        const float* p = X + k * ld + row;
        v.x = p[0];
        if (k + 1 < K) v.y = p[ld];
        if (k + 2 < K) v.z = p[2 * ld];
        if (k + 3 < K) v.w = p[3 * ld];
    }
    return v;
}

// One 32 x 32 tile of C per work-group.  The problems this kernel serves are small (a few tiles,
// K up to a few thousand), so the time of a launch is the length of one work-group's dependent
// chain: the 8 waves split K between them (chunk c goes to wave c mod 8), every wave reads its
// operands straight from memory into the lanes of v_mfma_f32_32x32x2_f32 with 8 chunks of loads in
// flight, and the 8 partial tiles are summed through LDS in wave order (so the result does not
// depend on timing).
template <int EPI>
__global__ __launch_bounds__(FW * 64) void gemm_f32_kernel(const GemmF32Args g) {
    __shared__ float part[FW][FT][FT];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, h = lane >> 5;
    const int64_t m0 = (int64_t)blockIdx.x * FT, n0 = (int64_t)blockIdx.y * FT;
    const int64_t am = m0 + r, bn = n0 + r;
    const bool a_ok = am < g.M, b_ok = bn < g.N;
    const bool a_vec = !g.a_trans && (g.lda & 3) == 0 && aligned(g.A, 16);
    const bool b_vec = !g.b_trans && (g.ldb & 3) == 0 && aligned(g.B, 16);

    f32x16_t acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    const int64_t n_chunks = (g.K + FC - 1) / FC;
    for (int64_t c0 = wave; c0 < n_chunks; c0 += (int64_t)FW * FU) {
        float4 a[FU], b[FU];
#pragma unroll
        for (int u = 0; u < FU; ++u) {
            const int64_t k = (c0 + (int64_t)u * FW) * FC + 4 * h;  // past K for chunks beyond the last
            a[u] = load_chunk(g.A, g.lda, g.a_trans, am, a_ok, k, g.K, a_vec);
            b[u] = load_chunk(g.B, g.ldb, g.b_trans, bn, b_ok, k, g.K, b_vec);
        }
#pragma unroll
        for (int u = 0; u < FU; ++u) {
            if (c0 + (int64_t)u * FW >= n_chunks) break;  // the same for every lane of the wave
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].x, b[u].x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].y, b[u].y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].z, b[u].z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].w, b[u].w, acc, 0, 0, 0);
        }
    }
    // accumulator element e of lane (r, h) is C(m = 8 (e / 4) + 4 h + e % 4, n = r)
#pragma unroll
    for (int e = 0; e < 16; ++e) part[wave][8 * (e >> 2) + 4 * h + (e & 3)][r] = acc[e];
    __syncthreads();
    for (int o = tid; o < FT * FT; o += FW * 64) {
        const int i = o >> 5, j = o & 31;
        const int64_t m = m0 + i, n = n0 + j;
        if (m >= g.M || n >= g.N) continue;
        float v = part[0][i][j];
#pragma unroll
        for (int w = 1; w < FW; ++w) v += part[w][i][j];
        if ((EPI == PP_EPI_BIAS || EPI == PP_EPI_BIAS_RELU) && g.bias) v += g.bias[n];
        if (EPI == PP_EPI_BIAS_RELU) v = fmaxf(v, 0.f);
        if (EPI == PP_EPI_DRELU) v = g.aux_in[m * g.ld_aux + n] > 0.f ? v : 0.f;
        float* cp = g.C + m * g.ldc + n;
        if (EPI == PP_EPI_ACCUM_F32 && g.beta) v += *cp;
        *cp = v;
    }
}

template <int EPI>
static int launch_f32(const GemmF32Args& g, hipStream_t st) {
    const int64_t tm = (g.M + FT - 1) / FT, tn = (g.N + FT - 1) / FT;
    if (tm > 0x7fffffff || tn > 65535) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_f32: output too large");
    dim3 grid((uint32_t)tm, (uint32_t)tn);
    hipLaunchKernelGGL(gemm_f32_kernel<EPI>, grid, dim3(FW * 64), 0, st, g);
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
    if (d->colsum) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_f32: no column sums (pp_gemm_bf16 forms them)");
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
