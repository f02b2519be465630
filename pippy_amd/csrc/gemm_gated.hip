// SwiGLU fused into the GEMMs around it (a Llama-style feed-forward, down(silu(gate(x)) * up(x))).
//
//   forward:   one kernel computes x Wg^T and x Wu^T for the same 128 rows and 64 columns in one
//              128 x 128 tile (the B tile holds 64 rows of Wg followed by the same 64 rows of Wu), rounds
//              both to bf16, stores them side by side in gu [M, 2 N] (gate in columns [0, N), up in
//              [N, 2 N): the backward pass needs both) and writes h = silu(g) * u.  The element-wise
//              kernel that would read g and u back from memory is gone.
//   backward:  the input-gradient GEMM of the down projection, dh = dy Wd, applies the SwiGLU
//              derivative in its epilogue: it reads g and u and writes dg = dh u silu'(g) and
//              du = dh silu(g) side by side in dgu [M, 2 N]; dh itself never reaches memory.  The
//              gradients with respect to x then come from ONE GEMM over k = 2 N (dgu against the two
//              transposed weights side by side) instead of two GEMMs and an addition.
// Values are rounded exactly where the separate kernels round them (g, u, dh to bf16 before the
// activation arithmetic), so g, u, h, dg and du carry the same bits as the unfused sequence.
#include "gemm_core.h"

namespace pp {

constexpr int kGatedBM = 128, kGatedBN = 128, kGatedNS = 2;

// Forward tile: acc columns [0, 64) are the gate product, [64, 128) the up product of h columns
// [64 tile_n, 64 tile_n + 64).  Waves are 2 x 2: wave (wm, wn) holds rows 64 wm .. + 63 of the gate (wn = 0)
// or up (wn = 1) half, so the two halves of one element sit in different waves: every band of 32 rows
// goes through LDS, each wave writing its own region, and after a barrier each wave finishes 16 of the
// band's rows reading both regions.
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_swiglu_kernel(const GemmArgs g, uint16_t* gu, int64_t ld_gu) {
    typedef WaveTile<kGatedBM, kGatedBN> WT;
    static_assert(WT::WGM == 2 && WT::WGN == 2 && WT::TM == 2 && WT::TN == 2, "2 x 2 waves of 64 x 64");
    const uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= g.n_blocks) return;
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    f32x16_t acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;
    gemm_mainloop<kGatedBM, kGatedBN, false, false, kGatedNS, BK, true>(g, tile_m, tile_n, 0,
                                                                       (int)((g.K + BK - 1) / BK), acc);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int l32 = lane & 31, lh = lane >> 5;
    wait_lds();
    __builtin_amdgcn_s_barrier();  // every wave is done with the stages
    float* const regions = reinterpret_cast<float*>(smem);
    float* const mine = regions + wave * (32 * 64);
    const float* const gate_r = regions + wm * (32 * 64);
    const float* const up_r = regions + (wm + 2) * (32 * 64);
    constexpr int UPR = 16;  // 16-byte units per row of 64 floats
    auto unit_at = [](int u, int r) { return u ^ (r & (UPR - 1)); };
    const int ru = lane % UPR, rr = lane / UPR;  // this lane's 4 columns, and its row inside a pass of 4 rows
    const int64_t col = (int64_t)tile_n * 64 + ru * 4;
    const int64_t row0 = (int64_t)tile_m * kGatedBM + wm * 64;
    uint16_t* const hp = static_cast<uint16_t*>(g.C);
    static_for<2>([&](auto band) {
        constexpr int b = decltype(band)::value;
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int u = a * 8 + 2 * q + lh;
                *reinterpret_cast<float4*>(mine + l32 * 64 + (unit_at(u, l32) << 2)) =
                    make_float4(acc[a][b][4 * q], acc[a][b][4 * q + 1], acc[a][b][4 * q + 2], acc[a][b][4 * q + 3]);
            }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = 16 * wn + 4 * i + rr;  // row inside the band
            const int64_t row = row0 + b * 32 + m;
            const float4 gv = *reinterpret_cast<const float4*>(gate_r + m * 64 + (unit_at(ru, m) << 2));
            const float4 uv = *reinterpret_cast<const float4*>(up_r + m * 64 + (unit_at(ru, m) << 2));
            if (row < g.M && col < g.N) {
                const uint32_t g0 = pack_bf16(gv.x, gv.y), g1 = pack_bf16(gv.z, gv.w);
                const uint32_t u0 = pack_bf16(uv.x, uv.y), u1 = pack_bf16(uv.z, uv.w);
                const float h0 = swiglu_value(bf16lo(g0), bf16lo(u0)), h1 = swiglu_value(bf16hi(g0), bf16hi(u0));
                const float h2 = swiglu_value(bf16lo(g1), bf16lo(u1)), h3 = swiglu_value(bf16hi(g1), bf16hi(u1));
                *reinterpret_cast<uint2*>(gu + row * ld_gu + col) = make_uint2(g0, g1);
                *reinterpret_cast<uint2*>(gu + row * ld_gu + g.N + col) = make_uint2(u0, u1);
                *reinterpret_cast<uint2*>(hp + row * g.ldc + col) = make_uint2(pack_bf16(h0, h1), pack_bf16(h2, h3));
            }
        }
        __syncthreads();  // the regions are rewritten by the next band
    });
}

// Backward tile: an ordinary 128 x 128 tile of dh = dy Wd whose epilogue turns it into dg and du.
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_dswiglu_kernel(const GemmArgs g, const uint16_t* gu,
                                                                        int64_t ld_gu) {
    typedef WaveTile<kGatedBM, kGatedBN> WT;
    const uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= g.n_blocks) return;
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    f32x16_t acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;
    gemm_mainloop<kGatedBM, kGatedBN, false, false, kGatedNS, BK>(g, tile_m, tile_n, 0, (int)((g.K + BK - 1) / BK), acc);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int l32 = lane & 31, lh = lane >> 5;
    wait_lds();
    __builtin_amdgcn_s_barrier();
    float* const mine = reinterpret_cast<float*>(smem) + wave * (32 * 64);
    constexpr int UPR = 16;
    auto unit_at = [](int u, int r) { return u ^ (r & (UPR - 1)); };
    const int ru = lane % UPR, rr = lane / UPR;
    const int64_t col = (int64_t)tile_n * kGatedBN + wn * 64 + ru * 4;
    const int64_t row0 = (int64_t)tile_m * kGatedBM + wm * 64;
    uint16_t* const out = static_cast<uint16_t*>(g.C);  // dgu [M, 2 N] with row stride ldc
    static_for<2>([&](auto band) {
        constexpr int b = decltype(band)::value;
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int u = a * 8 + 2 * q + lh;
                *reinterpret_cast<float4*>(mine + l32 * 64 + (unit_at(u, l32) << 2)) =
                    make_float4(acc[a][b][4 * q], acc[a][b][4 * q + 1], acc[a][b][4 * q + 2], acc[a][b][4 * q + 3]);
            }
        // the region is private to the wave: its own LDS accesses complete in order
        float4 dh[8];
        uint2 gw[8], uw[8];
        bool ok[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int m = 4 * i + rr;
            const int64_t row = row0 + b * 32 + m;
            dh[i] = *reinterpret_cast<const float4*>(mine + m * 64 + (unit_at(ru, m) << 2));
            ok[i] = row < g.M && col < g.N;
            if (ok[i]) {
                gw[i] = *reinterpret_cast<const uint2*>(gu + row * ld_gu + col);
                uw[i] = *reinterpret_cast<const uint2*>(gu + row * ld_gu + g.N + col);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (!ok[i]) continue;
            const int64_t row = row0 + b * 32 + 4 * i + rr;
            // dh is rounded to bf16 first: what a separate GEMM would have stored
            const uint32_t d0 = pack_bf16(dh[i].x, dh[i].y), d1 = pack_bf16(dh[i].z, dh[i].w);
            const float d[4] = {bf16lo(d0), bf16hi(d0), bf16lo(d1), bf16hi(d1)};
            const float gg[4] = {bf16lo(gw[i].x), bf16hi(gw[i].x), bf16lo(gw[i].y), bf16hi(gw[i].y)};
            const float uu[4] = {bf16lo(uw[i].x), bf16hi(uw[i].x), bf16lo(uw[i].y), bf16hi(uw[i].y)};
            float dg[4], du[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) swiglu_grads(gg[e], uu[e], d[e], &dg[e], &du[e]);
            *reinterpret_cast<uint2*>(out + row * g.ldc + col) = make_uint2(pack_bf16(dg[0], dg[1]), pack_bf16(dg[2], dg[3]));
            *reinterpret_cast<uint2*>(out + row * g.ldc + g.N + col) =
                make_uint2(pack_bf16(du[0], du[1]), pack_bf16(du[2], du[3]));
        }
    });
}

static int gated_check(const char* who, const void* a, const void* b, int64_t M, int64_t N, int64_t K, int64_t lda,
                       int64_t ldb) {
    if (M < 0 || N < 0 || K < 0) return fail(PP_ERR_INVALID, "%s: negative size", who);
    if (!a || !b) return fail(PP_ERR_INVALID, "%s: null operand", who);
    if (!aligned(a, 16) || !aligned(b, 16)) return fail(PP_ERR_INVALID, "%s: operands must be 16-byte aligned", who);
    if ((K & 7) || (lda & 7) || (ldb & 7) || lda < K || ldb < K)
        return fail(PP_ERR_INVALID, "%s: K and the leading dimensions of A and B must be multiples of 8 and at least K", who);
    if (N & 7) return fail(PP_ERR_UNSUPPORTED, "%s: N must be a multiple of 8 (N=%lld)", who, (long long)N);
    if ((uint64_t)M * (uint64_t)lda * 2 >= 0x7ffffff0ull || (uint64_t)N * (uint64_t)ldb * 2 >= 0x7ffffff0ull)
        return fail(PP_ERR_UNSUPPORTED, "%s: an operand spans 2 GiB or more", who);
    return PP_OK;
}

static void fill_args(GemmArgs& g, const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                      int64_t ldb, int64_t ldc) {
    g.A = static_cast<const uint16_t*>(A);
    g.B = static_cast<const uint16_t*>(B);
    g.B2 = nullptr;
    g.C = C;
    g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc;
    g.bias = nullptr; g.aux_in = nullptr; g.aux_out = nullptr;
    g.ld_aux = 0; g.beta = 0; g.round_bf16 = 0; g.epi = PP_EPI_NONE;
}

}  // namespace pp

using namespace pp;

extern "C" int pp_gemm_bf16_swiglu(const void* x, const void* w_gate, const void* w_up, void* gu, void* h,
                                   int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ld_gu,
                                   int64_t ldh, pp_stream stream) {
    int rc = gated_check("pp_gemm_bf16_swiglu", x, w_gate, M, N, K, ldx, ldw);
    if (rc) return rc;
    if (M == 0 || N == 0) return PP_OK;
    if (!w_up || !gu || !h) return fail(PP_ERR_INVALID, "pp_gemm_bf16_swiglu: null pointer");
    if (!aligned(w_up, 16) || !aligned(gu, 8) || !aligned(h, 8))
        return fail(PP_ERR_INVALID, "pp_gemm_bf16_swiglu: misaligned pointer");
    if (ld_gu < 2 * N || (ld_gu & 3) || ldh < N || (ldh & 3))
        return fail(PP_ERR_INVALID, "pp_gemm_bf16_swiglu: ld_gu >= 2 N and ldh >= N, both multiples of 4");
    GemmArgs g;
    fill_args(g, x, w_gate, h, M, N, K, ldx, ldw, ldh);
    g.B2 = static_cast<const uint16_t*>(w_up);
    g.tiles_m = (uint32_t)((M + kGatedBM - 1) / kGatedBM);
    g.tiles_n = (uint32_t)((N + 63) / 64);  // a tile covers 64 columns of h
    const uint64_t nb = (uint64_t)g.tiles_m * g.tiles_n;
    if (nb > 0x0fffff00ull) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_swiglu: too many tiles");
    g.n_blocks = (uint32_t)nb;
    constexpr size_t lds = (size_t)kGatedNS * (kGatedBM + kGatedBN) * BK * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_swiglu_kernel, lds);
    if (attr_rc) return attr_rc;
    hipLaunchKernelGGL(gemm_bf16_swiglu_kernel, dim3((g.n_blocks + 7) / 8 * 8), dim3(kGemmThreads), lds,
                       static_cast<hipStream_t>(stream), g, static_cast<uint16_t*>(gu), ld_gu);
    return check_launch("gemm_bf16_swiglu_kernel");
}

extern "C" int pp_gemm_bf16_dswiglu(const void* dy, const void* w_down_t, const void* gu, void* dgu, int64_t M,
                                    int64_t N, int64_t K, int64_t ldy, int64_t ldw, int64_t ld_gu, int64_t ld_dgu,
                                    pp_stream stream) {
    int rc = gated_check("pp_gemm_bf16_dswiglu", dy, w_down_t, M, N, K, ldy, ldw);
    if (rc) return rc;
    if (M == 0 || N == 0) return PP_OK;
    if (!gu || !dgu) return fail(PP_ERR_INVALID, "pp_gemm_bf16_dswiglu: null pointer");
    if (!aligned(gu, 8) || !aligned(dgu, 8)) return fail(PP_ERR_INVALID, "pp_gemm_bf16_dswiglu: misaligned pointer");
    if (ld_gu < 2 * N || (ld_gu & 3) || ld_dgu < 2 * N || (ld_dgu & 3))
        return fail(PP_ERR_INVALID, "pp_gemm_bf16_dswiglu: ld_gu and ld_dgu >= 2 N, multiples of 4");
    GemmArgs g;
    fill_args(g, dy, w_down_t, dgu, M, N, K, ldy, ldw, ld_dgu);
    rc = count_tiles<kGatedBM, kGatedBN>(g);
    if (rc) return rc;
    constexpr size_t lds = (size_t)kGatedNS * (kGatedBM + kGatedBN) * BK * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_dswiglu_kernel, lds);
    if (attr_rc) return attr_rc;
    hipLaunchKernelGGL(gemm_bf16_dswiglu_kernel, dim3((g.n_blocks + 7) / 8 * 8), dim3(kGemmThreads), lds,
                       static_cast<hipStream_t>(stream), g, static_cast<const uint16_t*>(gu), ld_gu);
    return check_launch("gemm_bf16_dswiglu_kernel");
}
