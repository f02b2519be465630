// SwiGLU fused into the GEMMs around it (a Llama-style feed-forward, down(silu(gate(x)) * up(x))).
//
//   forward:   one kernel computes x Wg^T and x Wu^T for the same rows and columns in one tile (128 x 128:
//              the B tile holds 64 rows of Wg followed by the same 64 rows of Wu; or 256 x 256), rounds
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

// Forward tile of BM rows and BN / 2 columns of h: the B tile holds BN / 2 rows of Wg followed by the same
// BN / 2 rows of Wu, and the main loop hands every wave the gate and the up product of the same columns
// (the first half of its accumulator tiles is the gate, the second the up product), so that a band of 32
// rows goes through the wave's own LDS region and comes back with both values of an element in one lane.
template <int BM, int BN, int NS, int W>
__device__ __forceinline__ void swiglu_tile(const GemmArgs& g, uint16_t* gu, int64_t ld_gu, uint32_t tile_m,
                                            uint32_t tile_n) {
    typedef WaveTile<BM, BN, W> WT;
    constexpr int WTM = WT::WTM, WTN = WT::WTN, TM = WT::TM, TN = WT::TN;
    constexpr int H = WTN / 2;      // columns of h per wave
    constexpr int UPR = WTN / 4;    // 16-byte units per row of the region
    constexpr int UPH = H / 4;      // ... of which the gate half, and as many lanes per row
    constexpr int RPP = 64 / UPH;   // rows per pass
    constexpr int kPasses = 32 / RPP;
    static_assert(TN % 2 == 0 && (UPR & (UPR - 1)) == 0 && 64 % UPH == 0 && 32 % RPP == 0, "wave tile of 64 or 128 columns");
    f32x16_t acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;
    gemm_mainloop<BM, BN, false, false, NS, BK, true, W>(g, tile_m, tile_n, 0, (int)((g.K + BK - 1) / BK), acc);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WT::WGM, wn = wave / WT::WGM;
    const int l32 = lane & 31, lh = lane >> 5;
    wait_lds();
    __builtin_amdgcn_s_barrier();  // every wave is done with the stages
    float* const cw = reinterpret_cast<float*>(smem) + wave * (32 * WTN);
    auto unit_at = [](int u, int r) { return u ^ (r & (UPR - 1)); };
    const int ru = lane % UPH, rr = lane / UPH;  // this lane's 4 columns of h, and its row inside a pass
    const int64_t col = (int64_t)tile_n * (BN / 2) + wn * H + ru * 4;
    const int64_t row0 = (int64_t)tile_m * BM + wm * WTM;
    uint16_t* const hp = static_cast<uint16_t*>(g.C);
    static_for<TM>([&](auto band) {
        constexpr int b = decltype(band)::value;
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int u = a * 8 + 2 * q + lh;
                *reinterpret_cast<float4*>(cw + l32 * WTN + (unit_at(u, l32) << 2)) =
                    make_float4(acc[a][b][4 * q], acc[a][b][4 * q + 1], acc[a][b][4 * q + 2], acc[a][b][4 * q + 3]);
            }
        // the region is private to the wave: its own LDS accesses complete in order
        float4 gv[kPasses], uv[kPasses];
#pragma unroll
        for (int i = 0; i < kPasses; ++i) {
            const int m = i * RPP + rr;  // row inside the band
            gv[i] = *reinterpret_cast<const float4*>(cw + m * WTN + (unit_at(ru, m) << 2));
            uv[i] = *reinterpret_cast<const float4*>(cw + m * WTN + (unit_at(UPH + ru, m) << 2));
        }
#pragma unroll
        for (int i = 0; i < kPasses; ++i) {
            const int64_t row = row0 + b * 32 + i * RPP + rr;
            if (row < g.M && col < g.N) {
                const uint32_t g0 = pack_bf16(gv[i].x, gv[i].y), g1 = pack_bf16(gv[i].z, gv[i].w);
                const uint32_t u0 = pack_bf16(uv[i].x, uv[i].y), u1 = pack_bf16(uv[i].z, uv[i].w);
                const float h0 = swiglu_value(bf16lo(g0), bf16lo(u0)), h1 = swiglu_value(bf16hi(g0), bf16hi(u0));
                const float h2 = swiglu_value(bf16lo(g1), bf16lo(u1)), h3 = swiglu_value(bf16hi(g1), bf16hi(u1));
                *reinterpret_cast<uint2*>(gu + row * ld_gu + col) = make_uint2(g0, g1);
                *reinterpret_cast<uint2*>(gu + row * ld_gu + g.N + col) = make_uint2(u0, u1);
                *reinterpret_cast<uint2*>(hp + row * g.ldc + col) = make_uint2(pack_bf16(h0, h1), pack_bf16(h2, h3));
            }
        }
    });
}

// Backward tile: an ordinary tile of dh = dy Wd whose epilogue turns it into dg and du.
template <int BM, int BN, int NS, int W>
__device__ __forceinline__ void dswiglu_tile(const GemmArgs& g, const uint16_t* gu, int64_t ld_gu, uint32_t tile_m,
                                             uint32_t tile_n) {
    typedef WaveTile<BM, BN, W> WT;
    constexpr int WTM = WT::WTM, WTN = WT::WTN, TM = WT::TM, TN = WT::TN;
    constexpr int UPR = WTN / 4;   // 16-byte units per row
    constexpr int RPP = 64 / UPR;  // rows per pass of the wave
    constexpr int kPasses = 32 / RPP;
    constexpr int kBatch = kPasses < 8 ? kPasses : 8;  // passes whose loads are in flight together
    static_assert(UPR % 8 == 0 && 32 % RPP == 0 && kPasses % kBatch == 0, "the unit swizzle works on groups of 8 units");
    f32x16_t acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;
    gemm_mainloop<BM, BN, false, false, NS, BK, false, W>(g, tile_m, tile_n, 0, (int)((g.K + BK - 1) / BK), acc);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WT::WGM, wn = wave / WT::WGM;
    const int l32 = lane & 31, lh = lane >> 5;
    wait_lds();
    __builtin_amdgcn_s_barrier();
    float* const cw = reinterpret_cast<float*>(smem) + wave * (32 * WTN);
    // unit u of row r lives at unit (u with its low 3 bits XORed by r) when UPR is not a power of two
    auto unit_at = [](int u, int r) {
        return (UPR & (UPR - 1)) == 0 ? (u ^ (r & (UPR - 1))) : ((u & ~7) | ((u ^ r) & 7));
    };
    const bool lane_on = lane < RPP * UPR;  // 24 units per row (96 columns): two rows fill 48 lanes of a pass
    const int ru = lane % UPR, rr = lane / UPR;
    const int64_t col = (int64_t)tile_n * BN + wn * WTN + ru * 4;
    const int64_t row0 = (int64_t)tile_m * BM + wm * WTM;
    uint16_t* const out = static_cast<uint16_t*>(g.C);  // dgu [M, 2 N] with row stride ldc
    // The passes of the tile's bands run in batches of kBatch; the g and u values of a batch are fetched one
    // batch ahead (two register sets), so that their way from memory overlaps the arithmetic and the stores
    // of the batch before (with one work-group per CU nothing else would run meanwhile).
    constexpr int kPerBand = kPasses / kBatch, kBatches = TM * kPerBand;
    uint2 gw[2][kBatch], uw[2][kBatch];
    auto fetch = [&](auto set_c, int k) {
        constexpr int set = decltype(set_c)::value;
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int64_t row = row0 + (k / kPerBand) * 32 + ((k % kPerBand) * kBatch + j) * RPP + rr;
            if (lane_on && row < g.M && col < g.N) {
                gw[set][j] = *reinterpret_cast<const uint2*>(gu + row * ld_gu + col);
                uw[set][j] = *reinterpret_cast<const uint2*>(gu + row * ld_gu + g.N + col);
            }
        }
    };
    fetch(std::integral_constant<int, 0>{}, 0);
    static_for<kBatches>([&](auto batch) {
        constexpr int k = decltype(batch)::value, b = k / kPerBand, i0 = (k % kPerBand) * kBatch, set = k & 1;
        if constexpr (k + 1 < kBatches) fetch(std::integral_constant<int, (k + 1) & 1>{}, k + 1);
        if constexpr (i0 == 0) {
#pragma unroll
            for (int a = 0; a < TN; ++a)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int u = a * 8 + 2 * q + lh;
                    *reinterpret_cast<float4*>(cw + l32 * WTN + (unit_at(u, l32) << 2)) =
                        make_float4(acc[a][b][4 * q], acc[a][b][4 * q + 1], acc[a][b][4 * q + 2], acc[a][b][4 * q + 3]);
                }
        }
        // the region is private to the wave: its own LDS accesses complete in order
        float4 dh[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int m = (i0 + j) * RPP + rr;
            dh[j] = *reinterpret_cast<const float4*>(cw + (lane_on ? m : 0) * WTN + (unit_at(lane_on ? ru : 0, m) << 2));
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int64_t row = row0 + b * 32 + (i0 + j) * RPP + rr;
            if (!(lane_on && row < g.M && col < g.N)) continue;
            // dh is rounded to bf16 first: what a separate GEMM would have stored
            const uint32_t d0 = pack_bf16(dh[j].x, dh[j].y), d1 = pack_bf16(dh[j].z, dh[j].w);
            const float d[4] = {bf16lo(d0), bf16hi(d0), bf16lo(d1), bf16hi(d1)};
            const float gg[4] = {bf16lo(gw[set][j].x), bf16hi(gw[set][j].x), bf16lo(gw[set][j].y), bf16hi(gw[set][j].y)};
            const float uu[4] = {bf16lo(uw[set][j].x), bf16hi(uw[set][j].x), bf16lo(uw[set][j].y), bf16hi(uw[set][j].y)};
            float dg[4], du[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) swiglu_grads(gg[e], uu[e], d[e], &dg[e], &du[e]);
            *reinterpret_cast<uint2*>(out + row * g.ldc + col) = make_uint2(pack_bf16(dg[0], dg[1]), pack_bf16(dg[2], dg[3]));
            *reinterpret_cast<uint2*>(out + row * g.ldc + g.N + col) =
                make_uint2(pack_bf16(du[0], du[1]), pack_bf16(du[2], du[3]));
        }
    });
}

template <int BM, int BN, int NS, int W>
__global__ __launch_bounds__(W * 64) void gemm_bf16_swiglu_kernel(const GemmArgs g, uint16_t* gu, int64_t ld_gu) {
    const uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= g.n_blocks) return;
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    swiglu_tile<BM, BN, NS, W>(g, gu, ld_gu, tile_m, tile_n);
}

template <int BM, int BN, int NS, int W>
__global__ __launch_bounds__(W * 64) void gemm_bf16_dswiglu_kernel(const GemmArgs g, const uint16_t* gu, int64_t ld_gu) {
    const uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= g.n_blocks) return;
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    dswiglu_tile<BM, BN, NS, W>(g, gu, ld_gu, tile_m, tile_n);
}

// The same two tiles over rows that are partitioned into segments with a weight of their own each (the
// experts of a mixture-of-experts layer over its permuted token rows): segment e multiplies its rows by
// w_a[e] (and w_b[e], forward).  The segment bounds live in device memory; see seg_rows_locate.
struct GatedSegArgs {
    GemmArgs g;  // M = total rows; B and B2 unused
    const int32_t* seg_start;
    const void* const* w_a;
    const void* const* w_b;
    int n_seg;
};

template <int BM, int BN, int NS, int W, bool FWD>
__global__ __launch_bounds__(W * 64) void gemm_bf16_seg_gated_kernel(const GatedSegArgs sa, uint16_t* gu, int64_t ld_gu) {
    int e;
    int32_t r0, r1;
    uint32_t tiles_m, bid;
    if (!seg_rows_locate<BM>(sa.seg_start, sa.n_seg, sa.g.tiles_n, &e, &r0, &r1, &tiles_m, &bid)) return;
    GemmArgs g = sa.g;
    g.M = r1 - r0;
    g.A += (int64_t)r0 * g.lda;
    g.B = static_cast<const uint16_t*>(sa.w_a[e]);
    if (FWD) g.B2 = static_cast<const uint16_t*>(sa.w_b[e]);
    g.C = static_cast<uint16_t*>(g.C) + (int64_t)r0 * g.ldc;
    gu += (int64_t)r0 * ld_gu;
    uint32_t tile_m, tile_n;
    grouped_tile(bid, tiles_m, g.tiles_n, &tile_m, &tile_n);
    if constexpr (FWD) swiglu_tile<BM, BN, NS, W>(g, gu, ld_gu, tile_m, tile_n);
    else dswiglu_tile<BM, BN, NS, W>(g, gu, ld_gu, tile_m, tile_n);
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

// Tile choice.  Small problems keep 128 x 128 tiles on 4 waves (two work-groups per CU).  A problem whose
// 256-row tiles on 8 waves fill the CUs takes those: the forward 256 x 256 (128 columns of h), the backward
// 256 x 192 or 256 x 256, whichever needs less time by rounds of work-groups x tile area (Llama-2-7B feed-forward,
// 2048 tokens: forward 466 -> 403 us, backward 247 -> 226 us; with one work-group per CU nothing runs beside
// a tile's epilogue and all CUs reach it together, which is why the gain is smaller than that of the plain
// GEMM on the same tiles).
template <int BM, int BN, int NS, int W>
static int launch_swiglu(GemmArgs& g, uint16_t* gu, int64_t ld_gu, hipStream_t st) {
    g.tiles_m = (uint32_t)((g.M + BM - 1) / BM);
    g.tiles_n = (uint32_t)((g.N + BN / 2 - 1) / (BN / 2));  // a tile covers BN / 2 columns of h
    const uint64_t nb = (uint64_t)g.tiles_m * g.tiles_n;
    if (nb > 0x0fffff00ull) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_swiglu: too many tiles");
    g.n_blocks = (uint32_t)nb;
    constexpr size_t lds = (size_t)NS * (BM + BN) * BK * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_swiglu_kernel<BM, BN, NS, W>, lds);
    if (attr_rc) return attr_rc;
    hipLaunchKernelGGL((gemm_bf16_swiglu_kernel<BM, BN, NS, W>), dim3((g.n_blocks + 7) / 8 * 8), dim3(W * 64), lds, st,
                       g, gu, ld_gu);
    return check_launch("gemm_bf16_swiglu_kernel");
}

template <int BM, int BN, int NS, int W>
static int launch_dswiglu(GemmArgs& g, const uint16_t* gu, int64_t ld_gu, hipStream_t st) {
    int rc = count_tiles<BM, BN>(g);
    if (rc) return rc;
    constexpr size_t lds = (size_t)NS * (BM + BN) * BK * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_dswiglu_kernel<BM, BN, NS, W>, lds);
    if (attr_rc) return attr_rc;
    hipLaunchKernelGGL((gemm_bf16_dswiglu_kernel<BM, BN, NS, W>), dim3((g.n_blocks + 7) / 8 * 8), dim3(W * 64), lds, st,
                       g, gu, ld_gu);
    return check_launch("gemm_bf16_dswiglu_kernel");
}

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
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (wide_tile_for(M, 2 * N, /*allow_192=*/false) == 256)
        return launch_swiglu<256, 256, 2, 8>(g, static_cast<uint16_t*>(gu), ld_gu, st);
    return launch_swiglu<128, 128, 2, 4>(g, static_cast<uint16_t*>(gu), ld_gu, st);
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
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint16_t* gup = static_cast<const uint16_t*>(gu);
    switch (wide_tile_for(M, N, /*allow_192=*/true)) {
        case 256: return launch_dswiglu<256, 256, 2, 8>(g, gup, ld_gu, st);
        case 192: return launch_dswiglu<256, 192, 2, 8>(g, gup, ld_gu, st);
        default: return launch_dswiglu<128, 128, 2, 4>(g, gup, ld_gu, st);
    }
}

// Rows-segmented forms (the expert feed-forwards of a mixture-of-experts layer): 128 x 128 tiles on 4 waves,
// two work-groups per CU, as the segmented GEMMs they replace; the grid is an upper bound on the tiles.
template <bool FWD>
static int launch_seg_gated(GatedSegArgs& sa, uint16_t* gu, int64_t ld_gu, hipStream_t st, const char* who) {
    constexpr int BM = 128, BN = 128, NS = 2, W = 4;
    constexpr size_t lds = (size_t)NS * (BM + BN) * BK * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_seg_gated_kernel<BM, BN, NS, W, FWD>, lds);
    if (attr_rc) return attr_rc;
    const int64_t cols = FWD ? BN / 2 : BN;  // columns of N per tile
    sa.g.tiles_n = (uint32_t)((sa.g.N + cols - 1) / cols);
    // every segment may end in a partly filled tile row
    const uint64_t bound = ((uint64_t)(sa.g.M + BM - 1) / BM + (uint64_t)sa.n_seg) * sa.g.tiles_n;
    if (bound > 0x0fffff00ull) return fail(PP_ERR_UNSUPPORTED, "%s: too many tiles", who);
    const uint32_t grid = ((uint32_t)bound + 7) / 8 * 8;
    hipLaunchKernelGGL((gemm_bf16_seg_gated_kernel<BM, BN, NS, W, FWD>), dim3(grid), dim3(W * 64), lds, st, sa, gu, ld_gu);
    return check_launch("gemm_bf16_seg_gated_kernel");
}

extern "C" int pp_gemm_bf16_segmented_swiglu(const void* x, const void* const* w_gate_of, const void* const* w_up_of,
                                             const int32_t* seg_start, int n_seg, void* gu, void* h, int64_t M,
                                             int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ld_gu,
                                             int64_t ldh, pp_stream stream) {
    const char* who = "pp_gemm_bf16_segmented_swiglu";
    if (!w_gate_of || !w_up_of || !seg_start || n_seg < 1 || n_seg > PP_GEMM_MAX_SEGMENTS)
        return fail(PP_ERR_INVALID, "%s: bad segment list (n_seg=%d)", who, n_seg);
    // the weights are checked for null only: their pointers live in device memory
    int rc = gated_check(who, x, x, M, N, K, ldx, ldw);
    if (rc) return rc;
    if (M == 0 || N == 0) return PP_OK;
    if (!gu || !h) return fail(PP_ERR_INVALID, "%s: null pointer", who);
    if (!aligned(gu, 8) || !aligned(h, 8)) return fail(PP_ERR_INVALID, "%s: misaligned pointer", who);
    if (ld_gu < 2 * N || (ld_gu & 3) || ldh < N || (ldh & 3))
        return fail(PP_ERR_INVALID, "%s: ld_gu >= 2 N and ldh >= N, both multiples of 4", who);
    GatedSegArgs sa;
    fill_args(sa.g, x, nullptr, h, M, N, K, ldx, ldw, ldh);
    sa.seg_start = seg_start;
    sa.w_a = w_gate_of;
    sa.w_b = w_up_of;
    sa.n_seg = n_seg;
    return launch_seg_gated<true>(sa, static_cast<uint16_t*>(gu), ld_gu, static_cast<hipStream_t>(stream), who);
}

extern "C" int pp_gemm_bf16_segmented_dswiglu(const void* dy, const void* const* w_down_t_of, const int32_t* seg_start,
                                              int n_seg, const void* gu, void* dgu, int64_t M, int64_t N, int64_t K,
                                              int64_t ldy, int64_t ldw, int64_t ld_gu, int64_t ld_dgu,
                                              pp_stream stream) {
    const char* who = "pp_gemm_bf16_segmented_dswiglu";
    if (!w_down_t_of || !seg_start || n_seg < 1 || n_seg > PP_GEMM_MAX_SEGMENTS)
        return fail(PP_ERR_INVALID, "%s: bad segment list (n_seg=%d)", who, n_seg);
    int rc = gated_check(who, dy, dy, M, N, K, ldy, ldw);
    if (rc) return rc;
    if (M == 0 || N == 0) return PP_OK;
    if (!gu || !dgu) return fail(PP_ERR_INVALID, "%s: null pointer", who);
    if (!aligned(gu, 8) || !aligned(dgu, 8)) return fail(PP_ERR_INVALID, "%s: misaligned pointer", who);
    if (ld_gu < 2 * N || (ld_gu & 3) || ld_dgu < 2 * N || (ld_dgu & 3))
        return fail(PP_ERR_INVALID, "%s: ld_gu and ld_dgu >= 2 N, multiples of 4", who);
    GatedSegArgs sa;
    fill_args(sa.g, dy, nullptr, dgu, M, N, K, ldy, ldw, ld_dgu);
    sa.seg_start = seg_start;
    sa.w_a = w_down_t_of;
    sa.w_b = nullptr;
    sa.n_seg = n_seg;
    // the kernel reads gu; it is passed through the same parameter as the forward's output
    return launch_seg_gated<false>(sa, const_cast<uint16_t*>(static_cast<const uint16_t*>(gu)), ld_gu,
                                   static_cast<hipStream_t>(stream), who);
}
