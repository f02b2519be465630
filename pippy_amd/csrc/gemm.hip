// bf16 GEMM for gfx950 on v_mfma_f32_32x32x16_bf16 with LDS-staged tiles and fused epilogues.
//
//   C[M,N] = epilogue( sum_k A(m,k) * B(n,k) ),  fp32 accumulation.
//
// Tiling: a work-group of 256 lanes (4 waves) owns a BM x BN output tile and walks K in steps of 64
// (32 for the segmented weight gradients).  The tile shape is chosen per problem so that the grid
// fits the 256 CUs: 128 x 128 by default (waves 2 x 2), 128 x 96 (waves 4 x 1) when that puts a tile
// on more CUs, 128 x 192 when it replaces a full wave of work-groups plus a mostly empty one by a
// single wave, 256 x 256 for very large outputs.  Tiles are staged with direct-to-LDS buffer loads
// (no staging registers, no ds_write):
//   * a k-contiguous operand (memory [rows][ld]) lives in LDS as [row][64 k] with the 16-byte chunk
//     index XOR-swizzled by the row, and fragments are plain ds_read_b128;
//   * a transposed operand (memory [K][ld]: the weight of an input-gradient GEMM, both operands of a
//     weight-gradient GEMM) lives in LDS as it does in memory, [64 k][rows], and fragments come out
//     through ds_read_b64_tr_b16, which transposes 4 k x 16 rows across each 16 lanes.
// The loads of up to 3 tiles are in flight (vmcnt waits leave the younger ones outstanding); the
// single barrier of a tile sits in the middle of its last k16 step, after which the stage it just
// finished is refilled; the LDS reads of a k16 step are interleaved with the MFMAs of the step
// before.  Tiles are visited in bands of 8 tile rows so that an XCD stays on a compact patch of C.
//
// The MFMA is issued with the B fragment as its first operand, so a lane ends up holding, for one
// output row m, groups of 4 consecutive columns n.  The epilogue passes the fp32 accumulators
// through LDS, 32 rows at a time, and comes back with lanes running along n, so that every global
// access of the epilogue (C, bias, auxiliary tensors) covers whole lines.
//
// This file holds the single-problem kernels (with the tile shape chosen per problem), the split along K
// and the segmented kernels; gemm_group.hip the grouped launches; gemm_core.h what they share.
#include "gemm_core.h"
#include <vector>

namespace pp {

template <int BM, int BN, bool AT, bool BT, int NS, int EPI, bool CF32, int KT = BK>
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_dma_kernel(const GemmArgs g) {
    const uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= g.n_blocks) return;
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    gemm_tile_dma<BM, BN, AT, BT, NS, EPI, CF32, KT>(g, tile_m, tile_n);
}

// The same tile on 8 waves (two per SIMD): each wave's part of the tile is half as large, and while one
// wave of a SIMD waits for its fragments or at the barrier the other one's MFMAs run.
template <int BM, int BN, bool AT, bool BT, int NS, int EPI, bool CF32, int KT = BK>
__global__ __launch_bounds__(2 * kGemmThreads) void gemm_bf16_dma8_kernel(const GemmArgs g) {
    const uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= g.n_blocks) return;
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    gemm_tile_dma<BM, BN, AT, BT, NS, EPI, CF32, KT, 0, 8>(g, tile_m, tile_n);
}

// Split along K on 256 x 256 tiles, for an output with few tiles and a long reduction (the input
// gradient of a vocabulary projection: 4096 x 768 with K = 50304).  Large tiles load half as many
// operand bytes per FLOP as 128-wide ones, and the split makes enough of them to fill the CUs.
// Split s of a tile reduces k-tiles [s * kt_per_split, (s + 1) * kt_per_split) into its own fp32
// copy of C in the workspace; splitk_reduce_kernel adds the copies in split order.
__global__ __launch_bounds__(2 * kGemmThreads) void gemm_bf16_splitk_kernel(const GemmArgs g, float* ws, int splits,
                                                                           int kt_per_split) {
    const uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= g.n_blocks * (uint32_t)splits) return;
    const int split = (int)(bid / g.n_blocks);
    uint32_t tile_m, tile_n;
    grouped_tile(bid % g.n_blocks, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    typedef WaveTile<256, 256, 8> WT;  // 8 waves, as the 256 x 256 tiles of the single-problem kernel
    f32x16_t acc[WT::TN][WT::TM];
#pragma unroll
    for (int a = 0; a < WT::TN; ++a)
#pragma unroll
        for (int b = 0; b < WT::TM; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;
    const int nk = (int)((g.K + BK - 1) / BK);
    const int kb = min(nk, split * kt_per_split), ke = min(nk, kb + kt_per_split);
    gemm_mainloop<256, 256, false, false, 2, BK, false, 8>(g, tile_m, tile_n, kb, ke, acc);
    GemmArgs part = g;
    part.C = ws + (size_t)split * (size_t)g.M * (size_t)g.N;
    part.ldc = g.N;
    gemm_epilogue<256, 256, PP_EPI_NONE, true, 0, 8>(part, tile_m, tile_n, acc);
}

// C (bf16) = ws[0] + ws[1] + ... + ws[splits - 1], added in that order; N and ldc multiples of 4.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, int splits, int64_t M,
                                                            int64_t N, uint16_t* __restrict__ C, int64_t ldc) {
    const int64_t n4 = N >> 2;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= M * n4) return;
    const int64_t m = idx / n4, c = (idx - m * n4) << 2;
    const int64_t plane = M * N;
    float4 t = *reinterpret_cast<const float4*>(ws + m * N + c);
    for (int s = 1; s < splits; ++s) {
        const float4 v = *reinterpret_cast<const float4*>(ws + (int64_t)s * plane + m * N + c);
        t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w;
    }
    *reinterpret_cast<uint2*>(C + m * ldc + c) = make_uint2(pack_bf16(t.x, t.y), pack_bf16(t.z, t.w));
}

// Segmented problems: the rows of one operand are partitioned into consecutive segments whose
// bounds seg_start[0 .. n_seg] live in device memory (the token counts of the experts of a
// mixture-of-experts layer), so the sizes are only known on the device and the grid is an upper
// bound.
//   rows mode: segment e is the GEMM of rows [seg_start[e], seg_start[e+1]) of A (and of C and the
//              auxiliary tensors) with its own B = seg_ptr[e];
//   k mode:    segment e reduces over k-rows [seg_start[e], seg_start[e+1]) of transposed A and B
//              into its own C = seg_ptr[e] (an empty segment writes zeros / adds nothing).
struct GemmSegArgs {
    GemmArgs g;  // rows mode: M = total rows, B unused;  k mode: K = total rows, C unused
    const int32_t* seg_start;
    const void* const* seg_ptr;
    int n_seg;
};

template <int BM, int BN, int NS, int EPI>
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_seg_rows_kernel(const GemmSegArgs sa) {
    int e;
    int32_t r0, r1;
    uint32_t tiles_m, bid;
    if (!seg_rows_locate<BM>(sa.seg_start, sa.n_seg, sa.g.tiles_n, &e, &r0, &r1, &tiles_m, &bid)) return;
    GemmArgs g = sa.g;
    g.M = r1 - r0;
    g.A += (int64_t)r0 * g.lda;
    g.B = static_cast<const uint16_t*>(sa.seg_ptr[e]);
    g.C = static_cast<uint16_t*>(g.C) + (int64_t)r0 * g.ldc;
    if (g.aux_in) g.aux_in += (int64_t)r0 * g.ld_aux;
    if (g.aux_out) g.aux_out += (int64_t)r0 * g.ld_aux;
    uint32_t tile_m, tile_n;
    grouped_tile(bid, tiles_m, g.tiles_n, &tile_m, &tile_n);
    gemm_tile_dma<BM, BN, false, false, NS, EPI, false>(g, tile_m, tile_n);
}

template <int BM, int BN, int NS, int EPI, bool CF32>
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_seg_k_kernel(const GemmSegArgs sa) {
    uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    const uint32_t per_seg = sa.g.tiles_m * sa.g.tiles_n;
    if (bid >= per_seg * (uint32_t)sa.n_seg) return;
    const int e = (int)(bid / per_seg);
    bid -= (uint32_t)e * per_seg;
    const int32_t r0 = sa.seg_start[e], r1 = sa.seg_start[e + 1];
    GemmArgs g = sa.g;
    g.K = r1 - r0;
    g.A += (int64_t)r0 * g.lda;
    g.B += (int64_t)r0 * g.ldb;
    g.C = const_cast<void*>(sa.seg_ptr[e]);
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    gemm_tile_dma<BM, BN, true, true, NS, EPI, CF32, 32, 2>(g, tile_m, tile_n);
}

// k mode over several microbatches in one launch: segment e of microbatch m reduces over the rows
// [seg_start_m[e], seg_start_m[e + 1]) of A_m and B_m (every microbatch has its own row partition), and
//   C_e = (beta ? C_e : 0) + g_{e,0} + g_{e,1} + ...   (g rounded to bf16 first when the descriptor says so)
// with the terms added one at a time in ascending m in fp32: bit for bit what one accumulating k-mode
// launch per microbatch leaves.  The running sum stays in registers, so the fp32 accumulators - which
// outweigh the operands of a microbatch by far - move once instead of once per microbatch.
struct GemmSegMultiArgs {
    GemmArgs g;                          // M, N, lda, ldb, ldc, beta, round_bf16; A, B, C, K unused
    const uint16_t* const* a_of;         // [n_mb] device array of the microbatches' A
    const uint16_t* const* b_of;         // [n_mb] ... B
    const int32_t* const* seg_start_of;  // [n_mb] ... row partitions, n_seg + 1 entries each
    const void* const* seg_ptr;          // [n_seg] C_e
    int n_seg, n_mb;
};

template <int BM, int BN, int NS, int KT>
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_seg_k_multi_kernel(const GemmSegMultiArgs sa) {
    uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    const uint32_t per_seg = sa.g.tiles_m * sa.g.tiles_n;
    if (bid >= per_seg * (uint32_t)sa.n_seg) return;
    const int e = (int)(bid / per_seg);
    bid -= (uint32_t)e * per_seg;
    GemmArgs g = sa.g;
    g.C = const_cast<void*>(sa.seg_ptr[e]);
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    typedef WaveTile<BM, BN> WT;
    f32x16_t total[WT::TN][WT::TM], acc[WT::TN][WT::TM];
    if (g.beta) {
        load_c_as_accumulators<BM, BN, 4>(g, tile_m, tile_n, total);
    } else {
#pragma unroll
        for (int a = 0; a < WT::TN; ++a)
#pragma unroll
            for (int b = 0; b < WT::TM; ++b)
#pragma unroll
                for (int q = 0; q < 16; ++q) total[a][b][q] = 0.f;
    }
    for (int m = 0; m < sa.n_mb; ++m) {
        const int32_t* seg = sa.seg_start_of[m];
        const int32_t r0 = seg[e], r1 = seg[e + 1];
        if (r1 <= r0) continue;  // an expert without rows in this microbatch adds nothing
        g.K = r1 - r0;
        g.A = sa.a_of[m] + (int64_t)r0 * g.lda;
        g.B = sa.b_of[m] + (int64_t)r0 * g.ldb;
#pragma unroll
        for (int a = 0; a < WT::TN; ++a)
#pragma unroll
            for (int b = 0; b < WT::TM; ++b)
#pragma unroll
                for (int q = 0; q < 16; ++q) acc[a][b][q] = 0.f;
        gemm_mainloop<BM, BN, true, true, NS, KT>(g, tile_m, tile_n, 0, (int)((g.K + KT - 1) / KT), acc);
#pragma unroll
        for (int a = 0; a < WT::TN; ++a)
#pragma unroll
            for (int b = 0; b < WT::TM; ++b)
#pragma unroll
                for (int q = 0; q < 16; q += 2) {
                    float lo = acc[a][b][q], hi = acc[a][b][q + 1];
                    if (g.round_bf16) {
                        const uint32_t w = pack_bf16(lo, hi);
                        lo = bf16lo(w);
                        hi = bf16hi(w);
                    }
                    total[a][b][q] += lo;
                    total[a][b][q + 1] += hi;
                }
    }
    g.beta = 0;
    g.round_bf16 = 0;
    gemm_epilogue<BM, BN, PP_EPI_NONE, true, 2>(g, tile_m, tile_n, total);
}

// Pipeline depth: with at most one tile per CU a block has the CU to itself and takes 3 stages;
// with more tiles 2 stages leave room for two resident blocks, whose prologues and epilogues overlap
// each other's main loops.

template <int BM, int BN, bool AT, bool BT, int NS, int EPI, bool CF32, int KT = BK>
static int launch_single(const GemmArgs& g, hipStream_t st) {
    constexpr size_t lds = (size_t)NS * (BM + BN) * KT * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_dma_kernel<BM, BN, AT, BT, NS, EPI, CF32, KT>, lds);
    if (attr_rc) return attr_rc;
    const uint32_t grid = (g.n_blocks + 7) / 8 * 8;
    hipLaunchKernelGGL((gemm_bf16_dma_kernel<BM, BN, AT, BT, NS, EPI, CF32, KT>), dim3(grid), dim3(kGemmThreads),
                       lds, st, g);
    return check_launch("gemm_bf16_dma_kernel");
}

template <int BM, int BN, bool AT, bool BT, int NS, int EPI, bool CF32, int KT = BK>
static int launch_single8(const GemmArgs& g, hipStream_t st) {
    constexpr size_t lds = (size_t)NS * (BM + BN) * KT * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_dma8_kernel<BM, BN, AT, BT, NS, EPI, CF32, KT>, lds);
    if (attr_rc) return attr_rc;
    const uint32_t grid = (g.n_blocks + 7) / 8 * 8;
    hipLaunchKernelGGL((gemm_bf16_dma8_kernel<BM, BN, AT, BT, NS, EPI, CF32, KT>), dim3(grid),
                       dim3(2 * kGemmThreads), lds, st, g);
    return check_launch("gemm_bf16_dma8_kernel");
}

template <int BM, int BN, bool AT, bool BT, int EPI, bool CF32>
static int launch_gemm(const GemmArgs* probs, hipStream_t st) {
    {
        if constexpr (EPI == PP_EPI_NONE && !CF32 && BM == 128 && !AT && !BT) {
            // a large output with both operands k-contiguous: 256-row tiles halve the LDS and L2 traffic
            // per MFMA; on 8 waves, so that every SIMD has a second wave to run while the first waits
            // (vocabulary projection 4096 x 50304 x 768: 880 against 840 TFLOP/s on 4 waves and 710 on
            // 128 x 128 tiles; 4096 x 4096 x 1024: 970 against 860)
            GemmArgs big = probs[0];
            const int wide = wide_tile_for(big.M, big.N, true);
            if (wide == 256) {
                int rc = count_tiles<256, 256>(big);
                if (rc) return rc;
                return launch_single8<256, 256, AT, BT, 2, EPI, CF32>(big, st);
            }
            if (wide == 192) {
                int rc = count_tiles<256, 192>(big);
                if (rc) return rc;
                return launch_single8<256, 192, AT, BT, 2, EPI, CF32>(big, st);
            }
        }
        if constexpr (BM == 128 && BN == 128 && !AT && !BT) {
            // an output that leaves CUs idle on 128-wide tiles but fills them on 96-wide ones
            // (4096 x 768: 192 tiles against 256)
            GemmArgs narrow = probs[0];
            const int64_t rows = (narrow.M + 127) / 128;
            const int64_t t128 = rows * ((narrow.N + 127) / 128), t96 = rows * ((narrow.N + 95) / 96);
            if (t128 < kComputeUnits && t96 > t128 && t96 <= kComputeUnits) {
                int rc = count_tiles<128, 96>(narrow);
                if (rc) return rc;
                return launch_single<128, 96, AT, BT, 3, EPI, CF32>(narrow, st);
            }
            // an output that needs a second, mostly empty wave of 128-wide tiles (two work-groups per
            // CU: 512 at once) but fits one wave of 192-wide ones (4096 x 3072: 768 tiles against 512)
            const int64_t t192 = rows * ((narrow.N + 191) / 192);
            if (t128 > 2 * kComputeUnits && t128 < 4 * kComputeUnits && t192 <= 2 * kComputeUnits) {
                int rc = count_tiles<128, 192>(narrow);
                if (rc) return rc;
                return launch_single<128, 192, AT, BT, 2, EPI, CF32>(narrow, st);
            }
        }
        if constexpr (!AT && !BT && !CF32 && (EPI == PP_EPI_NONE || EPI == PP_EPI_BIAS_RESIDUAL)) {
            // a long reduction into an output with at least one 128 x 256 tile per CU (the Llama-sized
            // down and input-gradient projections, 2048 x 4096 with K = 11008 ... 22016): tiles twice as wide
            // on 8 waves load a quarter fewer operand bytes per flop (921 -> 983, 938 -> 1016 TFLOP/s); with
            // K = 4096 the longer prologue and epilogue of the larger tile still outweigh that (1003 -> 930)
            GemmArgs w = probs[0];
            if (w.K >= 8192) {
                int rc = count_tiles<128, 256>(w);
                if (rc) return rc;
                if (w.n_blocks >= kComputeUnits) return launch_single8<128, 256, AT, BT, 3, EPI, CF32>(w, st);
            }
        }
        GemmArgs g = probs[0];
        int rc = count_tiles<BM, BN>(g);
        if (rc) return rc;
        return g.n_blocks <= kComputeUnits ? launch_single<BM, BN, AT, BT, 3, EPI, CF32>(g, st)
                                           : launch_single<BM, BN, AT, BT, 2, EPI, CF32>(g, st);
    }
}

template <int EPI, bool CF32>
static int dispatch_layout(const GemmArgs* g, int at, int bt, hipStream_t st) {
    if (!at && !bt) return launch_gemm<128, 128, false, false, EPI, CF32>(g, st);
    if (!at && bt) return launch_gemm<128, 128, false, true, EPI, CF32>(g, st);
    if (at && !bt) return launch_gemm<128, 128, true, false, EPI, CF32>(g, st);
    return launch_gemm<128, 128, true, true, EPI, CF32>(g, st);
}

int gemm_dispatch_single(const GemmArgs& prob, int at, int bt, int epi, bool cf32, hipStream_t st) {
    const GemmArgs* g = &prob;
    if (epi == PP_EPI_ACCUM_ROUNDED) epi = PP_EPI_ACCUM_F32;  // the same kernels; GemmArgs::round_bf16 is set
    if (cf32) {
        switch (epi) {
            case PP_EPI_NONE: return dispatch_layout<PP_EPI_NONE, true>(g, at, bt, st);
            case PP_EPI_ACCUM_F32: return dispatch_layout<PP_EPI_ACCUM_F32, true>(g, at, bt, st);
            default: return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16: epilogue %d with fp32 C", epi);
        }
    }
    switch (epi) {
        case PP_EPI_NONE: return dispatch_layout<PP_EPI_NONE, false>(g, at, bt, st);
        case PP_EPI_BIAS: return dispatch_layout<PP_EPI_BIAS, false>(g, at, bt, st);
        case PP_EPI_BIAS_GELU_ERF: return dispatch_layout<PP_EPI_BIAS_GELU_ERF, false>(g, at, bt, st);
        case PP_EPI_BIAS_GELU_TANH: return dispatch_layout<PP_EPI_BIAS_GELU_TANH, false>(g, at, bt, st);
        case PP_EPI_BIAS_RESIDUAL: return dispatch_layout<PP_EPI_BIAS_RESIDUAL, false>(g, at, bt, st);
        case PP_EPI_DGELU_ERF: return dispatch_layout<PP_EPI_DGELU_ERF, false>(g, at, bt, st);
        case PP_EPI_DGELU_TANH: return dispatch_layout<PP_EPI_DGELU_TANH, false>(g, at, bt, st);
        case PP_EPI_BIAS_RELU: return dispatch_layout<PP_EPI_BIAS_RELU, false>(g, at, bt, st);
        case PP_EPI_DRELU: return dispatch_layout<PP_EPI_DRELU, false>(g, at, bt, st);
        default: return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16: epilogue %d", epi);
    }
}

template <int EPI>
static int launch_seg_rows(GemmSegArgs& sa, hipStream_t st) {
    constexpr int BM = 128, BN = 128, NS = 2;
    constexpr size_t lds = (size_t)NS * (BM + BN) * BK * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_seg_rows_kernel<BM, BN, NS, EPI>, lds);
    if (attr_rc) return attr_rc;
    sa.g.tiles_n = (uint32_t)((sa.g.N + BN - 1) / BN);
    // every segment may end in a partly filled tile row
    const uint64_t bound = ((uint64_t)(sa.g.M + BM - 1) / BM + (uint64_t)sa.n_seg) * sa.g.tiles_n;
    if (bound > 0x0fffff00ull) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_segmented: too many tiles");
    const uint32_t grid = ((uint32_t)bound + 7) / 8 * 8;
    hipLaunchKernelGGL((gemm_bf16_seg_rows_kernel<BM, BN, NS, EPI>), dim3(grid), dim3(kGemmThreads), lds, st, sa);
    return check_launch("gemm_bf16_seg_rows_kernel");
}

template <int EPI, bool CF32>
static int launch_seg_k(GemmSegArgs& sa, hipStream_t st) {
    constexpr int BM = 128, BN = 128, NS = 2;
    constexpr size_t lds = (size_t)NS * (BM + BN) * 32 * sizeof(uint16_t);  // tiles of 32 k: with about 8 k-tiles per expert, four work-groups per CU cover each other's prologues
    static const int attr_rc = reserve_lds(&gemm_bf16_seg_k_kernel<BM, BN, NS, EPI, CF32>, lds);
    if (attr_rc) return attr_rc;
    int rc = count_tiles<BM, BN>(sa.g);
    if (rc) return rc;
    const uint64_t total = (uint64_t)sa.g.n_blocks * (uint64_t)sa.n_seg;
    if (total > 0x0fffff00ull) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_segmented: too many tiles");
    const uint32_t grid = ((uint32_t)total + 7) / 8 * 8;
    hipLaunchKernelGGL((gemm_bf16_seg_k_kernel<BM, BN, NS, EPI, CF32>), dim3(grid), dim3(kGemmThreads), lds, st, sa);
    return check_launch("gemm_bf16_seg_k_kernel");
}

}  // namespace pp

using namespace pp;

extern "C" int pp_gemm_bf16_segmented(const pp_gemm_desc* d, const int32_t* seg_start,
                                      const void* const* seg_ptr, int n_seg, int mode, pp_stream stream) {
    if (!d || !seg_start || !seg_ptr || n_seg < 1 || n_seg > PP_GEMM_MAX_SEGMENTS)
        return fail(PP_ERR_INVALID, "pp_gemm_bf16_segmented: bad segment list (n_seg=%d)", n_seg);
    if (mode != PP_SEG_ROWS && mode != PP_SEG_K)
        return fail(PP_ERR_INVALID, "pp_gemm_bf16_segmented: unknown mode %d", mode);
    // the operand that every segment brings itself is checked on its first use only for null here:
    // its pointers live in device memory
    pp_gemm_desc dd = *d;
    if (mode == PP_SEG_ROWS) {
        if (dd.a_trans || dd.b_trans)
            return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_segmented: rows mode takes k-contiguous A and B");
        if (dd.epilogue != PP_EPI_NONE && dd.epilogue != PP_EPI_BIAS_RESIDUAL)
            return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_segmented: rows mode epilogue %d", dd.epilogue);
        if (dd.c_dtype != PP_BF16) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_segmented: rows mode writes bf16");
        if (dd.bias) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_segmented: no bias");
        dd.B = dd.A;  // placeholder that passes the checks; the kernel takes B from seg_ptr
    } else {
        if (!dd.a_trans || !dd.b_trans)
            return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_segmented: k mode takes transposed A and B");
        if (!((dd.epilogue == PP_EPI_NONE && dd.c_dtype == PP_BF16) ||
              ((dd.epilogue == PP_EPI_ACCUM_F32 || dd.epilogue == PP_EPI_ACCUM_ROUNDED) && dd.c_dtype == PP_F32)))
            return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_segmented: k mode writes bf16 or accumulates into fp32");
        dd.C = const_cast<void*>(dd.A);
        dd.K = (dd.K + 7) & ~(int64_t)7;  // the reduction length of a segment need not be a multiple of 8
    }
    GemmSegArgs sa;
    bool empty;
    int rc = convert(&dd, &sa.g, &empty);
    if (rc || empty) return rc;
    sa.g.K = (mode == PP_SEG_K) ? d->K : sa.g.K;
    sa.seg_start = seg_start;
    sa.seg_ptr = seg_ptr;
    sa.n_seg = n_seg;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (mode == PP_SEG_ROWS) {
        sa.g.B = nullptr;
        return dd.epilogue == PP_EPI_NONE ? launch_seg_rows<PP_EPI_NONE>(sa, st)
                                          : launch_seg_rows<PP_EPI_BIAS_RESIDUAL>(sa, st);
    }
    sa.g.C = nullptr;
    return dd.c_dtype == PP_F32 ? launch_seg_k<PP_EPI_ACCUM_F32, true>(sa, st)
                                : launch_seg_k<PP_EPI_NONE, false>(sa, st);
}

extern "C" int pp_gemm_bf16_segmented_kseg(const pp_gemm_desc* d, const void* const* a_of, const void* const* b_of,
                                           const int32_t* const* seg_start_of, const void* const* seg_ptr,
                                           int n_seg, int n_mb, pp_stream stream) {
    if (!d || !a_of || !b_of || !seg_start_of || !seg_ptr || n_seg < 1 || n_seg > PP_GEMM_MAX_SEGMENTS ||
        n_mb < 1 || n_mb > PP_GEMM_MAX_KSEG)
        return fail(PP_ERR_INVALID, "pp_gemm_bf16_segmented_kseg: bad lists (n_seg=%d, n_mb=%d)", n_seg, n_mb);
    if (!d->a_trans || !d->b_trans || d->c_dtype != PP_F32 ||
        (d->epilogue != PP_EPI_ACCUM_F32 && d->epilogue != PP_EPI_ACCUM_ROUNDED))
        return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_segmented_kseg: transposed A and B accumulated into fp32 C");
    pp_gemm_desc dd = *d;
    // operands and outputs live behind device arrays: placeholders that pass the checks of a single product
    dd.A = dd.B = reinterpret_cast<const void*>(uintptr_t(16));
    dd.C = reinterpret_cast<void*>(uintptr_t(16));
    dd.K = 8;
    GemmSegMultiArgs sa;
    bool empty;
    int rc = convert(&dd, &sa.g, &empty);
    if (rc || empty) return rc;
    sa.g.A = sa.g.B = nullptr;
    sa.g.C = nullptr;
    sa.a_of = reinterpret_cast<const uint16_t* const*>(a_of);
    sa.b_of = reinterpret_cast<const uint16_t* const*>(b_of);
    sa.seg_start_of = seg_start_of;
    sa.seg_ptr = seg_ptr;
    sa.n_seg = n_seg;
    sa.n_mb = n_mb;
    // 64-deep k-tiles (the single-microbatch kernel takes 32-deep ones so that four work-groups share a CU;
    // this one holds two sets of accumulators, fits two, and its loop over the microbatches is long enough
    // to pay for the deeper tiles: 51.3 against 53.6 ms per Mixtral-style step)
    constexpr int BM = 128, BN = 128, NS = 2, KT = 64;
    constexpr size_t lds = (size_t)NS * (BM + BN) * KT * sizeof(uint16_t) < (size_t)4 * 32 * 64 * 4
                               ? (size_t)4 * 32 * 64 * 4 : (size_t)NS * (BM + BN) * KT * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_seg_k_multi_kernel<BM, BN, NS, KT>, lds);
    if (attr_rc) return attr_rc;
    rc = count_tiles<BM, BN>(sa.g);
    if (rc) return rc;
    const uint64_t total = (uint64_t)sa.g.n_blocks * (uint64_t)n_seg;
    if (total > 0x0fffff00ull) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_segmented_kseg: too many tiles");
    const uint32_t grid = ((uint32_t)total + 7) / 8 * 8;
    hipLaunchKernelGGL((gemm_bf16_seg_k_multi_kernel<BM, BN, NS, KT>), dim3(grid), dim3(kGemmThreads), lds,
                       static_cast<hipStream_t>(stream), sa);
    return check_launch("gemm_bf16_seg_k_multi_kernel");
}

extern "C" int pp_gemm_bf16(const pp_gemm_desc* d, pp_stream stream) {
    GemmArgs g;
    bool empty;
    int rc = convert(d, &g, &empty);
    if (rc || empty) return rc;
    return gemm_dispatch_single(g, d->a_trans ? 1 : 0, d->b_trans ? 1 : 0, d->epilogue, d->c_dtype == PP_F32,
                                static_cast<hipStream_t>(stream));
}

// Number of k-splits on 256 x 256 tiles that pays for this problem, or 0: k-contiguous operands, a
// plain bf16 C, at most a quarter of a wave of such tiles and at least 64 k-tiles left per split.
static int splitk_plan(const pp_gemm_desc* d, int64_t workspace_elems, int* kt_per_split) {
    if (d->a_trans || d->b_trans || d->epilogue != PP_EPI_NONE || d->c_dtype != PP_BF16) return 0;
    if ((d->N & 3) || (d->ldc & 3) || !aligned(d->C, 8)) return 0;
    const int64_t tiles = ((d->M + 255) / 256) * ((d->N + 255) / 256);
    const int64_t nk = (d->K + BK - 1) / BK;
    if (tiles <= 0 || tiles > kComputeUnits / 4) return 0;  // 2048 x 4096 x 11008 (128 tiles) is faster unsplit
    int64_t splits = kComputeUnits / tiles;
    if (splits > nk / 64) splits = nk / 64;
    if (splits > 8) splits = 8;
    if (splits > workspace_elems / (d->M * d->N)) splits = workspace_elems / (d->M * d->N);
    if (splits < 2) return 0;
    *kt_per_split = (int)((nk + splits - 1) / splits);
    return (int)splits;
}

extern "C" int pp_gemm_bf16_splitk(const pp_gemm_desc* d, float* workspace, int64_t workspace_elems,
                                   pp_stream stream) {
    GemmArgs g;
    bool empty;
    int rc = convert(d, &g, &empty);
    if (rc || empty) return rc;
    int kt_per_split = 0;
    // the column sums of an activation-derivative epilogue are formed by the single-launch epilogue only
    const int splits = (workspace && aligned(workspace, 16) && !g.colsum) ? splitk_plan(d, workspace_elems, &kt_per_split) : 0;
    if (!splits) return pp_gemm_bf16(d, stream);
    rc = count_tiles<256, 256>(g);
    if (rc) return rc;
    constexpr size_t lds = (size_t)2 * (256 + 256) * BK * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_splitk_kernel, lds);
    if (attr_rc) return attr_rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t grid = (g.n_blocks * (uint32_t)splits + 7) / 8 * 8;
    hipLaunchKernelGGL(gemm_bf16_splitk_kernel, dim3(grid), dim3(2 * kGemmThreads), lds, st, g, workspace, splits,
                       kt_per_split);
    rc = check_launch("gemm_bf16_splitk_kernel");
    if (rc) return rc;
    const int64_t quads = g.M * (g.N >> 2);
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((uint32_t)((quads + 255) / 256)), dim3(256), 0, st, workspace,
                       splits, g.M, g.N, static_cast<uint16_t*>(g.C), g.ldc);
    return check_launch("splitk_reduce_kernel");
}
