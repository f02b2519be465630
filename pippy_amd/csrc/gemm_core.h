// Building blocks shared by the bf16 GEMM kernels: argument block, epilogue, main loop, one whole tile,
// the grouped kernel, and the host-side checks of a descriptor.
#pragma once
#include "tile.h"
#include "act_math.h"
#include <type_traits>
#include <vector>

namespace pp {

struct GemmArgs {
    const uint16_t* A;
    const uint16_t* B;
    const uint16_t* B2;  // second k-contiguous operand of a kernel that computes two products per tile
    void* C;
    int64_t M, N, K, lda, ldb, ldc;
    const uint16_t* bias;
    const uint16_t* aux_in;
    uint16_t* aux_out;
    int64_t ld_aux;
    int beta;
    int round_bf16;  // fp32 C: round the sums to bf16 before they are stored or added
    int epi;         // the problem's epilogue, for kernels that take it at run time (kEpiRuntime)
    uint32_t tiles_m, tiles_n, n_blocks;
    // activation-derivative epilogues: fp32 [ceil(M / 32)][N], the column sums of every band of 32 rows of C
    // as stored (what the bias gradient of the layer in front of the activation is the sum of), or null
    float* colsum = nullptr;
};
__host__ __device__ constexpr bool epi_may_sum_columns(int epi) {
    return epi == PP_EPI_DGELU_ERF || epi == PP_EPI_DGELU_TANH || epi == PP_EPI_DRELU;
}

// Template value of EPI for kernels whose problems bring their own epilogue (GemmArgs::epi): the
// grouped launches of problems that differ in it.  Only for a bf16 C.
constexpr int kEpiRuntime = -1;
// Unroll factor of the per-pass loops of the epilogue: everything (a factor beyond any trip count) for
// a compile-time epilogue, none for the kernel that holds the arithmetic of all of them.
template <int EPI>
struct EpiUnroll {
    static constexpr int value = EPI == kEpiRuntime ? 1 : 64;
};
template <int EPI>
__device__ __forceinline__ int epi_of(const GemmArgs& g) {
    return EPI == kEpiRuntime ? g.epi : EPI;
}

__host__ __device__ constexpr bool epi_has_bias(int epi) {
    return epi == PP_EPI_BIAS || epi == PP_EPI_BIAS_GELU_ERF || epi == PP_EPI_BIAS_GELU_TANH ||
           epi == PP_EPI_BIAS_RESIDUAL || epi == PP_EPI_BIAS_RELU;
}
__host__ __device__ constexpr bool epi_reads_aux(int epi) {
    return epi == PP_EPI_BIAS_RESIDUAL || epi == PP_EPI_DGELU_ERF || epi == PP_EPI_DGELU_TANH ||
           epi == PP_EPI_DRELU;
}
__host__ __device__ constexpr bool epi_is_gelu(int epi) { return epi == PP_EPI_BIAS_GELU_ERF || epi == PP_EPI_BIAS_GELU_TANH; }

// The bias of 4 consecutive columns starting at n0 (zero past N or without a bias).
template <int EPI>
__device__ __forceinline__ void load_bias4(const GemmArgs& g, int64_t n0, float (&bias)[4]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) bias[e] = 0.f;
    if (!epi_has_bias(epi_of<EPI>(g)) || !g.bias || n0 >= g.N) return;
    if (n0 + 3 < g.N && aligned(g.bias + n0, 8)) {
        const uint2 w = *reinterpret_cast<const uint2*>(g.bias + n0);
        bias[0] = bf16lo(w.x); bias[1] = bf16hi(w.x); bias[2] = bf16lo(w.y); bias[3] = bf16hi(w.y);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (n0 + e < g.N) bias[e] = bf16_to_f32(g.bias[n0 + e]);
    }
}

// The arithmetic of the epilogue on 4 values: v becomes the output, pre the value before the
// activation (what a GELU epilogue saves for the backward pass).
// `epi_rt` is the problem's own epilogue, used when EPI is kEpiRuntime (the branches below are then
// uniform run-time branches instead of compile-time ones).
template <int EPI>
__device__ __forceinline__ void epilogue_math4(float (&v)[4], float (&pre)[4], const float (&bias)[4],
                                               const float (&a)[4], int epi_rt) {
    const int epi = EPI == kEpiRuntime ? epi_rt : EPI;
    if (epi_has_bias(epi)) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += bias[e];
    }
    if (epi == PP_EPI_BIAS_RESIDUAL) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += a[e];
    } else if (epi == PP_EPI_DGELU_ERF) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] *= dgelu_erf(a[e]);
    } else if (epi == PP_EPI_DGELU_TANH) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] *= dgelu_tanh(a[e]);
    } else if (epi == PP_EPI_DRELU) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = a[e] > 0.f ? v[e] : 0.f;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) pre[e] = v[e];
    if (epi == PP_EPI_BIAS_GELU_ERF) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = gelu_erf(v[e]);
    } else if (epi == PP_EPI_BIAS_GELU_TANH) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = gelu_tanh(v[e]);
    } else if (epi == PP_EPI_BIAS_RELU) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = fmaxf(v[e], 0.f);
    }
}

// Applies the epilogue to 4 consecutive columns n0..n0+3 of row m and stores them; handles rows
// and columns past the edge of C and unaligned operands.
template <int EPI, bool CF32>
__device__ __forceinline__ void epilogue4(const GemmArgs& g, int64_t m, int64_t n0, float v0, float v1,
                                          float v2, float v3, const float (&bias)[4], bool vec_ok,
                                          float* colsum4 = nullptr) {
    if (m >= g.M || n0 >= g.N) return;
    float v[4] = {v0, v1, v2, v3}, pre[4];
    const int nv = (g.N - n0 >= 4) ? 4 : (int)(g.N - n0);
    const bool full = vec_ok && nv == 4;

    const int epi = epi_of<EPI>(g);
    float a[4] = {0.f, 0.f, 0.f, 0.f};
    if (epi_reads_aux(epi)) {
        const uint16_t* ap = g.aux_in + m * g.ld_aux + n0;
        if (full) {
            const uint2 w = *reinterpret_cast<const uint2*>(ap);
            a[0] = bf16lo(w.x); a[1] = bf16hi(w.x); a[2] = bf16lo(w.y); a[3] = bf16hi(w.y);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (e < nv) a[e] = bf16_to_f32(ap[e]);
        }
    }
    epilogue_math4<EPI>(v, pre, bias, a, epi);
    if (epi_is_gelu(epi) && g.aux_out) {
        uint16_t* op = g.aux_out + m * g.ld_aux + n0;
        if (full) {
            *reinterpret_cast<uint2*>(op) = make_uint2(pack_bf16(pre[0], pre[1]), pack_bf16(pre[2], pre[3]));
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (e < nv) op[e] = f32_to_bf16(pre[e]);
        }
    }

    if (CF32) {
        float* cp = static_cast<float*>(g.C) + m * g.ldc + n0;
        if (EPI == PP_EPI_ACCUM_F32 && g.round_bf16) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = bf16_to_f32(f32_to_bf16(v[e]));
        }
        if (EPI == PP_EPI_ACCUM_F32 && g.beta) {
            if (full) {
                const float4 old = *reinterpret_cast<const float4*>(cp);
                *reinterpret_cast<float4*>(cp) =
                    make_float4(old.x + v[0], old.y + v[1], old.z + v[2], old.w + v[3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (e < nv) cp[e] += v[e];
            }
        } else {
            if (full) {
                *reinterpret_cast<float4*>(cp) = make_float4(v[0], v[1], v[2], v[3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (e < nv) cp[e] = v[e];
            }
        }
    } else {
        uint16_t* cp = static_cast<uint16_t*>(g.C) + m * g.ldc + n0;
        if (colsum4) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (e < nv) colsum4[e] += bf16_to_f32(f32_to_bf16(v[e]));
        }
        if (full) {
            *reinterpret_cast<uint2*>(cp) = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (e < nv) cp[e] = f32_to_bf16(v[e]);
        }
    }
}

// ---- the kernel -----------------------------------------------------------------------------
extern __shared__ __attribute__((aligned(16))) uint16_t smem[];

// Tile order of the direct-to-LDS kernels: bands of kGroupM tile rows, walked m-fastest, so that
// the tiles resident on an XCD at one time share few A and B panels.
constexpr uint32_t kGroupM = 8;
__device__ __forceinline__ void grouped_tile(uint32_t bid, uint32_t tiles_m, uint32_t tiles_n,
                                             uint32_t* tile_m, uint32_t* tile_n) {
    const uint32_t per_group = kGroupM * tiles_n;
    const uint32_t grp = bid / per_group, rem = bid % per_group;
    const uint32_t rows = min(kGroupM, tiles_m - grp * kGroupM);
    *tile_m = grp * kGroupM + rem % rows;
    *tile_n = rem / rows;
}

// Scheduling hint for one k16 step: R LDS reads (the fragments of the next step) spread evenly
// between M MFMAs.  (Issuing all reads right after the first MFMA, with the tile's barrier at the
// start of its last step, measured slower on the transformer shapes: 41.0 against 38.6 ms of GEMM
// time per GPT-2-small step.)
template <int R, int M, int I>
__device__ __forceinline__ void interleave_reads() {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, R * (I + 1) / M - R * I / M, 0);
    if constexpr (I + 1 < M) interleave_reads<R, M, I + 1>();
}

// How the W waves of a work-group share a BM x BN tile: two columns of waves when BN is a multiple of
// 64 (4 waves: 2 x 2, 8 waves: 4 x 2), else one (a 128 x 96 tile: each of 4 waves 32 rows by 96
// columns).  A wave's part is TM x TN MFMA tiles of 32 x 32.
template <int BM, int BN, int W = 4>
struct WaveTile {
    static constexpr int WGN = (BN % 64 == 0) ? 2 : 1;
    static constexpr int WGM = W / WGN;
    static constexpr int WTM = BM / WGM, WTN = BN / WGN;
    static constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "a wave's part of the tile is made of 32 x 32 MFMA tiles");
};

// Main loop of one BM x BN output tile over the k-tiles [kt_begin, kt_end) of KT values each, through
// NS LDS stages filled by direct-to-LDS loads; the products are added to acc.  Starts with a barrier,
// so that it may follow an epilogue (or another main loop) that used the same LDS.
// DUAL: the BN rows of the B tile are BN / 2 rows of g.B followed by the same BN / 2 rows of g.B2, so
// that one tile holds two products of the same A rows (tile_n then counts blocks of BN / 2 rows).
template <int BM, int BN, bool AT, bool BT, int NS, int KT, bool DUAL = false, int W = 4>
__device__ __forceinline__ void gemm_mainloop(const GemmArgs& g, uint32_t tile_m, uint32_t tile_n, int kt_begin,
                                              int kt_end,
                                              f32x16_t (&acc)[WaveTile<BM, BN, W>::TN][WaveTile<BM, BN, W>::TM]) {
    typedef WaveTile<BM, BN, W> WT;
    constexpr int WTM = WT::WTM, WTN = WT::WTN, TM = WT::TM, TN = WT::TN;
    constexpr int KS = KT / 16;  // MFMA k-steps per tile
    constexpr int kStageElems = (BM + BN) * KT;
    // loads per tile per wave (the two half loaders of a DUAL tile issue as many as one whole loader)
    constexpr int LPT = DmaStage<BM, AT, KT, W>::kLoads + DmaStage<BN, BT, KT, W>::kLoads;
    constexpr int kReadsPerStep = TM * FragReader<BM, AT, KT>::kReads + TN * FragReader<BN, BT, KT>::kReads;
    static_assert(NS >= 2 && NS <= 4 && (NS - 1) * LPT < 64, "pipeline depth exceeds vmcnt");
    static_assert(KS >= 2 && TN >= 2, "the last k-step is split in two parts around the barrier");
    static_assert(NS * kStageElems * 2 >= W * 32 * WTN * 4, "the epilogue stages fp32 bands in the tile memory");
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave % WT::WGM) * WTM, wn0 = (wave / WT::WGM) * WTN;

    constexpr int BNL = DUAL ? BN / 2 : BN;  // rows that one loader of B brings
    static_assert(!DUAL || (!AT && !BT), "two products per tile: k-contiguous operands");
    DmaStage<BM, AT, KT, W> sa;
    DmaStage<BNL, BT, KT, W> sb, sb2;
    sa.init(g.A, g.lda, m0, g.M, g.K, wave, lane);
    sb.init(g.B, g.ldb, DUAL ? n0 / 2 : n0, g.N, g.K, wave, lane);
    if (DUAL) sb2.init(g.B2, g.ldb, n0 / 2, g.N, g.K, wave, lane);
    const int nk = kt_end - kt_begin;
    auto issue = [&](int stage, int kt) {
        sa.load(smem + stage * kStageElems, (kt_begin + kt) * KT, wave);
        sb.load(smem + stage * kStageElems + BM * KT, (kt_begin + kt) * KT, wave);
        if (DUAL) sb2.load(smem + stage * kStageElems + (BM + BNL) * KT, (kt_begin + kt) * KT, wave);
    };

    FragReader<BM, AT, KT> ra[TM];
    FragReader<BN, BT, KT> rb[TN];
#pragma unroll
    for (int t = 0; t < TM; ++t) ra[t].init(wm0 + t * 32, lane);
    // DUAL: the first half of a wave's accumulator tiles is its columns of the first product, the second
    // half the same columns of the second product (rows BN / 2 ... of the B tile)
    static_assert(!DUAL || TN % 2 == 0, "two products per tile: an even number of accumulator tiles per wave");
#pragma unroll
    for (int t = 0; t < TN; ++t)
        rb[t].init(DUAL ? (t < TN / 2 ? 0 : BN / 2) + wn0 / 2 + (t % (TN / 2 > 0 ? TN / 2 : 1)) * 32 : wn0 + t * 32, lane);
    bf16x8_t fa[2][TM], fb[2][TN];
    auto read_frags = [&](int sel, const uint16_t* st, int ks) {
#pragma unroll
        for (int t = 0; t < TM; ++t) fa[sel][t] = ra[t].read(st, ks);
#pragma unroll
        for (int t = 0; t < TN; ++t) fb[sel][t] = rb[t].read(st + BM * KT, ks);
    };
    auto mma = [&](int sel, int a_lo, int a_hi) {
#pragma unroll
        for (int a = a_lo; a < a_hi; ++a)
#pragma unroll
            for (int b = 0; b < TM; ++b) {
                acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[sel][a], fa[sel][b], acc[a][b], 0, 0, 0);
            }
    };
    auto interleave = [&]() { interleave_reads<kReadsPerStep, TM * TN, 0>(); };

    // prologue: tiles 0 .. NS-1 in flight, tile 0 awaited
    wait_lds();
    __builtin_amdgcn_s_barrier();  // whatever used the stages before is done with them
#pragma unroll
    for (int t = 0; t < NS; ++t)
        if (t < nk) issue(t, t);
    if (nk >= NS) wait_vmcnt<(NS - 1) * LPT>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    read_frags(0, smem, 0);

    int stage = 0;
    constexpr int kLast = (KS - 1) & 1;  // fragment set of a tile's last k-step
    for (int kt = 0; kt < nk; ++kt) {
        const uint16_t* st = smem + stage * kStageElems;
#pragma unroll
        for (int ks = 1; ks < KS; ++ks) {
            read_frags(ks & 1, st, ks);
            mma((ks - 1) & 1, 0, TN);
            interleave();
        }
        mma(kLast, 0, TN / 2);
        // tile kt+1 must have landed; tiles kt+2 .. kt+NS-1 may stay in flight
        const int ahead = nk - 2 - kt;
        if (NS >= 4 && ahead >= 2) wait_vmcnt<(NS >= 4 ? 2 : 0) * LPT>();
        else if (NS >= 3 && ahead >= 1) wait_vmcnt<(NS >= 3 ? 1 : 0) * LPT>();
        else wait_vmcnt<0>();
        wait_lds();  // this wave's reads of the current stage are done: the stage may be refilled
        __builtin_amdgcn_s_barrier();
        if (kt + NS < nk) issue(stage, kt + NS);
        stage = stage + 1 == NS ? 0 : stage + 1;
        if (kt + 1 < nk) read_frags(0, smem + stage * kStageElems, 0);
        mma(kLast, TN / 2, TN);
    }
}

// Epilogue of one BM x BN tile: one band of 32 rows at a time goes through a wave-private LDS region
// as fp32, [32][WTN] with the 16-byte unit index XORed by the row, and comes back with lanes running
// along n, so that epilogue4 reads and writes whole lines.
template <int BM, int BN, int EPI, bool CF32, int EB = 0, int W = 4>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& g, uint32_t tile_m, uint32_t tile_n,
                                              f32x16_t (&acc)[WaveTile<BM, BN, W>::TN][WaveTile<BM, BN, W>::TM]) {
    typedef WaveTile<BM, BN, W> WT;
    constexpr int WTM = WT::WTM, WTN = WT::WTN, TM = WT::TM, TN = WT::TN;
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave % WT::WGM) * WTM, wn0 = (wave / WT::WGM) * WTN;
    wait_lds();
    __builtin_amdgcn_s_barrier();  // every wave is done with the stages
    const int l32 = lane & 31, lh = lane >> 5;
    float* cw = reinterpret_cast<float*>(smem) + wave * (32 * WTN);
    constexpr int UPR = WTN / 4;   // 16-byte units per row
    constexpr int RPP = 64 / UPR;  // rows per pass of the wave
    static_assert(UPR % 8 == 0 && 32 % RPP == 0, "the unit swizzle works on groups of 8 units");
    // With 24 units per row (96 columns) two rows fill 48 lanes of a pass and 16 lanes sit out.
    const bool lane_on = lane < RPP * UPR;
    const int ru = lane % UPR, rr = lane / UPR;
    // unit u of row r lives at unit (u with its low 3 bits XORed by r) when UPR is not a power of two
    auto unit_at = [](int u, int r) {
        return (UPR & (UPR - 1)) == 0 ? (u ^ (r & (UPR - 1))) : ((u & ~7) | ((u ^ r) & 7));
    };
    const bool vec_ok = CF32 ? ((g.ldc & 3) == 0 && aligned(g.C, 16))
                             : ((g.ldc & 3) == 0 && aligned(g.C, 8) && (g.ld_aux & 3) == 0 &&
                                aligned(g.aux_in, 8) && aligned(g.aux_out, 8));
    const int64_t gn = n0 + wn0 + ru * 4;  // this lane's 4 columns, the same in every pass
    const int epi = epi_of<EPI>(g);
    float bias[4];
    load_bias4<EPI>(g, gn, bias);
    // a tile in the interior of C with aligned operands takes the path without bounds checks, in
    // which the loads of a band (LDS, auxiliary tensor, old C) are issued before any arithmetic
    const bool interior = vec_ok && m0 + BM <= g.M && n0 + BN <= g.N;
    constexpr int kPasses = 32 / RPP;
    // EB passes at a time (all of them by default): fewer values in flight for a kernel that counts
    // on many resident waves rather than on long runs of independent loads
    constexpr int kBatch = EB > 0 && EB < kPasses ? EB : kPasses;
    static_assert(kPasses % kBatch == 0, "the passes of a band split into whole batches");
    // a kernel that carries every epilogue keeps one copy of their arithmetic per band: its batches
    // run as a loop, see EpiUnroll (the bands themselves are unrolled by construction, they index the
    // accumulators)
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
        const int64_t gm = m0 + wm0 + b * 32 + rr;  // row of pass 0; pass i adds i * RPP
        constexpr bool kMaySum = !CF32 && (EPI == kEpiRuntime || epi_may_sum_columns(EPI));
        const bool sums = kMaySum && g.colsum && epi_may_sum_columns(epi);
        float cs[4] = {0.f, 0.f, 0.f, 0.f};  // this lane's rows of the band, its 4 columns
        if (interior && lane_on) {
#pragma unroll EpiUnroll<EPI>::value
          for (int i0 = 0; i0 < kPasses; i0 += kBatch) {
            float4 v4[kBatch];
            uint2 aw[kBatch];
            float4 old[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                const int m = (i0 + j) * RPP + rr;
                v4[j] = *reinterpret_cast<const float4*>(cw + m * WTN + (unit_at(ru, m) << 2));
            }
            if (epi_reads_aux(epi)) {
#pragma unroll
                for (int j = 0; j < kBatch; ++j)
                    aw[j] = *reinterpret_cast<const uint2*>(g.aux_in + (gm + (i0 + j) * RPP) * g.ld_aux + gn);
            }
            if (CF32 && EPI == PP_EPI_ACCUM_F32 && g.beta) {
#pragma unroll
                for (int j = 0; j < kBatch; ++j)
                    old[j] = *reinterpret_cast<const float4*>(static_cast<const float*>(g.C) +
                                                              (gm + (i0 + j) * RPP) * g.ldc + gn);
            }
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                float v[4] = {v4[j].x, v4[j].y, v4[j].z, v4[j].w}, pre[4];
                float av[4] = {0.f, 0.f, 0.f, 0.f};
                if (epi_reads_aux(epi)) {
                    av[0] = bf16lo(aw[j].x); av[1] = bf16hi(aw[j].x); av[2] = bf16lo(aw[j].y); av[3] = bf16hi(aw[j].y);
                }
                epilogue_math4<EPI>(v, pre, bias, av, epi);
                const int64_t row = gm + (i0 + j) * RPP;
                if (epi_is_gelu(epi) && g.aux_out)
                    *reinterpret_cast<uint2*>(g.aux_out + row * g.ld_aux + gn) =
                        make_uint2(pack_bf16(pre[0], pre[1]), pack_bf16(pre[2], pre[3]));
                if (CF32) {
                    float* cp = static_cast<float*>(g.C) + row * g.ldc + gn;
                    if (EPI == PP_EPI_ACCUM_F32 && g.round_bf16) {
                        const uint32_t w0 = pack_bf16(v[0], v[1]), w1 = pack_bf16(v[2], v[3]);
                        v[0] = bf16lo(w0); v[1] = bf16hi(w0); v[2] = bf16lo(w1); v[3] = bf16hi(w1);
                    }
                    if (EPI == PP_EPI_ACCUM_F32 && g.beta)
                        *reinterpret_cast<float4*>(cp) = make_float4(old[j].x + v[0], old[j].y + v[1], old[j].z + v[2], old[j].w + v[3]);
                    else
                        *reinterpret_cast<float4*>(cp) = make_float4(v[0], v[1], v[2], v[3]);
                } else {
                    const uint32_t w0 = pack_bf16(v[0], v[1]), w1 = pack_bf16(v[2], v[3]);
                    *reinterpret_cast<uint2*>(static_cast<uint16_t*>(g.C) + row * g.ldc + gn) = make_uint2(w0, w1);
                    if (kMaySum && sums) {
                        cs[0] += bf16lo(w0); cs[1] += bf16hi(w0); cs[2] += bf16lo(w1); cs[3] += bf16hi(w1);
                    }
                }
            }
          }
        } else if (lane_on) {
#pragma unroll EpiUnroll<EPI>::value
            for (int i = 0; i < kPasses; ++i) {
                const int m = i * RPP + rr;
                const float4 v = *reinterpret_cast<const float4*>(cw + m * WTN + (unit_at(ru, m) << 2));
                epilogue4<EPI, CF32>(g, gm + i * RPP, gn, v.x, v.y, v.z, v.w, bias, vec_ok,
                                     kMaySum && sums ? cs : nullptr);
            }
        }
        if (kMaySum && sums) {
            // the RPP lanes that share these 4 columns, added in row order; the first of them writes
            float t[4] = {cs[0], cs[1], cs[2], cs[3]};
#pragma unroll
            for (int r = 1; r < RPP; ++r)
#pragma unroll
                for (int e = 0; e < 4; ++e) t[e] += __shfl(cs[e], ru + r * UPR, 64);
            const int64_t band_row = m0 + wm0 + b * 32;
            if (lane < UPR && band_row < g.M) {
                float* out = g.colsum + (band_row >> 5) * g.N + gn;
                if (gn + 3 < g.N && aligned(out, 16)) {
                    *reinterpret_cast<float4*>(out) = make_float4(t[0], t[1], t[2], t[3]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (gn + e < g.N) out[e] = t[e];
                }
            }
        }
    });
}

// The BM x BN tile of an fp32 C in the accumulator layout of the main loop (the running sum of a kernel
// that adds several products to C in registers).
template <int BM, int BN, int W>
__device__ __forceinline__ void load_c_as_accumulators(const GemmArgs& g, uint32_t tile_m, uint32_t tile_n,
                                                       f32x16_t (&t)[WaveTile<BM, BN, W>::TN][WaveTile<BM, BN, W>::TM]) {
    typedef WaveTile<BM, BN, W> WT;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    const int64_t m_base = (int64_t)tile_m * BM + (wave % WT::WGM) * WT::WTM + l32;
    const int64_t n_base = (int64_t)tile_n * BN + (wave / WT::WGM) * WT::WTN + 4 * lh;
    const float* C = static_cast<const float*>(g.C);
    const bool vec_ok = (g.ldc & 3) == 0 && aligned(g.C, 16);
#pragma unroll
    for (int a = 0; a < WT::TN; ++a)
#pragma unroll
        for (int b = 0; b < WT::TM; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                // the accumulator layout of v_mfma_f32_32x32x16 with B as the first operand: a lane holds,
                // for one row, four groups of four consecutive columns
                const int64_t m = m_base + b * 32, n = n_base + a * 32 + 8 * q;
                float v[4] = {0.f, 0.f, 0.f, 0.f};
                if (m < g.M) {
                    if (vec_ok && n + 3 < g.N) {
                        const float4 w = *reinterpret_cast<const float4*>(C + m * g.ldc + n);
                        v[0] = w.x; v[1] = w.y; v[2] = w.z; v[3] = w.w;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (n + e < g.N) v[e] = C[m * g.ldc + n + e];
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) t[a][b][4 * q + e] = v[e];
            }
}

// One whole output tile: main loop over all of K, then the epilogue.
template <int BM, int BN, bool AT, bool BT, int NS, int EPI, bool CF32, int KT = BK, int EB = 0, int W = 4>
__device__ __forceinline__ void gemm_tile_dma(const GemmArgs& g, uint32_t tile_m, uint32_t tile_n) {
    f32x16_t acc[WaveTile<BM, BN, W>::TN][WaveTile<BM, BN, W>::TM];
#pragma unroll
    for (int a = 0; a < WaveTile<BM, BN, W>::TN; ++a)
#pragma unroll
        for (int b = 0; b < WaveTile<BM, BN, W>::TM; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;
    gemm_mainloop<BM, BN, AT, BT, NS, KT, false, W>(g, tile_m, tile_n, 0, (int)((g.K + KT - 1) / KT), acc);
    gemm_epilogue<BM, BN, EPI, CF32, EB, W>(g, tile_m, tile_n, acc);
}


// Several independent problems in one grid: the tiles of problem i are the block ids
// [tile_start[i], tile_start[i + 1]).
struct GemmGroupArgs {
    GemmArgs p[PP_GEMM_MAX_GROUP];
    uint32_t tile_start[PP_GEMM_MAX_GROUP + 1];
    int n;
};

template <int BM, int BN, bool AT, bool BT, int NS, int EPI, bool CF32, int KT = BK, int W = 4>
__global__ __launch_bounds__(W * 64) void gemm_bf16_group_kernel(const GemmGroupArgs ga) {
    uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= ga.tile_start[ga.n]) return;
    int i = 0;
    while (i + 1 < ga.n && bid >= ga.tile_start[i + 1]) ++i;
    bid -= ga.tile_start[i];
    const GemmArgs& g = ga.p[i];
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    gemm_tile_dma<BM, BN, AT, BT, NS, EPI, CF32, KT, 0, W>(g, tile_m, tile_n);
}


template <typename Kernel>
static inline int reserve_lds(Kernel kernel, size_t lds) {
    const hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (rc != hipSuccess)
        return fail(PP_ERR_LAUNCH, "pp_gemm_bf16: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(rc));
    return PP_OK;
}

template <int BM, int BN>
static inline int count_tiles(GemmArgs& g) {
    g.tiles_m = (uint32_t)((g.M + BM - 1) / BM);
    g.tiles_n = (uint32_t)((g.N + BN - 1) / BN);
    const uint64_t nb = (uint64_t)g.tiles_m * g.tiles_n;
    if (nb > 0x0fffff00ull) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16: too many tiles");
    g.n_blocks = (uint32_t)nb;
    return PP_OK;
}


// The tile of a rows-segmented launch: the rows of A are partitioned into n_seg consecutive segments whose
// bounds seg_start[0 .. n_seg] live in device memory; every segment has its own ceil(rows / BM) x tiles_n
// tiles, numbered segment after segment, and the grid is an upper bound.  Finds the segment e, its rows
// [r0, r1), its tiles_m and the tile's number inside it for this work-group; false when the work-group has
// no tile.  The ids that exist are renumbered XCD-contiguously.
template <int BM>
__device__ __forceinline__ bool seg_rows_locate(const int32_t* seg_start, int n_seg, uint32_t tiles_n, int* e_out,
                                                int32_t* r0_out, int32_t* r1_out, uint32_t* tiles_m_out,
                                                uint32_t* bid_out) {
    int e = 0;
    int32_t r0, r1;
    uint32_t tiles_m, bid;
    if (n_seg < 64) {
        // one vector load of the bounds (lane l holds segment l) and a prefix sum over the lanes,
        // instead of a chain of dependent scalar loads that would cost as much as a third of a tile
        const int lane = threadIdx.x & 63;
        const int32_t lo = seg_start[min(lane, n_seg)], hi = seg_start[min(lane + 1, n_seg)];
        const uint32_t mine = (uint32_t)((hi - lo + BM - 1) / BM) * tiles_n;  // 0 for lanes past n_seg
        uint32_t incl = mine;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t up = __shfl_up(incl, o, 64);
            if (lane >= o) incl += up;
        }
        const uint32_t total = __shfl(incl, 63, 64);
        const uint32_t total8 = (total + 7) & ~7u;
        if (blockIdx.x >= total8) return false;
        bid = xcd_remap(blockIdx.x, total8);
        if (bid >= total) return false;
        const uint64_t past = __ballot(incl > bid);  // lanes whose segments end after this tile
        e = __builtin_amdgcn_readfirstlane(__builtin_ctzll(past));
        bid = __builtin_amdgcn_readfirstlane(bid - __shfl(incl - mine, e, 64));
        r0 = __builtin_amdgcn_readfirstlane(__shfl(lo, e, 64));
        r1 = __builtin_amdgcn_readfirstlane(__shfl(hi, e, 64));
        tiles_m = (uint32_t)((r1 - r0 + BM - 1) / BM);
    } else {
        uint32_t total = 0;
        for (int q = 0; q < n_seg; ++q) total += (uint32_t)((seg_start[q + 1] - seg_start[q] + BM - 1) / BM) * tiles_n;
        const uint32_t total8 = (total + 7) & ~7u;
        if (blockIdx.x >= total8) return false;
        bid = xcd_remap(blockIdx.x, total8);
        if (bid >= total) return false;
        r0 = seg_start[0];
        r1 = r0;
        tiles_m = 0;
        for (; e < n_seg; ++e) {
            r1 = seg_start[e + 1];
            tiles_m = (uint32_t)((r1 - r0 + BM - 1) / BM);
            const uint32_t nt = tiles_m * tiles_n;
            if (bid < nt) break;
            bid -= nt;
            r0 = r1;
        }
    }
    *e_out = e;
    *r0_out = r0;
    *r1_out = r1;
    *tiles_m_out = tiles_m;
    *bid_out = bid;
    return true;
}

constexpr uint32_t kComputeUnits = 256;

// Whether an M x N output with both operands k-contiguous takes 256-row tiles on 8 waves (one work-group
// per CU), and how wide: 256 (half the LDS and L2 traffic per MFMA of a 128 x 128 tile) when the tiles fill at
// least seven tenths of the rounds of 256 work-groups they need, 192 when those fill at least 85 %; with both
// eligible, the one with fewer rounds x tile width, the narrower tile counted 6 % dearer per column (measured:
// 2048 x 12288 x 4096, 384 tiles in 2 rounds against 512 in 2: 224 -> 203 us; 2048 x 11008 x 4096, 344 tiles
// (too empty) against 464: 208 -> 184 us; 2048 x 22016 x 4096, 3 rounds against 4: 347 against 367 us;
// 4096 x 50304 x 768, 13 rounds against 17: 364 against 397 us).  Returns 0, 192 or 256.
static inline int wide_tile_for(int64_t M, int64_t N, bool allow_192) {
    const int64_t cu = kComputeUnits, rows = (M + 255) / 256;
    const int64_t t256 = rows * ((N + 255) / 256), t192 = rows * ((N + 191) / 192);
    const int64_t r256 = (t256 + cu - 1) / cu, r192 = (t192 + cu - 1) / cu;
    const bool ok256 = t256 >= cu && 10 * t256 >= 7 * r256 * cu;
    const bool ok192 = allow_192 && t192 >= cu && 100 * t192 >= 85 * r192 * cu;
    if (!ok256 && !ok192) return 0;
    if (ok256 && ok192) return r192 * 192 * 106 < r256 * 256 * 100 ? 192 : 256;
    return ok256 ? 256 : 192;
}

// Validates one descriptor and converts it to kernel arguments.  Returns PP_OK with *empty set
// when the problem has no output (M or N zero).
static inline int convert(const pp_gemm_desc* d, GemmArgs* g, bool* empty) {
    *empty = false;
    if (!d) return fail(PP_ERR_INVALID, "pp_gemm_bf16: null descriptor");
    if (d->M < 0 || d->N < 0 || d->K < 0) return fail(PP_ERR_INVALID, "pp_gemm_bf16: negative size");
    if (d->M == 0 || d->N == 0) {
        *empty = true;
        return PP_OK;
    }
    if (!d->A || !d->B || !d->C) return fail(PP_ERR_INVALID, "pp_gemm_bf16: null operand");
    if (!aligned(d->A, 16) || !aligned(d->B, 16))
        return fail(PP_ERR_INVALID, "pp_gemm_bf16: A and B must be 16-byte aligned");
    // a k-contiguous operand is read in 16-byte chunks along k; a transposed one row of k by row, any K
    // (rows past K fail the range check of the buffer loads and read as zero)
    if ((d->lda & 7) || (d->ldb & 7) || ((d->K & 7) && !(d->a_trans && d->b_trans)))
        return fail(PP_ERR_INVALID, "pp_gemm_bf16: lda, ldb (and K, unless both operands are transposed) must be "
                    "multiples of 8 (K=%lld lda=%lld ldb=%lld)", (long long)d->K, (long long)d->lda, (long long)d->ldb);
    if (d->a_trans && (d->M & 7)) return fail(PP_ERR_INVALID, "pp_gemm_bf16: transposed A needs M %% 8 == 0");
    if (d->b_trans && (d->N & 7)) return fail(PP_ERR_INVALID, "pp_gemm_bf16: transposed B needs N %% 8 == 0");
    if (d->lda < (d->a_trans ? d->M : d->K) || d->ldb < (d->b_trans ? d->N : d->K) || d->ldc < d->N)
        return fail(PP_ERR_INVALID, "pp_gemm_bf16: leading dimension too small");
    {
        // staging uses 32-bit byte offsets from the tile origin
        const uint64_t a_bytes = (uint64_t)(d->a_trans ? d->K : d->M) * (uint64_t)d->lda * 2;
        const uint64_t b_bytes = (uint64_t)(d->b_trans ? d->K : d->N) * (uint64_t)d->ldb * 2;
        if (a_bytes >= 0x7ffffff0ull || b_bytes >= 0x7ffffff0ull)
            return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16: an operand spans 2 GiB or more");
    }
    const int epi = d->epilogue == PP_EPI_ACCUM_ROUNDED ? PP_EPI_ACCUM_F32 : d->epilogue;
    const bool needs_aux = epi == PP_EPI_BIAS_RESIDUAL || epi == PP_EPI_DGELU_ERF ||
                           epi == PP_EPI_DGELU_TANH || epi == PP_EPI_DRELU;
    if (needs_aux && (!d->aux_in || d->ld_aux < d->N))
        return fail(PP_ERR_INVALID, "pp_gemm_bf16: epilogue %d needs aux_in with ld_aux >= N", epi);
    if (d->aux_out && d->ld_aux < d->N) return fail(PP_ERR_INVALID, "pp_gemm_bf16: ld_aux < N");
    if (epi == PP_EPI_ACCUM_F32 && d->c_dtype != PP_F32)
        return fail(PP_ERR_INVALID, "pp_gemm_bf16: PP_EPI_ACCUM_F32 / PP_EPI_ACCUM_ROUNDED need an fp32 C");
    g->A = static_cast<const uint16_t*>(d->A);
    g->B = static_cast<const uint16_t*>(d->B);
    g->C = d->C;
    g->M = d->M; g->N = d->N; g->K = d->K;
    g->lda = d->lda; g->ldb = d->ldb; g->ldc = d->ldc;
    g->bias = static_cast<const uint16_t*>(d->bias);
    g->aux_in = static_cast<const uint16_t*>(d->aux_in);
    g->aux_out = static_cast<uint16_t*>(d->aux_out);
    g->ld_aux = d->ld_aux;
    g->beta = d->beta;
    g->B2 = nullptr;
    g->round_bf16 = d->epilogue == PP_EPI_ACCUM_ROUNDED;
    g->epi = epi;
    g->tiles_m = g->tiles_n = g->n_blocks = 0;
    if (d->colsum && (!epi_may_sum_columns(epi) || d->c_dtype != PP_BF16))
        return fail(PP_ERR_INVALID, "pp_gemm_bf16: column sums come with the activation-derivative epilogues "
                    "and a bf16 C (epilogue %d)", epi);
    g->colsum = d->colsum;
    return PP_OK;
}


// One problem through the kernels of gemm.hip (tile shape and pipeline depth chosen per problem).
int gemm_dispatch_single(const GemmArgs& g, int at, int bt, int epi, bool cf32, hipStream_t st);

}  // namespace pp
