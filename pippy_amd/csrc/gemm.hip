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
#include "tile.h"
#include "act_math.h"
#include <vector>

namespace pp {

struct GemmArgs {
    const uint16_t* A;
    const uint16_t* B;
    void* C;
    int64_t M, N, K, lda, ldb, ldc;
    const uint16_t* bias;
    const uint16_t* aux_in;
    uint16_t* aux_out;
    int64_t ld_aux;
    int beta;
    int round_bf16;  // fp32 C: round the sums to bf16 before they are stored or added
    uint32_t tiles_m, tiles_n, n_blocks;
};

constexpr bool epi_has_bias(int epi) {
    return epi == PP_EPI_BIAS || epi == PP_EPI_BIAS_GELU_ERF || epi == PP_EPI_BIAS_GELU_TANH ||
           epi == PP_EPI_BIAS_RESIDUAL || epi == PP_EPI_BIAS_RELU;
}
constexpr bool epi_reads_aux(int epi) {
    return epi == PP_EPI_BIAS_RESIDUAL || epi == PP_EPI_DGELU_ERF || epi == PP_EPI_DGELU_TANH ||
           epi == PP_EPI_DRELU;
}
constexpr bool epi_is_gelu(int epi) { return epi == PP_EPI_BIAS_GELU_ERF || epi == PP_EPI_BIAS_GELU_TANH; }

// The bias of 4 consecutive columns starting at n0 (zero past N or without a bias).
template <int EPI>
__device__ __forceinline__ void load_bias4(const GemmArgs& g, int64_t n0, float (&bias)[4]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) bias[e] = 0.f;
    if (!epi_has_bias(EPI) || !g.bias || n0 >= g.N) return;
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
template <int EPI>
__device__ __forceinline__ void epilogue_math4(float (&v)[4], float (&pre)[4], const float (&bias)[4],
                                               const float (&a)[4]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (epi_has_bias(EPI)) v[e] += bias[e];
        if (EPI == PP_EPI_BIAS_RESIDUAL) v[e] += a[e];
        if (EPI == PP_EPI_DGELU_ERF) v[e] *= dgelu_erf(a[e]);
        if (EPI == PP_EPI_DGELU_TANH) v[e] *= dgelu_tanh(a[e]);
        if (EPI == PP_EPI_DRELU) v[e] = a[e] > 0.f ? v[e] : 0.f;
        pre[e] = v[e];
        if (EPI == PP_EPI_BIAS_GELU_ERF) v[e] = gelu_erf(v[e]);
        if (EPI == PP_EPI_BIAS_GELU_TANH) v[e] = gelu_tanh(v[e]);
        if (EPI == PP_EPI_BIAS_RELU) v[e] = fmaxf(v[e], 0.f);
    }
}

// Applies the epilogue to 4 consecutive columns n0..n0+3 of row m and stores them; handles rows
// and columns past the edge of C and unaligned operands.
template <int EPI, bool CF32>
__device__ __forceinline__ void epilogue4(const GemmArgs& g, int64_t m, int64_t n0, float v0, float v1,
                                          float v2, float v3, const float (&bias)[4], bool vec_ok) {
    if (m >= g.M || n0 >= g.N) return;
    float v[4] = {v0, v1, v2, v3}, pre[4];
    const int nv = (g.N - n0 >= 4) ? 4 : (int)(g.N - n0);
    const bool full = vec_ok && nv == 4;

    float a[4] = {0.f, 0.f, 0.f, 0.f};
    if (epi_reads_aux(EPI)) {
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
    epilogue_math4<EPI>(v, pre, bias, a);
    if (epi_is_gelu(EPI) && g.aux_out) {
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

// How the 4 waves of a work-group share a BM x BN tile: 2 x 2 when BN is a multiple of 64, else 4 x 1
// (a 128 x 96 tile: each wave 32 rows by 96 columns).  A wave's part is TM x TN MFMA tiles of 32 x 32.
template <int BM, int BN>
struct WaveTile {
    static constexpr int WGN = (BN % 64 == 0) ? 2 : 1;
    static constexpr int WGM = 4 / WGN;
    static constexpr int WTM = BM / WGM, WTN = BN / WGN;
    static constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "a wave's part of the tile is made of 32 x 32 MFMA tiles");
};

// Main loop of one BM x BN output tile over the k-tiles [kt_begin, kt_end) of KT values each, through
// NS LDS stages filled by direct-to-LDS loads; the products are added to acc.  Starts with a barrier,
// so that it may follow an epilogue (or another main loop) that used the same LDS.
template <int BM, int BN, bool AT, bool BT, int NS, int KT>
__device__ __forceinline__ void gemm_mainloop(const GemmArgs& g, uint32_t tile_m, uint32_t tile_n, int kt_begin,
                                              int kt_end,
                                              f32x16_t (&acc)[WaveTile<BM, BN>::TN][WaveTile<BM, BN>::TM]) {
    typedef WaveTile<BM, BN> WT;
    constexpr int WTM = WT::WTM, WTN = WT::WTN, TM = WT::TM, TN = WT::TN;
    constexpr int KS = KT / 16;  // MFMA k-steps per tile
    constexpr int kStageElems = (BM + BN) * KT;
    constexpr int LPT = DmaStage<BM, AT, KT>::kLoads + DmaStage<BN, BT, KT>::kLoads;  // loads per tile per wave
    constexpr int kReadsPerStep = TM * FragReader<BM, AT, KT>::kReads + TN * FragReader<BN, BT, KT>::kReads;
    static_assert(NS >= 2 && NS <= 4 && (NS - 1) * LPT < 64, "pipeline depth exceeds vmcnt");
    static_assert(KS >= 2 && TN >= 2, "the last k-step is split in two parts around the barrier");
    static_assert(NS * kStageElems * 2 >= 4 * 32 * WTN * 4, "the epilogue stages fp32 bands in the tile memory");
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave % WT::WGM) * WTM, wn0 = (wave / WT::WGM) * WTN;

    DmaStage<BM, AT, KT> sa;
    DmaStage<BN, BT, KT> sb;
    sa.init(g.A, g.lda, m0, g.M, g.K, wave, lane);
    sb.init(g.B, g.ldb, n0, g.N, g.K, wave, lane);
    const int nk = kt_end - kt_begin;
    auto issue = [&](int stage, int kt) {
        sa.load(smem + stage * kStageElems, (kt_begin + kt) * KT, wave);
        sb.load(smem + stage * kStageElems + BM * KT, (kt_begin + kt) * KT, wave);
    };

    FragReader<BM, AT, KT> ra[TM];
    FragReader<BN, BT, KT> rb[TN];
#pragma unroll
    for (int t = 0; t < TM; ++t) ra[t].init(wm0 + t * 32, lane);
#pragma unroll
    for (int t = 0; t < TN; ++t) rb[t].init(wn0 + t * 32, lane);
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
            for (int b = 0; b < TM; ++b)
                acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[sel][a], fa[sel][b], acc[a][b], 0, 0, 0);
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
template <int BM, int BN, int EPI, bool CF32, int EB = 0>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& g, uint32_t tile_m, uint32_t tile_n,
                                              f32x16_t (&acc)[WaveTile<BM, BN>::TN][WaveTile<BM, BN>::TM]) {
    typedef WaveTile<BM, BN> WT;
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
    float bias[4];
    load_bias4<EPI>(g, gn, bias);
    // a tile in the interior of C with aligned operands takes the path without bounds checks, in
    // which the loads of a band (LDS, auxiliary tensor, old C) are issued before any arithmetic
    const bool interior = vec_ok && m0 + BM <= g.M && n0 + BN <= g.N;
    constexpr int kPasses = 32 / RPP;
#pragma unroll
    for (int b = 0; b < TM; ++b) {
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int u = a * 8 + 2 * q + lh;
                *reinterpret_cast<float4*>(cw + l32 * WTN + (unit_at(u, l32) << 2)) =
                    make_float4(acc[a][b][4 * q], acc[a][b][4 * q + 1], acc[a][b][4 * q + 2], acc[a][b][4 * q + 3]);
            }
        const int64_t gm = m0 + wm0 + b * 32 + rr;  // row of pass 0; pass i adds i * RPP
        if (interior && lane_on) {
          // EB passes at a time (all of them by default): fewer values in flight for a kernel that
          // counts on many resident waves rather than on long runs of independent loads
          constexpr int kBatch = EB > 0 && EB < kPasses ? EB : kPasses;
          static_assert(kPasses % kBatch == 0, "the passes of a band split into whole batches");
#pragma unroll
          for (int i0 = 0; i0 < kPasses; i0 += kBatch) {
            float4 v4[kPasses];
            uint2 aw[kPasses];
            float4 old[kPasses];
#pragma unroll
            for (int i = i0; i < i0 + kBatch; ++i) {
                const int m = i * RPP + rr;
                v4[i] = *reinterpret_cast<const float4*>(cw + m * WTN + (unit_at(ru, m) << 2));
            }
            if (epi_reads_aux(EPI)) {
#pragma unroll
                for (int i = i0; i < i0 + kBatch; ++i)
                    aw[i] = *reinterpret_cast<const uint2*>(g.aux_in + (gm + i * RPP) * g.ld_aux + gn);
            }
            if (CF32 && EPI == PP_EPI_ACCUM_F32 && g.beta) {
#pragma unroll
                for (int i = i0; i < i0 + kBatch; ++i)
                    old[i] = *reinterpret_cast<const float4*>(static_cast<const float*>(g.C) + (gm + i * RPP) * g.ldc + gn);
            }
#pragma unroll
            for (int i = i0; i < i0 + kBatch; ++i) {
                float v[4] = {v4[i].x, v4[i].y, v4[i].z, v4[i].w}, pre[4];
                float av[4] = {0.f, 0.f, 0.f, 0.f};
                if (epi_reads_aux(EPI)) {
                    av[0] = bf16lo(aw[i].x); av[1] = bf16hi(aw[i].x); av[2] = bf16lo(aw[i].y); av[3] = bf16hi(aw[i].y);
                }
                epilogue_math4<EPI>(v, pre, bias, av);
                const int64_t row = gm + i * RPP;
                if (epi_is_gelu(EPI) && g.aux_out)
                    *reinterpret_cast<uint2*>(g.aux_out + row * g.ld_aux + gn) =
                        make_uint2(pack_bf16(pre[0], pre[1]), pack_bf16(pre[2], pre[3]));
                if (CF32) {
                    float* cp = static_cast<float*>(g.C) + row * g.ldc + gn;
                    if (EPI == PP_EPI_ACCUM_F32 && g.round_bf16) {
                        const uint32_t w0 = pack_bf16(v[0], v[1]), w1 = pack_bf16(v[2], v[3]);
                        v[0] = bf16lo(w0); v[1] = bf16hi(w0); v[2] = bf16lo(w1); v[3] = bf16hi(w1);
                    }
                    if (EPI == PP_EPI_ACCUM_F32 && g.beta)
                        *reinterpret_cast<float4*>(cp) = make_float4(old[i].x + v[0], old[i].y + v[1], old[i].z + v[2], old[i].w + v[3]);
                    else
                        *reinterpret_cast<float4*>(cp) = make_float4(v[0], v[1], v[2], v[3]);
                } else {
                    *reinterpret_cast<uint2*>(static_cast<uint16_t*>(g.C) + row * g.ldc + gn) =
                        make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
                }
            }
          }
        } else if (lane_on) {
#pragma unroll
            for (int i = 0; i < kPasses; ++i) {
                const int m = i * RPP + rr;
                const float4 v = *reinterpret_cast<const float4*>(cw + m * WTN + (unit_at(ru, m) << 2));
                epilogue4<EPI, CF32>(g, gm + i * RPP, gn, v.x, v.y, v.z, v.w, bias, vec_ok);
            }
        }
    }
}

// One whole output tile: main loop over all of K, then the epilogue.
template <int BM, int BN, bool AT, bool BT, int NS, int EPI, bool CF32, int KT = BK, int EB = 0>
__device__ __forceinline__ void gemm_tile_dma(const GemmArgs& g, uint32_t tile_m, uint32_t tile_n) {
    f32x16_t acc[WaveTile<BM, BN>::TN][WaveTile<BM, BN>::TM];
#pragma unroll
    for (int a = 0; a < WaveTile<BM, BN>::TN; ++a)
#pragma unroll
        for (int b = 0; b < WaveTile<BM, BN>::TM; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;
    gemm_mainloop<BM, BN, AT, BT, NS, KT>(g, tile_m, tile_n, 0, (int)((g.K + KT - 1) / KT), acc);
    gemm_epilogue<BM, BN, EPI, CF32, EB>(g, tile_m, tile_n, acc);
}

template <int BM, int BN, bool AT, bool BT, int NS, int EPI, bool CF32, int KT = BK>
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_dma_kernel(const GemmArgs g) {
    const uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= g.n_blocks) return;
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    gemm_tile_dma<BM, BN, AT, BT, NS, EPI, CF32, KT>(g, tile_m, tile_n);
}

// Split along K on 256 x 256 tiles, for an output with few tiles and a long reduction (the input
// gradient of a vocabulary projection: 4096 x 768 with K = 50304).  Large tiles load half as many
// operand bytes per FLOP as 128-wide ones, and the split makes enough of them to fill the CUs.
// Split s of a tile reduces k-tiles [s * kt_per_split, (s + 1) * kt_per_split) into its own fp32
// copy of C in the workspace; splitk_reduce_kernel adds the copies in split order.
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_splitk_kernel(const GemmArgs g, float* ws, int splits,
                                                                       int kt_per_split) {
    const uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= g.n_blocks * (uint32_t)splits) return;
    const int split = (int)(bid / g.n_blocks);
    uint32_t tile_m, tile_n;
    grouped_tile(bid % g.n_blocks, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    f32x16_t acc[WaveTile<256, 256>::TN][WaveTile<256, 256>::TM];
#pragma unroll
    for (int a = 0; a < WaveTile<256, 256>::TN; ++a)
#pragma unroll
        for (int b = 0; b < WaveTile<256, 256>::TM; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;
    const int nk = (int)((g.K + BK - 1) / BK);
    const int kb = min(nk, split * kt_per_split), ke = min(nk, kb + kt_per_split);
    gemm_mainloop<256, 256, false, false, 2, BK>(g, tile_m, tile_n, kb, ke, acc);
    GemmArgs part = g;
    part.C = ws + (size_t)split * (size_t)g.M * (size_t)g.N;
    part.ldc = g.N;
    gemm_epilogue<256, 256, PP_EPI_NONE, true>(part, tile_m, tile_n, acc);
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

// Several independent problems in one grid: the tiles of problem i are the block ids
// [tile_start[i], tile_start[i + 1]).
struct GemmGroupArgs {
    GemmArgs p[PP_GEMM_MAX_GROUP];
    uint32_t tile_start[PP_GEMM_MAX_GROUP + 1];
    int n;
};

template <int BM, int BN, bool AT, bool BT, int NS, int EPI, bool CF32, int KT = BK>
__global__ __launch_bounds__(kGemmThreads) void gemm_bf16_group_kernel(const GemmGroupArgs ga) {
    uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= ga.tile_start[ga.n]) return;
    int i = 0;
    while (i + 1 < ga.n && bid >= ga.tile_start[i + 1]) ++i;
    bid -= ga.tile_start[i];
    const GemmArgs& g = ga.p[i];
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    gemm_tile_dma<BM, BN, AT, BT, NS, EPI, CF32, KT>(g, tile_m, tile_n);
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
    // tiles of every segment, then an XCD-contiguous numbering of exactly that many ids
    int e = 0;
    int32_t r0, r1;
    uint32_t tiles_m, bid;
    if (sa.n_seg < 64) {
        // one vector load of the bounds (lane l holds segment l) and a prefix sum over the lanes,
        // instead of a chain of dependent scalar loads that would cost as much as a third of a tile
        const int lane = threadIdx.x & 63;
        const int32_t lo = sa.seg_start[min(lane, sa.n_seg)], hi = sa.seg_start[min(lane + 1, sa.n_seg)];
        const uint32_t mine = (uint32_t)((hi - lo + BM - 1) / BM) * sa.g.tiles_n;  // 0 for lanes past n_seg
        uint32_t incl = mine;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t up = __shfl_up(incl, o, 64);
            if (lane >= o) incl += up;
        }
        const uint32_t total = __shfl(incl, 63, 64);
        const uint32_t total8 = (total + 7) & ~7u;
        if (blockIdx.x >= total8) return;
        bid = xcd_remap(blockIdx.x, total8);
        if (bid >= total) return;
        const uint64_t past = __ballot(incl > bid);  // lanes whose segments end after this tile
        e = __builtin_amdgcn_readfirstlane(__builtin_ctzll(past));
        bid = __builtin_amdgcn_readfirstlane(bid - __shfl(incl - mine, e, 64));
        r0 = __builtin_amdgcn_readfirstlane(__shfl(lo, e, 64));
        r1 = __builtin_amdgcn_readfirstlane(__shfl(hi, e, 64));
        tiles_m = (uint32_t)((r1 - r0 + BM - 1) / BM);
    } else {
        uint32_t total = 0;
        for (int q = 0; q < sa.n_seg; ++q)
            total += (uint32_t)((sa.seg_start[q + 1] - sa.seg_start[q] + BM - 1) / BM) * sa.g.tiles_n;
        const uint32_t total8 = (total + 7) & ~7u;
        if (blockIdx.x >= total8) return;
        bid = xcd_remap(blockIdx.x, total8);
        if (bid >= total) return;
        r0 = sa.seg_start[0];
        r1 = r0;
        tiles_m = 0;
        for (; e < sa.n_seg; ++e) {
            r1 = sa.seg_start[e + 1];
            tiles_m = (uint32_t)((r1 - r0 + BM - 1) / BM);
            const uint32_t nt = tiles_m * sa.g.tiles_n;
            if (bid < nt) break;
            bid -= nt;
            r0 = r1;
        }
    }
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

template <typename Kernel>
static int reserve_lds(Kernel kernel, size_t lds) {
    const hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (rc != hipSuccess)
        return fail(PP_ERR_LAUNCH, "pp_gemm_bf16: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(rc));
    return PP_OK;
}

template <int BM, int BN>
static int count_tiles(GemmArgs& g) {
    g.tiles_m = (uint32_t)((g.M + BM - 1) / BM);
    g.tiles_n = (uint32_t)((g.N + BN - 1) / BN);
    const uint64_t nb = (uint64_t)g.tiles_m * g.tiles_n;
    if (nb > 0x0fffff00ull) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16: too many tiles");
    g.n_blocks = (uint32_t)nb;
    return PP_OK;
}

// Pipeline depth: with at most one tile per CU a block has the CU to itself and takes 3 stages;
// with more tiles 2 stages leave room for two resident blocks, whose prologues and epilogues overlap
// each other's main loops.
constexpr uint32_t kComputeUnits = 256;
constexpr int64_t kBigTileMinTiles = 1024;  // 256 x 256 tiles are used from this many of them

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
static int launch_group(const GemmGroupArgs& ga, hipStream_t st) {
    constexpr size_t lds = (size_t)NS * (BM + BN) * KT * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_group_kernel<BM, BN, AT, BT, NS, EPI, CF32, KT>, lds);
    if (attr_rc) return attr_rc;
    const uint32_t grid = (ga.tile_start[ga.n] + 7) / 8 * 8;
    hipLaunchKernelGGL((gemm_bf16_group_kernel<BM, BN, AT, BT, NS, EPI, CF32, KT>), dim3(grid), dim3(kGemmThreads),
                       lds, st, ga);
    return check_launch("gemm_bf16_group_kernel");
}

template <int BM, int BN, bool AT, bool BT, int EPI, bool CF32>
static int launch_gemm(const GemmArgs* probs, int n, hipStream_t st) {
    if (n == 1) {
        if constexpr (EPI == PP_EPI_NONE && !CF32 && BM == 128 && !AT && !BT) {
            // a large output with both operands k-contiguous: 256 x 256 tiles halve the LDS and L2
            // traffic per MFMA (vocabulary projection 4096 x 50304 x 768: 776 against 707 TFLOP/s)
            GemmArgs big = probs[0];
            if (((big.M + 255) / 256) * ((big.N + 255) / 256) >= kBigTileMinTiles) {
                int rc = count_tiles<256, 256>(big);
                if (rc) return rc;
                return launch_single<256, 256, AT, BT, 2, EPI, CF32>(big, st);
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
        GemmArgs g = probs[0];
        int rc = count_tiles<BM, BN>(g);
        if (rc) return rc;
        return g.n_blocks <= kComputeUnits ? launch_single<BM, BN, AT, BT, 3, EPI, CF32>(g, st)
                                           : launch_single<BM, BN, AT, BT, 2, EPI, CF32>(g, st);
    }
    if constexpr (EPI == PP_EPI_NONE || EPI == PP_EPI_ACCUM_F32) {
        for (int i0 = 0; i0 < n; i0 += PP_GEMM_MAX_GROUP) {
            GemmGroupArgs ga;
            ga.n = (n - i0 < PP_GEMM_MAX_GROUP) ? n - i0 : PP_GEMM_MAX_GROUP;
            uint64_t total = 0;
            for (int i = 0; i < ga.n; ++i) {
                ga.p[i] = probs[i0 + i];
                int rc = count_tiles<BM, BN>(ga.p[i]);
                if (rc) return rc;
                ga.tile_start[i] = (uint32_t)total;
                total += ga.p[i].n_blocks;
            }
            if (total > 0x7fffff00ull) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_grouped: too many tiles");
            ga.tile_start[ga.n] = (uint32_t)total;
            if (total == 0) continue;
            int rc = total <= kComputeUnits ? launch_group<BM, BN, AT, BT, 3, EPI, CF32>(ga, st)
                                            : launch_group<BM, BN, AT, BT, 2, EPI, CF32>(ga, st);
            if (rc) return rc;
        }
        return PP_OK;
    } else {
        // epilogues that chain kernels are launched one by one
        for (int i = 0; i < n; ++i) {
            int rc = launch_gemm<BM, BN, AT, BT, EPI, CF32>(probs + i, 1, st);
            if (rc) return rc;
        }
        return PP_OK;
    }
}

template <int EPI, bool CF32>
static int dispatch_layout(const GemmArgs* g, int n, int at, int bt, hipStream_t st) {
    if (!at && !bt) return launch_gemm<128, 128, false, false, EPI, CF32>(g, n, st);
    if (!at && bt) return launch_gemm<128, 128, false, true, EPI, CF32>(g, n, st);
    if (at && !bt) return launch_gemm<128, 128, true, false, EPI, CF32>(g, n, st);
    return launch_gemm<128, 128, true, true, EPI, CF32>(g, n, st);
}

static int dispatch(const GemmArgs* g, int n, int at, int bt, int epi, bool cf32, hipStream_t st) {
    if (epi == PP_EPI_ACCUM_ROUNDED) epi = PP_EPI_ACCUM_F32;  // the same kernels; GemmArgs::round_bf16 is set
    if (cf32) {
        switch (epi) {
            case PP_EPI_NONE: return dispatch_layout<PP_EPI_NONE, true>(g, n, at, bt, st);
            case PP_EPI_ACCUM_F32: return dispatch_layout<PP_EPI_ACCUM_F32, true>(g, n, at, bt, st);
            default: return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16: epilogue %d with fp32 C", epi);
        }
    }
    switch (epi) {
        case PP_EPI_NONE: return dispatch_layout<PP_EPI_NONE, false>(g, n, at, bt, st);
        case PP_EPI_BIAS: return dispatch_layout<PP_EPI_BIAS, false>(g, n, at, bt, st);
        case PP_EPI_BIAS_GELU_ERF: return dispatch_layout<PP_EPI_BIAS_GELU_ERF, false>(g, n, at, bt, st);
        case PP_EPI_BIAS_GELU_TANH: return dispatch_layout<PP_EPI_BIAS_GELU_TANH, false>(g, n, at, bt, st);
        case PP_EPI_BIAS_RESIDUAL: return dispatch_layout<PP_EPI_BIAS_RESIDUAL, false>(g, n, at, bt, st);
        case PP_EPI_DGELU_ERF: return dispatch_layout<PP_EPI_DGELU_ERF, false>(g, n, at, bt, st);
        case PP_EPI_DGELU_TANH: return dispatch_layout<PP_EPI_DGELU_TANH, false>(g, n, at, bt, st);
        case PP_EPI_BIAS_RELU: return dispatch_layout<PP_EPI_BIAS_RELU, false>(g, n, at, bt, st);
        case PP_EPI_DRELU: return dispatch_layout<PP_EPI_DRELU, false>(g, n, at, bt, st);
        default: return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16: epilogue %d", epi);
    }
}

// Validates one descriptor and converts it to kernel arguments.  Returns PP_OK with *empty set
// when the problem has no output (M or N zero).
static int convert(const pp_gemm_desc* d, GemmArgs* g, bool* empty) {
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
    if ((d->K & 7) || (d->lda & 7) || (d->ldb & 7))
        return fail(PP_ERR_INVALID, "pp_gemm_bf16: K, lda, ldb must be multiples of 8 (K=%lld lda=%lld ldb=%lld)",
                    (long long)d->K, (long long)d->lda, (long long)d->ldb);
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
    g->round_bf16 = d->epilogue == PP_EPI_ACCUM_ROUNDED;
    g->tiles_m = g->tiles_n = g->n_blocks = 0;
    return PP_OK;
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

extern "C" int pp_gemm_bf16(const pp_gemm_desc* d, pp_stream stream) {
    GemmArgs g;
    bool empty;
    int rc = convert(d, &g, &empty);
    if (rc || empty) return rc;
    return dispatch(&g, 1, d->a_trans ? 1 : 0, d->b_trans ? 1 : 0, d->epilogue, d->c_dtype == PP_F32,
                    static_cast<hipStream_t>(stream));
}

extern "C" int pp_gemm_bf16_grouped(const pp_gemm_desc* descs, int n, pp_stream stream) {
    if (n < 0 || (n > 0 && !descs)) return fail(PP_ERR_INVALID, "pp_gemm_bf16_grouped: bad list");
    if (n == 0) return PP_OK;
    std::vector<GemmArgs> probs;
    probs.reserve(n);
    const pp_gemm_desc& f = descs[0];
    for (int i = 0; i < n; ++i) {
        const pp_gemm_desc& d = descs[i];
        if ((d.a_trans != 0) != (f.a_trans != 0) || (d.b_trans != 0) != (f.b_trans != 0) ||
            d.epilogue != f.epilogue || d.c_dtype != f.c_dtype)
            return fail(PP_ERR_INVALID, "pp_gemm_bf16_grouped: problem %d differs in layout, epilogue or dtype", i);
        GemmArgs g;
        bool empty;
        int rc = convert(&d, &g, &empty);
        if (rc) return rc;
        if (!empty) probs.push_back(g);
    }
    if (probs.empty()) return PP_OK;
    return dispatch(probs.data(), (int)probs.size(), f.a_trans ? 1 : 0, f.b_trans ? 1 : 0, f.epilogue,
                    f.c_dtype == PP_F32, static_cast<hipStream_t>(stream));
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
    const int splits = (workspace && aligned(workspace, 16)) ? splitk_plan(d, workspace_elems, &kt_per_split) : 0;
    if (!splits) return pp_gemm_bf16(d, stream);
    rc = count_tiles<256, 256>(g);
    if (rc) return rc;
    constexpr size_t lds = (size_t)2 * (256 + 256) * BK * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_splitk_kernel, lds);
    if (attr_rc) return attr_rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t grid = (g.n_blocks * (uint32_t)splits + 7) / 8 * 8;
    hipLaunchKernelGGL(gemm_bf16_splitk_kernel, dim3(grid), dim3(kGemmThreads), lds, st, g, workspace, splits,
                       kt_per_split);
    rc = check_launch("gemm_bf16_splitk_kernel");
    if (rc) return rc;
    const int64_t quads = g.M * (g.N >> 2);
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((uint32_t)((quads + 255) / 256)), dim3(256), 0, st, workspace,
                       splits, g.M, g.N, static_cast<uint16_t*>(g.C), g.ldc);
    return check_launch("splitk_reduce_kernel");
}
