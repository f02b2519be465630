// Grouped bf16 GEMM launches: several independent problems in one grid (see gemm_core.h for the
// kernel).  Two families:
//   * problems with a bf16 C, whatever their epilogues: one kernel that takes each problem's epilogue at
//     run time, so the GEMMs that several pipeline stages reach at the same position of their passes go
//     out together (forward and input-gradient GEMMs of different virtual stages);
//   * problems that add to (or write) an fp32 C: the weight-gradient GEMMs of one or more passes.
#include "gemm_core.h"
#include <vector>

namespace pp {

template <int BM, int BN, bool AT, bool BT, int NS, int EPI, bool CF32, int KT, int W = 4>
static int launch_group(GemmGroupArgs& ga, hipStream_t st) {
    constexpr size_t lds = (size_t)NS * (BM + BN) * KT * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_group_kernel<BM, BN, AT, BT, NS, EPI, CF32, KT, W>, lds);
    if (attr_rc) return attr_rc;
    uint64_t total = 0;
    for (int i = 0; i < ga.n; ++i) {
        int rc = count_tiles<BM, BN>(ga.p[i]);
        if (rc) return rc;
        ga.tile_start[i] = (uint32_t)total;
        total += ga.p[i].n_blocks;
    }
    if (total > 0x7fffff00ull) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_grouped: too many tiles");
    ga.tile_start[ga.n] = (uint32_t)total;
    if (total == 0) return PP_OK;
    const uint32_t grid = ((uint32_t)total + 7) / 8 * 8;
    hipLaunchKernelGGL((gemm_bf16_group_kernel<BM, BN, AT, BT, NS, EPI, CF32, KT, W>), dim3(grid), dim3(W * 64),
                       lds, st, ga);
    return check_launch("gemm_bf16_group_kernel");
}

static uint64_t tiles_128(const GemmGroupArgs& ga) {
    uint64_t t = 0;
    for (int i = 0; i < ga.n; ++i)
        t += (uint64_t)((ga.p[i].M + 127) / 128) * (uint64_t)((ga.p[i].N + 127) / 128);
    return t;
}

// 128 x 128 tiles: with at most one tile per CU a work-group has the CU to itself and takes 3 LDS
// stages; with more tiles 2 stages leave room for two resident work-groups.  (Wider tiles were
// measured on groups of 2 to 4 transformer-sized problems per launch, 256 x 128, 128 x 256 and
// 256 x 256 with 2 to 4 stages of 32 or 64 k: none ran a forward-shaped group faster than 128 x 128.)
template <bool AT, bool BT, int EPI, bool CF32>
static int launch_auto(GemmGroupArgs& ga, hipStream_t st) {
    if constexpr (AT && BT && CF32) {
        // the weight gradients of a stage pass: more 128 x 128 tiles than two per CU.  256 x 128 tiles on
        // 8 waves load a quarter less per flop and, with the CU to themselves, keep 3 stages (two tiles
        // in flight): 880 against 800 TFLOP/s on the 12 problems of three GPT-2-small layers
        if (tiles_128(ga) > 2 * kComputeUnits) return launch_group<256, 128, AT, BT, 3, EPI, CF32, 64, 8>(ga, st);
    }
    return tiles_128(ga) <= kComputeUnits ? launch_group<128, 128, AT, BT, 3, EPI, CF32, 64>(ga, st)
                                          : launch_group<128, 128, AT, BT, 2, EPI, CF32, 64>(ga, st);
}

template <int EPI, bool CF32>
static int launch_layout(GemmGroupArgs& ga, int at, int bt, hipStream_t st) {
    if (!at && !bt) return launch_auto<false, false, EPI, CF32>(ga, st);
    if (!at && bt) return launch_auto<false, true, EPI, CF32>(ga, st);
    if (at && !bt) return launch_auto<true, false, EPI, CF32>(ga, st);
    return launch_auto<true, true, EPI, CF32>(ga, st);
}

// ---- weight gradients of several microbatches in one launch --------------------------------------
// Problem i is  C_i = (beta ? C_i : 0) + g_0 + g_1 + ... + g_{S-1}  with  g_s = A_{i,s}^T B_{i,s}  (rounded to
// bf16 first when the problem says so), the terms added one by one in ascending s in fp32: bit for bit
// what S accumulating launches, one per microbatch, leave in C.  A tile keeps the running sum in
// registers over all S reductions, so C is read (at most) once and written once instead of S times, and
// the k-loop of a tile is S times as long.  GemmArgs::A and ::B of a problem point to DEVICE arrays of
// its S operand pointers.
template <int BM, int BN, int NS, int KT, int W>
__global__ __launch_bounds__(W * 64) void gemm_bf16_group_kseg_kernel(const GemmGroupArgs ga, const int n_seg) {
    uint32_t bid = xcd_remap(blockIdx.x, gridDim.x);
    if (bid >= ga.tile_start[ga.n]) return;
    int i = 0;
    while (i + 1 < ga.n && bid >= ga.tile_start[i + 1]) ++i;
    bid -= ga.tile_start[i];
    GemmArgs g = ga.p[i];
    uint32_t tile_m, tile_n;
    grouped_tile(bid, g.tiles_m, g.tiles_n, &tile_m, &tile_n);
    typedef WaveTile<BM, BN, W> WT;
    const uint16_t* const* seg_a = reinterpret_cast<const uint16_t* const*>(g.A);
    const uint16_t* const* seg_b = reinterpret_cast<const uint16_t* const*>(g.B);
    f32x16_t total[WT::TN][WT::TM], acc[WT::TN][WT::TM];
    if (g.beta) load_c_as_accumulators<BM, BN, W>(g, tile_m, tile_n, total);
    const int nk = (int)((g.K + KT - 1) / KT);
    for (int s = 0; s < n_seg; ++s) {
        g.A = seg_a[s];
        g.B = seg_b[s];
#pragma unroll
        for (int a = 0; a < WT::TN; ++a)
#pragma unroll
            for (int b = 0; b < WT::TM; ++b)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;
        gemm_mainloop<BM, BN, true, true, NS, KT, false, W>(g, tile_m, tile_n, 0, nk, acc);
        const bool first = s == 0 && !g.beta;  // the first term of a fresh sum is stored, not added to zero
#pragma unroll
        for (int a = 0; a < WT::TN; ++a)
#pragma unroll
            for (int b = 0; b < WT::TM; ++b)
#pragma unroll
                for (int e = 0; e < 16; e += 2) {
                    float lo = acc[a][b][e], hi = acc[a][b][e + 1];
                    if (g.round_bf16) {
                        const uint32_t w = pack_bf16(lo, hi);
                        lo = bf16lo(w);
                        hi = bf16hi(w);
                    }
                    total[a][b][e] = first ? lo : total[a][b][e] + lo;
                    total[a][b][e + 1] = first ? hi : total[a][b][e + 1] + hi;
                }
    }
    g.beta = 0;
    g.round_bf16 = 0;
    gemm_epilogue<BM, BN, PP_EPI_NONE, true, 0, W>(g, tile_m, tile_n, total);
}

template <int BM, int BN, int NS, int KT, int W>
static int launch_group_kseg(GemmGroupArgs& ga, int n_seg, hipStream_t st) {
    constexpr size_t lds = (size_t)NS * (BM + BN) * KT * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_group_kseg_kernel<BM, BN, NS, KT, W>, lds);
    if (attr_rc) return attr_rc;
    uint64_t total = 0;
    for (int i = 0; i < ga.n; ++i) {
        int rc = count_tiles<BM, BN>(ga.p[i]);
        if (rc) return rc;
        ga.tile_start[i] = (uint32_t)total;
        total += ga.p[i].n_blocks;
    }
    if (total > 0x7fffff00ull) return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_grouped_kseg: too many tiles");
    ga.tile_start[ga.n] = (uint32_t)total;
    if (total == 0) return PP_OK;
    const uint32_t grid = ((uint32_t)total + 7) / 8 * 8;
    hipLaunchKernelGGL((gemm_bf16_group_kseg_kernel<BM, BN, NS, KT, W>), dim3(grid), dim3(W * 64), lds, st, ga,
                       n_seg);
    return check_launch("gemm_bf16_group_kseg_kernel");
}

}  // namespace pp

using namespace pp;

extern "C" int pp_gemm_bf16_grouped_kseg(const pp_gemm_desc* descs, int n, int n_seg, pp_stream stream) {
    if (n < 0 || (n > 0 && !descs)) return fail(PP_ERR_INVALID, "pp_gemm_bf16_grouped_kseg: bad list");
    if (n_seg < 1 || n_seg > PP_GEMM_MAX_KSEG)
        return fail(PP_ERR_INVALID, "pp_gemm_bf16_grouped_kseg: n_seg %d out of [1, %d]", n_seg, PP_GEMM_MAX_KSEG);
    std::vector<GemmArgs> probs;
    probs.reserve(n);
    for (int i = 0; i < n; ++i) {
        const pp_gemm_desc& d = descs[i];
        if (!d.a_trans || !d.b_trans || d.c_dtype != PP_F32 ||
            (d.epilogue != PP_EPI_ACCUM_F32 && d.epilogue != PP_EPI_ACCUM_ROUNDED))
            return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_grouped_kseg: problem %d is not a transposed-operand "
                        "product accumulated into an fp32 C", i);
        if (!aligned(d.A, 8) || !aligned(d.B, 8))
            return fail(PP_ERR_INVALID, "pp_gemm_bf16_grouped_kseg: problem %d: A and B are device arrays of "
                        "pointers", i);
        // the operand checks of a single product, on a copy whose operands pass the alignment test (the
        // real operand pointers live in device memory; the caller vouches for their 16-byte alignment)
        pp_gemm_desc probe = d;
        probe.A = probe.B = reinterpret_cast<const void*>(uintptr_t(16));
        GemmArgs g;
        bool empty;
        int rc = convert(&probe, &g, &empty);
        if (rc) return rc;
        if (empty) continue;
        g.A = static_cast<const uint16_t*>(d.A);
        g.B = static_cast<const uint16_t*>(d.B);
        probs.push_back(g);
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int total = (int)probs.size();
    const int launches = (total + PP_GEMM_MAX_GROUP - 1) / PP_GEMM_MAX_GROUP;
    int done = 0;
    for (int l = 0; l < launches; ++l) {
        const int cnt = (total - done + (launches - l) - 1) / (launches - l);
        GemmGroupArgs ga;
        ga.n = cnt;
        for (int i = 0; i < cnt; ++i) ga.p[i] = probs[done + i];
        done += cnt;
        // as for one pass: 256 x 128 tiles on 8 waves once there are more 128 x 128 tiles than two per CU (the
        // running sum doubles the accumulator registers, which 8 waves per CU leave room for; Llama-2-7B
        // stage step with one pass per step: 389 -> 375 ms)
        int rc = tiles_128(ga) > 2 * kComputeUnits ? launch_group_kseg<256, 128, 3, 64, 8>(ga, n_seg, st)
                                                   : launch_group_kseg<128, 128, 2, 64, 4>(ga, n_seg, st);
        if (rc) return rc;
    }
    return PP_OK;
}

extern "C" int pp_gemm_bf16_grouped(const pp_gemm_desc* descs, int n, pp_stream stream) {
    if (n < 0 || (n > 0 && !descs)) return fail(PP_ERR_INVALID, "pp_gemm_bf16_grouped: bad list");
    if (n == 0) return PP_OK;
    std::vector<GemmArgs> probs;
    probs.reserve(n);
    const pp_gemm_desc& f = descs[0];
    const bool cf32 = f.c_dtype == PP_F32;
    // an fp32 C either takes plain sums or accumulates (rounded or not, per problem): two kernels
    auto f32_class = [](int epi) { return epi == PP_EPI_NONE ? 0 : 1; };
    for (int i = 0; i < n; ++i) {
        const pp_gemm_desc& d = descs[i];
        if ((d.a_trans != 0) != (f.a_trans != 0) || (d.b_trans != 0) != (f.b_trans != 0) || d.c_dtype != f.c_dtype)
            return fail(PP_ERR_INVALID, "pp_gemm_bf16_grouped: problem %d differs in layout or output dtype", i);
        if (cf32) {
            if (d.epilogue != PP_EPI_NONE && d.epilogue != PP_EPI_ACCUM_F32 && d.epilogue != PP_EPI_ACCUM_ROUNDED)
                return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_grouped: epilogue %d with fp32 C", d.epilogue);
            if (f32_class(d.epilogue) != f32_class(f.epilogue))
                return fail(PP_ERR_INVALID, "pp_gemm_bf16_grouped: problem %d mixes plain and accumulating fp32 outputs", i);
        } else if (d.epilogue < PP_EPI_NONE || d.epilogue > PP_EPI_DRELU || d.epilogue == PP_EPI_ACCUM_F32) {
            return fail(PP_ERR_UNSUPPORTED, "pp_gemm_bf16_grouped: epilogue %d with bf16 C", d.epilogue);
        }
        GemmArgs g;
        bool empty;
        int rc = convert(&d, &g, &empty);
        if (rc) return rc;
        if (!empty) probs.push_back(g);
    }
    if (probs.empty()) return PP_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int at = f.a_trans ? 1 : 0, bt = f.b_trans ? 1 : 0;
    if (probs.size() == 1)
        return gemm_dispatch_single(probs[0], at, bt, f.epilogue, cf32, st);
    // launches of at most PP_GEMM_MAX_GROUP problems, of about equal length
    const int total = (int)probs.size();
    const int launches = (total + PP_GEMM_MAX_GROUP - 1) / PP_GEMM_MAX_GROUP;
    int done = 0;
    for (int l = 0; l < launches; ++l) {
        const int cnt = (total - done + (launches - l) - 1) / (launches - l);
        GemmGroupArgs ga;
        ga.n = cnt;
        for (int i = 0; i < cnt; ++i) ga.p[i] = probs[done + i];
        done += cnt;
        int rc;
        if (!cf32) rc = launch_layout<kEpiRuntime, false>(ga, at, bt, st);
        else if (f.epilogue == PP_EPI_NONE) rc = launch_layout<PP_EPI_NONE, true>(ga, at, bt, st);
        else rc = launch_layout<PP_EPI_ACCUM_F32, true>(ga, at, bt, st);
        if (rc) return rc;
    }
    return PP_OK;
}
