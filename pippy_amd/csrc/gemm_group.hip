// Grouped bf16 GEMM launches: several independent problems in one grid (see gemm_core.h for the
// kernel).  Two families:
//   * problems with a bf16 C, whatever their epilogues: one kernel that takes each problem's epilogue at
//     run time, so the GEMMs that several pipeline stages reach at the same position of their passes go
//     out together (forward and input-gradient GEMMs of different virtual stages);
//   * problems that add to (or write) an fp32 C: the weight-gradient GEMMs of one or more passes.
#include "gemm_core.h"
#include <vector>

namespace pp {

template <int BM, int BN, bool AT, bool BT, int NS, int EPI, bool CF32, int KT>
static int launch_group(GemmGroupArgs& ga, hipStream_t st) {
    constexpr size_t lds = (size_t)NS * (BM + BN) * KT * sizeof(uint16_t);
    static const int attr_rc = reserve_lds(&gemm_bf16_group_kernel<BM, BN, AT, BT, NS, EPI, CF32, KT>, lds);
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
    hipLaunchKernelGGL((gemm_bf16_group_kernel<BM, BN, AT, BT, NS, EPI, CF32, KT>), dim3(grid), dim3(kGemmThreads),
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
// 256 x 256 with 2 to 4 stages of 32 or 64 k: none ran a forward-shaped group faster than 128 x 128,
// and the weight-gradient groups gained 2 % at best.)
template <bool AT, bool BT, int EPI, bool CF32>
static int launch_auto(GemmGroupArgs& ga, hipStream_t st) {
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

}  // namespace pp

using namespace pp;

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
