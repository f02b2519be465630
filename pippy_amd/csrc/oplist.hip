// Launch list: replays a host array of tagged descriptors on one stream.  A pipeline stage
// compiles its forward / input-gradient / weight-gradient pass for one microbatch into such a
// list once, so that a pass costs one call from the host language instead of one per kernel.
#include "common.h"
#include <vector>

using namespace pp;

static pp_gemm_desc gemm_desc_of(const pp_op& op) {
    pp_gemm_desc d;
    d.A = op.p[0]; d.B = op.p[1]; d.C = op.p[2];
    d.bias = op.p[3]; d.aux_in = op.p[4]; d.aux_out = op.p[5];
    d.M = op.i[0]; d.N = op.i[1]; d.K = op.i[2];
    d.lda = op.i[3]; d.ldb = op.i[4]; d.ldc = op.i[5]; d.ld_aux = op.i[6];
    d.a_trans = op.j[0]; d.b_trans = op.j[1]; d.epilogue = op.j[2]; d.c_dtype = op.j[3];
    d.beta = op.j[4]; d.reserved = 0;
    d.colsum = op.kind == PP_OP_GEMM_BF16 ? static_cast<float*>(op.p[9]) : nullptr;
    return d;
}

// Number of ops starting at ops[i] that can go into one grouped GEMM launch (0: not groupable).
static int group_length(const pp_op* ops, int i, int n_ops) {
    const pp_op& f = ops[i];
    if (f.kind != PP_OP_GEMM_BF16 || !(f.flags & PP_OP_GROUPED) || (f.flags & PP_OP_SKIP)) return 0;
    int len = 1;
    while (i + len < n_ops) {
        const pp_op& o = ops[i + len];
        if (o.kind != PP_OP_GEMM_BF16 || !(o.flags & PP_OP_GROUPED) || (o.flags & PP_OP_SKIP)) break;
        if (o.j[0] != f.j[0] || o.j[1] != f.j[1] || o.j[2] != f.j[2] || o.j[3] != f.j[3]) break;
        ++len;
    }
    return len;
}

// Number of consecutive weight-gradient ops over several microbatches (same segment count) from ops[i].
static int kseg_group_length(const pp_op* ops, int i, int n_ops) {
    if (ops[i].kind != PP_OP_GEMM_KSEG || (ops[i].flags & PP_OP_SKIP)) return 0;
    int len = 1;
    while (i + len < n_ops && ops[i + len].kind == PP_OP_GEMM_KSEG && !(ops[i + len].flags & PP_OP_SKIP) &&
           ops[i + len].i[7] == ops[i].i[7])
        ++len;
    return len;
}

static bool is_colreduce(const pp_op& o) {
    return (o.kind == PP_OP_COLSUM || o.kind == PP_OP_LN_BWD_WEIGHT) && (o.flags & PP_OP_GROUPED) &&
           !(o.flags & PP_OP_SKIP);
}

static int colreduce_group_length(const pp_op* ops, int i, int n_ops) {
    if (!is_colreduce(ops[i])) return 0;
    int len = 1;
    while (i + len < n_ops && is_colreduce(ops[i + len])) ++len;
    return len;
}

static pp_colreduce_desc colreduce_desc_of(const pp_op& op) {
    pp_colreduce_desc d;
    if (op.kind == PP_OP_COLSUM) {
        d.dy = op.p[0]; d.x = nullptr; d.mean = nullptr; d.rstd = nullptr;
        d.out_sum = op.p[1]; d.out_dot = nullptr;
        d.workspace = static_cast<float*>(op.p[2]);
        d.rows = op.i[0]; d.C = op.i[1]; d.ld_dy = op.i[2];
    } else {
        d.dy = op.p[0]; d.x = op.p[1];
        d.mean = static_cast<const float*>(op.p[2]); d.rstd = static_cast<const float*>(op.p[3]);
        d.out_dot = op.p[4]; d.out_sum = op.p[5];
        d.workspace = static_cast<float*>(op.p[6]);
        d.rows = op.i[0]; d.C = op.i[1]; d.ld_dy = op.i[1];
    }
    d.out_dtype = op.j[0];
    d.n_part_ready = op.j[1];
    return d;
}

static int run_one(const pp_op& op, pp_stream st) {
    switch (op.kind) {
        case PP_OP_GEMM_BF16:
        case PP_OP_GEMM_F32: {
            const pp_gemm_desc d = gemm_desc_of(op);
            if (op.kind == PP_OP_GEMM_BF16 && op.p[8])  // a workspace for a split along K
                return pp_gemm_bf16_splitk(&d, static_cast<float*>(op.p[8]), op.i[10], st);
            return op.kind == PP_OP_GEMM_BF16 ? pp_gemm_bf16(&d, st) : pp_gemm_f32(&d, st);
        }
        case PP_OP_COLSUM:
            if (op.j[1] > 0) {  // partial sums are there already: only the grouped call takes them
                const pp_colreduce_desc d = colreduce_desc_of(op);
                return pp_colreduce_grouped(&d, 1, st);
            }
            return pp_colsum_bf16(op.p[0], op.i[0], op.i[1], op.i[2], op.p[1], op.j[0],
                                  static_cast<float*>(op.p[2]), st);
        case PP_OP_LN_FWD:
            return pp_layernorm_fwd(op.p[0], op.p[1], op.p[2], op.p[3], static_cast<float*>(op.p[4]),
                                    static_cast<float*>(op.p[5]), op.i[0], op.i[1], op.f[0], st);
        case PP_OP_LN_BWD_INPUT:
            return pp_layernorm_bwd_input_sums(op.p[0], op.p[1], op.p[2], static_cast<const float*>(op.p[3]),
                                               static_cast<const float*>(op.p[4]), op.p[5], op.p[6], op.i[0],
                                               op.i[1], static_cast<float*>(op.p[7]), static_cast<float*>(op.p[8]),
                                               st);
        case PP_OP_LN_BWD_WEIGHT:
            if (op.j[1] > 0) {
                const pp_colreduce_desc d = colreduce_desc_of(op);
                return pp_colreduce_grouped(&d, 1, st);
            }
            return pp_layernorm_bwd_weight(op.p[0], op.p[1], static_cast<const float*>(op.p[2]),
                                           static_cast<const float*>(op.p[3]), op.p[4], op.p[5], op.j[0],
                                           static_cast<float*>(op.p[6]), op.i[0], op.i[1], st);
        case PP_OP_ATTN_FWD:
        case PP_OP_ATTN_BWD: {
            pp_attn_desc d;
            d.q = op.p[0]; d.k = op.p[1]; d.v = op.p[2]; d.o = op.p[3];
            d.lse = static_cast<float*>(op.p[4]); d.d_o = op.p[5];
            d.dq = op.p[6]; d.dk = op.p[7]; d.dv = op.p[8]; d.delta = static_cast<float*>(op.p[9]);
            d.B = op.i[0]; d.S = op.i[1]; d.H = op.i[2]; d.D = op.i[3];
            d.stride_b = op.i[4]; d.stride_s = op.i[5];
            d.scale = op.f[0]; d.causal = op.j[0]; d.kv_group = op.j[1]; d.kv_len = op.j[2]; d.flags = op.j[3];
            d.colsum = static_cast<float*>(op.p[10]); d.ld_colsum = op.i[6];
            return op.kind == PP_OP_ATTN_FWD ? pp_attn_fwd(&d, st) : pp_attn_bwd(&d, st);
        }
        case PP_OP_POSITION_IDS:
            return pp_position_ids_from_padding(static_cast<const int64_t*>(op.p[0]), static_cast<int64_t*>(op.p[1]),
                                                op.i[0], op.i[1], op.i[2], st);
        case PP_OP_EMBED_FWD:
            if (op.p[5])
                return pp_embed_fwd_at(static_cast<const int64_t*>(op.p[0]), static_cast<const int64_t*>(op.p[5]),
                                       op.p[1], op.p[2], op.p[4], op.p[3], op.i[0], op.i[4], op.i[2], op.i[3], st);
            return pp_embed_fwd(static_cast<const int64_t*>(op.p[0]), op.p[1], op.p[2], op.p[4], op.p[3], op.i[0],
                                op.i[1], op.i[2], op.i[3], st);
        case PP_OP_EMBED_BWD:
            return pp_embed_bwd(static_cast<const int64_t*>(op.p[0]), op.p[1], static_cast<float*>(op.p[2]),
                                static_cast<float*>(op.p[3]), op.i[0], op.i[1], op.i[2], op.i[3], op.j[0],
                                op.i[4] - 1, st);
        case PP_OP_CE_LOSS:
            return pp_ce_loss(op.p[0], static_cast<const int64_t*>(op.p[1]), static_cast<float*>(op.p[2]),
                              op.p[3], static_cast<float*>(op.p[4]), op.i[0], op.i[1], op.i[2], op.i[3],
                              op.j[0], st);
        case PP_OP_ACCUM_BF16:
            return pp_grad_accum_f32_bf16(static_cast<float*>(op.p[0]), static_cast<const uint16_t*>(op.p[1]),
                                          op.i[0], op.j[0], st);
        case PP_OP_ACCUM_F32:
            return pp_grad_accum_f32_f32(static_cast<float*>(op.p[0]), static_cast<const float*>(op.p[1]),
                                         op.i[0], op.j[0], st);
        case PP_OP_COPY_ROWS: {
            pp_copy_seg s;
            s.src = op.p[0]; s.dst = op.p[1];
            s.n_rows = op.i[0]; s.row_bytes = op.i[1]; s.src_stride = op.i[2]; s.dst_stride = op.i[3];
            return pp_copy_rows(&s, 1, st);
        }
        case PP_OP_FILL:
            return pp_fill_bytes(op.p[0], op.j[0], op.i[0], st);
        case PP_OP_ACT_BWD:
            return pp_activation_bwd(op.p[0], op.p[1], op.p[2], op.i[0], op.j[0], op.j[1], st);
        case PP_OP_SWIGLU_FWD:
            return pp_swiglu_fwd(op.p[0], op.p[1], op.p[2], op.i[0], st);
        case PP_OP_SWIGLU_BWD:
            return pp_swiglu_bwd(op.p[0], op.p[1], op.p[2], op.p[3], op.p[4], op.i[0], st);
        case PP_OP_GEMM_SWIGLU:
            return pp_gemm_bf16_swiglu(op.p[0], op.p[1], op.p[2], op.p[3], op.p[4], op.i[0], op.i[1], op.i[2], op.i[3],
                                       op.i[4], op.i[5], op.i[6], st);
        case PP_OP_GEMM_DSWIGLU:
            return pp_gemm_bf16_dswiglu(op.p[0], op.p[1], op.p[2], op.p[3], op.i[0], op.i[1], op.i[2], op.i[3], op.i[4],
                                        op.i[5], op.i[6], st);
        case PP_OP_GEMM_SEG_SWIGLU:
            return pp_gemm_bf16_segmented_swiglu(op.p[0], static_cast<const void* const*>(op.p[1]),
                                                 static_cast<const void* const*>(op.p[2]),
                                                 static_cast<const int32_t*>(op.p[5]), (int)op.i[7], op.p[3], op.p[4],
                                                 op.i[0], op.i[1], op.i[2], op.i[3], op.i[4], op.i[5], op.i[6], st);
        case PP_OP_GEMM_SEG_DSWIGLU:
            return pp_gemm_bf16_segmented_dswiglu(op.p[0], static_cast<const void* const*>(op.p[1]),
                                                  static_cast<const int32_t*>(op.p[4]), (int)op.i[7], op.p[2], op.p[3],
                                                  op.i[0], op.i[1], op.i[2], op.i[3], op.i[4], op.i[5], op.i[6], st);
        case PP_OP_ROPE:
            return pp_rope(op.p[0], static_cast<const float*>(op.p[1]), static_cast<const float*>(op.p[2]),
                           op.i[0], op.i[1], op.i[2], op.i[3], op.i[4], op.j[0], st);
        case PP_OP_GEMM_SEG: {
            const pp_gemm_desc d = gemm_desc_of(op);
            return pp_gemm_bf16_segmented(&d, static_cast<const int32_t*>(op.p[6]),
                                          static_cast<const void* const*>(op.p[7]), (int)op.i[7], op.j[5], st);
        }
        case PP_OP_GEMM_SEG_KSEG: {
            const pp_gemm_desc d = gemm_desc_of(op);
            return pp_gemm_bf16_segmented_kseg(&d, static_cast<const void* const*>(op.p[0]),
                                               static_cast<const void* const*>(op.p[1]),
                                               static_cast<const int32_t* const*>(op.p[6]),
                                               static_cast<const void* const*>(op.p[7]), (int)op.i[7], (int)op.i[8], st);
        }
        case PP_OP_MOE_ROUTER:
            return pp_moe_router_top2(op.p[0], op.i[0], op.i[1], (int)op.i[2], static_cast<int32_t*>(op.p[1]),
                                      static_cast<float*>(op.p[2]), st);
        case PP_OP_MOE_PERMUTE:
            return pp_moe_permute(static_cast<const int32_t*>(op.p[0]), op.i[0], (int)op.i[1],
                                  static_cast<int32_t*>(op.p[1]), static_cast<int32_t*>(op.p[2]),
                                  static_cast<int32_t*>(op.p[3]), st);
        case PP_OP_MOE_GATHER:
            return pp_moe_gather(op.p[0], op.i[0], static_cast<const int32_t*>(op.p[1]),
                                 static_cast<const int32_t*>(op.p[2]), (int)op.i[1],
                                 static_cast<const float*>(op.p[3]), op.p[4], op.i[2], op.i[3], op.i[4], st);
        case PP_OP_MOE_COMBINE:
            return pp_moe_combine(op.p[0], op.i[0], static_cast<const int32_t*>(op.p[1]),
                                  static_cast<const float*>(op.p[2]), (int)op.i[1], op.p[3], op.i[2], op.p[4],
                                  op.i[3], op.i[4], op.i[5], st);
        case PP_OP_MOE_GATE_BWD:
            return pp_moe_gate_bwd(op.p[0], op.i[0], op.p[1], op.i[1], static_cast<const int32_t*>(op.p[2]),
                                   static_cast<const int32_t*>(op.p[3]), static_cast<const float*>(op.p[4]),
                                   (int)op.i[2], (int)op.i[3], op.p[5], op.i[4], op.i[5], op.i[6], st);
        default:
            return fail(PP_ERR_INVALID, "unknown op kind %d", op.kind);
    }
}

// ---- per-launch timing with HIP events ---------------------------------------------------------
// When a profile is active every executed op is bracketed by two events recorded on the op's own
// stream; pp_profile_read synchronises and sums elapsed time and algorithmic work per op kind.
namespace {
struct ProfRecord {
    hipEvent_t a, b;
    int kind;
    double work;
};
std::vector<ProfRecord> g_prof;
size_t g_prof_used = 0;
bool g_prof_on = false;
long long g_prof_dropped = 0;

// Algorithmic work of one op: FLOPs for MFMA-bound kinds, bytes for HBM-bound kinds.
double op_work(const pp_op& op) {
    switch (op.kind) {
        case PP_OP_GEMM_BF16:
        case PP_OP_GEMM_F32:
        case PP_OP_GEMM_DSWIGLU:
        case PP_OP_GEMM_SEG_DSWIGLU:
        case PP_OP_GEMM_SEG:  // the segments partition the rows (rows mode: M, k mode: K)
            return 2.0 * (double)op.i[0] * (double)op.i[1] * (double)op.i[2];
        case PP_OP_GEMM_SEG_KSEG:  // per microbatch the segments partition K (the upper bound given in i[2])
            return 2.0 * (double)op.i[0] * (double)op.i[1] * (double)op.i[2] * (double)op.i[8];
        case PP_OP_GEMM_KSEG:  // one product per segment
            return 2.0 * (double)op.i[0] * (double)op.i[1] * (double)op.i[2] * (double)op.i[7];
        case PP_OP_GEMM_SWIGLU:  // two products of N columns each
        case PP_OP_GEMM_SEG_SWIGLU:
            return 4.0 * (double)op.i[0] * (double)op.i[1] * (double)op.i[2];
        case PP_OP_ATTN_FWD:  // dense count: QK^T and PV
            return 4.0 * (double)op.i[0] * (double)op.i[2] * (double)op.i[1] * (double)op.i[1] * (double)op.i[3];
        case PP_OP_ATTN_BWD:  // dQ, dK, dV, dP and the recomputed scores
            return 10.0 * (double)op.i[0] * (double)op.i[2] * (double)op.i[1] * (double)op.i[1] * (double)op.i[3];
        case PP_OP_ACCUM_BF16:
            return (double)op.i[0] * (op.j[0] ? 6.0 : 10.0);
        case PP_OP_ACCUM_F32:
            return (double)op.i[0] * (op.j[0] ? 8.0 : 12.0);
        case PP_OP_COPY_ROWS:
            return 2.0 * (double)op.i[0] * (double)op.i[1];
        case PP_OP_LN_FWD:
            return 4.0 * (double)op.i[0] * (double)op.i[1];  // read x, write y (bf16)
        case PP_OP_LN_BWD_INPUT:
            return (op.p[5] ? 8.0 : 6.0) * (double)op.i[0] * (double)op.i[1];
        case PP_OP_LN_BWD_WEIGHT:  // dy and x, or the partial sums that their producer left
            return op.j[1] > 0 ? 8.0 * (double)op.j[1] * (double)op.i[1] : 4.0 * (double)op.i[0] * (double)op.i[1];
        case PP_OP_COLSUM:
            return op.j[1] > 0 ? 4.0 * (double)op.j[1] * (double)op.i[1] : 2.0 * (double)op.i[0] * (double)op.i[1];
        case PP_OP_CE_LOSS:  // read logits, write their gradient
            return (op.p[3] ? 2.0 : 1.0) * (double)op.i[0] * (double)op.i[2] * (op.j[0] == PP_F32 ? 4.0 : 2.0);
        case PP_OP_EMBED_FWD:
            return 6.0 * (double)op.i[0] * (double)op.i[2];
        case PP_OP_EMBED_BWD:
            return 10.0 * (double)op.i[0] * (double)op.i[2];
        case PP_OP_FILL:
            return (double)op.i[0];
        case PP_OP_ACT_BWD:
            return 3.0 * (double)op.i[0] * (op.j[1] == PP_F32 ? 4.0 : 2.0);
        case PP_OP_SWIGLU_FWD:
            return 6.0 * (double)op.i[0];
        case PP_OP_SWIGLU_BWD:
            return 10.0 * (double)op.i[0];
        case PP_OP_ROPE:
            return 4.0 * (double)op.i[0] * (double)op.i[2] * (double)op.i[3];
        case PP_OP_MOE_GATHER:  // read and write R rows of C bf16
            return 4.0 * (double)op.i[3] * (double)op.i[4];
        case PP_OP_MOE_COMBINE:  // read topk rows (+ the residual), write one, per token
            return 2.0 * ((double)op.i[1] + (op.p[3] ? 2.0 : 1.0)) * (double)op.i[4] * (double)op.i[5];
        default:
            return 0.0;
    }
}
}  // namespace

extern "C" int pp_profile_start(int max_records) {
    if (max_records <= 0) return fail(PP_ERR_INVALID, "pp_profile_start: max_records <= 0");
    if (g_prof.size() < (size_t)max_records) {
        const size_t old = g_prof.size();
        g_prof.resize((size_t)max_records);
        for (size_t i = old; i < g_prof.size(); ++i) {
            if (hipEventCreate(&g_prof[i].a) != hipSuccess || hipEventCreate(&g_prof[i].b) != hipSuccess) {
                g_prof.resize(i);
                return fail(PP_ERR_LAUNCH, "pp_profile_start: cannot create events");
            }
        }
    }
    g_prof_used = 0;
    g_prof_dropped = 0;
    g_prof_on = true;
    return PP_OK;
}

extern "C" int pp_profile_stop(void) {
    g_prof_on = false;
    return PP_OK;
}

extern "C" int pp_profile_read(int kind, double* total_ms, double* total_work, int64_t* count) {
    if (!total_ms || !total_work || !count) return fail(PP_ERR_INVALID, "pp_profile_read: null pointer");
    *total_ms = 0.0;
    *total_work = 0.0;
    *count = 0;
    for (size_t i = 0; i < g_prof_used; ++i) {
        const ProfRecord& r = g_prof[i];
        if (r.kind != kind) continue;
        if (hipEventSynchronize(r.b) != hipSuccess) return fail(PP_ERR_LAUNCH, "pp_profile_read: event sync failed");
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, r.a, r.b) != hipSuccess) return fail(PP_ERR_LAUNCH, "pp_profile_read: elapsed failed");
        *total_ms += ms;
        *total_work += r.work;
        *count += 1;
    }
    if (g_prof_dropped) return fail(PP_ERR_UNSUPPORTED, "pp_profile_read: %lld ops were not recorded (pool too small)", g_prof_dropped);
    return PP_OK;
}

extern "C" int pp_run_ops(const pp_op* ops, int n_ops, pp_stream stream) {
    if (n_ops < 0 || (n_ops > 0 && !ops)) return fail(PP_ERR_INVALID, "pp_run_ops: bad list");
    for (int i = 0; i < n_ops; ++i) {
        if (ops[i].flags & PP_OP_SKIP) continue;
        int glen = group_length(ops, i, n_ops);
        const int clen = glen ? 0 : colreduce_group_length(ops, i, n_ops);
        if (clen > 1) glen = clen;
        const int klen = kseg_group_length(ops, i, n_ops);
        if (klen) glen = klen;
        ProfRecord* rec = nullptr;
        if (g_prof_on) {
            if (g_prof_used < g_prof.size()) {
                rec = &g_prof[g_prof_used++];
                rec->kind = ops[i].kind;
                rec->work = op_work(ops[i]);
                for (int q = 1; q < glen; ++q) rec->work += op_work(ops[i + q]);
                (void)hipEventRecord(rec->a, static_cast<hipStream_t>(stream));
            } else {
                ++g_prof_dropped;
            }
        }
        int rc;
        if (klen) {
            std::vector<pp_gemm_desc> descs;
            descs.reserve(klen);
            for (int q = 0; q < klen; ++q) descs.push_back(gemm_desc_of(ops[i + q]));
            rc = pp_gemm_bf16_grouped_kseg(descs.data(), klen, (int)ops[i].i[7], stream);
        } else if (clen > 1) {
            std::vector<pp_colreduce_desc> descs;
            descs.reserve(clen);
            for (int q = 0; q < clen; ++q) descs.push_back(colreduce_desc_of(ops[i + q]));
            rc = pp_colreduce_grouped(descs.data(), clen, stream);
        } else if (glen > 1) {
            std::vector<pp_gemm_desc> descs;
            descs.reserve(glen);
            for (int q = 0; q < glen; ++q) descs.push_back(gemm_desc_of(ops[i + q]));
            rc = pp_gemm_bf16_grouped(descs.data(), glen, stream);
        } else {
            rc = run_one(ops[i], stream);
        }
        if (rec) (void)hipEventRecord(rec->b, static_cast<hipStream_t>(stream));
        if (rc != PP_OK) {
            char msg[400];
            snprintf(msg, sizeof msg, "%s", pp_last_error());
            return fail(rc, "pp_run_ops: op %d (kind %d): %s", i, ops[i].kind, msg);
        }
        if (glen > 1) i += glen - 1;
    }
    return PP_OK;
}
