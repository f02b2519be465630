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
    d.reserved = 0;
    return d;
}

static int run_one(const pp_op& op, pp_stream st) {
    switch (op.kind) {
        case PP_OP_GEMM_BF16:
        case PP_OP_GEMM_F32: {
            const pp_gemm_desc d = gemm_desc_of(op);
            return op.kind == PP_OP_GEMM_BF16 ? pp_gemm_bf16(&d, st) : pp_gemm_f32(&d, st);
        }
        case PP_OP_COLSUM:
            return pp_colsum_bf16(op.p[0], op.i[0], op.i[1], op.i[2], op.p[1], op.j[0],
                                  static_cast<float*>(op.p[2]), st);
        case PP_OP_LN_FWD:
            return pp_layernorm_fwd(op.p[0], op.p[1], op.p[2], op.p[3], static_cast<float*>(op.p[4]),
                                    static_cast<float*>(op.p[5]), op.i[0], op.i[1], op.f[0], st);
        case PP_OP_LN_BWD_INPUT:
            return pp_layernorm_bwd_input(op.p[0], op.p[1], op.p[2], static_cast<const float*>(op.p[3]),
                                          static_cast<const float*>(op.p[4]), op.p[5], op.p[6], op.i[0],
                                          op.i[1], st);
        case PP_OP_LN_BWD_WEIGHT:
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
            d.scale = op.f[0]; d.causal = op.j[0];
            return op.kind == PP_OP_ATTN_FWD ? pp_attn_fwd(&d, st) : pp_attn_bwd(&d, st);
        }
        case PP_OP_EMBED_FWD:
            return pp_embed_fwd(static_cast<const int64_t*>(op.p[0]), op.p[1], op.p[2], op.p[4], op.p[3], op.i[0],
                                op.i[1], op.i[2], op.i[3], st);
        case PP_OP_EMBED_BWD:
            return pp_embed_bwd(static_cast<const int64_t*>(op.p[0]), op.p[1], static_cast<float*>(op.p[2]),
                                static_cast<float*>(op.p[3]), op.i[0], op.i[1], op.i[2], op.i[3], st);
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
        case PP_OP_ROPE:
            return pp_rope(op.p[0], static_cast<const float*>(op.p[1]), static_cast<const float*>(op.p[2]),
                           op.i[0], op.i[1], op.i[2], op.i[3], op.i[4], op.j[0], st);
        case PP_OP_GEMM_SEG: {
            const pp_gemm_desc d = gemm_desc_of(op);
            return pp_gemm_bf16_segmented(&d, static_cast<const int32_t*>(op.p[6]),
                                          static_cast<const void* const*>(op.p[7]), (int)op.i[7], op.j[5], st);
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
        case PP_OP_GEMM_SEG:  // the segments partition the rows (rows mode: M, k mode: K)
            return 2.0 * (double)op.i[0] * (double)op.i[1] * (double)op.i[2];
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
        case PP_OP_LN_BWD_WEIGHT:
            return 4.0 * (double)op.i[0] * (double)op.i[1];
        case PP_OP_COLSUM:
            return 2.0 * (double)op.i[0] * (double)op.i[1];
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
        if (clen > 1) {
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

// ---- launch lists replayed as HIP graphs ------------------------------------------------------
// A launch list is a fixed sequence of kernel launches (no allocation, no memset, no host
// synchronisation), so once its descriptors stop changing it can be captured into a graph and
// replayed with one call.  The cache is keyed by a hash of the descriptor bytes: patching a pointer
// or a flag of the list simply selects (or creates) another graph.
namespace pp {

struct GraphEntry {
    uint64_t hash = 0;
    int n_ops = 0;
    int seen = 0;          // eager runs of exactly this content
    bool refused = false;  // capture failed once: stay eager
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    uint64_t last_use = 0;
};

struct GraphCache {
    std::vector<GraphEntry> entries;
    uint64_t clock = 0;
};

constexpr size_t kMaxGraphsPerList = 6;
constexpr int kEagerRunsBeforeCapture = 2;

// A graph pays when the list is bound by launching its kernels, not by running them: measured on
// this part, a 2-stage decoder of width 128 steps 2.8 times faster with graphs (1.7 against 4.8 ms),
// lists of two to four kernels run slower (one graph launch costs more than a few kernel launches)
// and the GPT-2-small step, whose kernels average 40 us, loses 1 %.  The estimate below prices
// MFMA-bound ops at 400 TFLOP/s and the others at 3 TB/s.
constexpr int kMinOpsForGraph = 8;
constexpr double kMaxAvgOpMicrosForGraph = 8.0;

static bool launch_bound(const pp_op* ops, int n) {
    int launches = 0;
    double us = 0.0;
    for (int i = 0; i < n; ++i) {
        if (ops[i].flags & PP_OP_SKIP) continue;
        ++launches;
        const int k = ops[i].kind;
        const bool mfma = k == PP_OP_GEMM_BF16 || k == PP_OP_GEMM_F32 || k == PP_OP_GEMM_SEG ||
                          k == PP_OP_ATTN_FWD || k == PP_OP_ATTN_BWD;
        us += op_work(ops[i]) / (mfma ? 400e6 : 3e6);
    }
    return launches >= kMinOpsForGraph && us <= kMaxAvgOpMicrosForGraph * launches;
}

static uint64_t hash_ops(const pp_op* ops, int n) {
    // FNV-1a over 64-bit words (pp_op is a multiple of 8 bytes)
    static_assert(sizeof(pp_op) % 8 == 0, "pp_op hashes as 64-bit words");
    const uint64_t* w = reinterpret_cast<const uint64_t*>(ops);
    const size_t nw = (size_t)n * sizeof(pp_op) / 8;
    uint64_t h = 1469598103934665603ull ^ (uint64_t)n;
    for (size_t i = 0; i < nw; ++i) {
        h ^= w[i];
        h *= 1099511628211ull;
    }
    return h;
}

static void release(GraphEntry& e) {
    if (e.exec) (void)hipGraphExecDestroy(e.exec);
    if (e.graph) (void)hipGraphDestroy(e.graph);
    e.exec = nullptr;
    e.graph = nullptr;
}

}  // namespace pp

extern "C" int pp_graph_cache_create(pp_graph_cache* out) {
    if (!out) return fail(PP_ERR_INVALID, "pp_graph_cache_create: null pointer");
    *out = new GraphCache();
    return PP_OK;
}

extern "C" int pp_graph_cache_destroy(pp_graph_cache cache) {
    GraphCache* c = static_cast<GraphCache*>(cache);
    if (!c) return PP_OK;
    for (GraphEntry& e : c->entries) release(e);
    delete c;
    return PP_OK;
}

extern "C" int pp_graph_cache_size(pp_graph_cache cache) {
    GraphCache* c = static_cast<GraphCache*>(cache);
    int n = 0;
    if (c)
        for (const GraphEntry& e : c->entries) n += e.exec != nullptr;
    return n;
}

extern "C" int pp_run_ops_graphed(const pp_op* ops, int n_ops, pp_stream stream, pp_graph_cache cache,
                                  int always) {
    GraphCache* c = static_cast<GraphCache*>(cache);
    hipStream_t st = static_cast<hipStream_t>(stream);
    // the default stream cannot be captured; per-op timing needs the ops as separate launches
    if (!c || !st || g_prof_on || n_ops <= 0) return pp_run_ops(ops, n_ops, stream);
    const uint64_t h = hash_ops(ops, n_ops);
    GraphEntry* e = nullptr;
    for (GraphEntry& x : c->entries)
        if (x.hash == h && x.n_ops == n_ops) e = &x;
    if (!e) {
        if (c->entries.size() >= kMaxGraphsPerList) {
            size_t victim = 0;
            for (size_t i = 1; i < c->entries.size(); ++i)
                if (c->entries[i].last_use < c->entries[victim].last_use) victim = i;
            release(c->entries[victim]);
            c->entries.erase(c->entries.begin() + victim);
        }
        c->entries.emplace_back();
        e = &c->entries.back();
        e->hash = h;
        e->n_ops = n_ops;
        e->refused = !always && !launch_bound(ops, n_ops);
    }
    e->last_use = ++c->clock;
    if (e->exec) {
        if (hipGraphLaunch(e->exec, st) != hipSuccess) return fail(PP_ERR_LAUNCH, "pp_run_ops_graphed: graph launch failed");
        return PP_OK;
    }
    if (e->refused || e->seen < kEagerRunsBeforeCapture) {
        ++e->seen;
        return pp_run_ops(ops, n_ops, stream);
    }
    // Every kernel of this list has run eagerly before (one-time function attributes are set), so
    // the capture records launches only; nothing executes until the graph is launched below.
    if (hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal) != hipSuccess) {
        (void)hipGetLastError();
        e->refused = true;
        return pp_run_ops(ops, n_ops, stream);
    }
    const int rc = pp_run_ops(ops, n_ops, stream);
    hipGraph_t graph = nullptr;
    const hipError_t end = hipStreamEndCapture(st, &graph);
    if (rc != PP_OK || end != hipSuccess || !graph) {
        (void)hipGetLastError();
        if (graph) (void)hipGraphDestroy(graph);
        e->refused = true;
        if (rc != PP_OK) return rc;  // a bad descriptor: the message is already set
        return pp_run_ops(ops, n_ops, stream);
    }
    hipGraphExec_t exec = nullptr;
    if (hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) != hipSuccess || !exec) {
        (void)hipGetLastError();
        (void)hipGraphDestroy(graph);
        e->refused = true;
        return pp_run_ops(ops, n_ops, stream);
    }
    e->graph = graph;
    e->exec = exec;
    if (hipGraphLaunch(exec, st) != hipSuccess) return fail(PP_ERR_LAUNCH, "pp_run_ops_graphed: graph launch failed");
    return PP_OK;
}
