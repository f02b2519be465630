/*
 * pippy_amd.h -- C ABI of the MI355X (gfx950) kernels behind the PiPPy-compatible
 * pipeline-stage hot path.
 *
 * The reference (pytorch/PiPPy 0.2.0) is pure Python and reaches all arithmetic through
 * torch calls; it has no FFI of its own.  Each entry point below names the reference call
 * site (file:line under the reference tree) whose torch call it replaces.
 *
 * Conventions
 *   - every pointer is a device pointer unless a comment says "host";
 *   - `stream` is a hipStream_t passed as void*; every launch is asynchronous on it;
 *   - functions return PP_OK (0) or a PP_ERR_* code and never throw; pp_last_error() returns
 *     a thread-local, human-readable description of the last failure;
 *   - no entry point allocates or frees device memory: outputs and workspaces are
 *     caller-provided;
 *   - bf16 values are raw uint16 bit patterns (upper half of an IEEE fp32).
 */
#ifndef PIPPY_AMD_H
#define PIPPY_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PP_OK 0
#define PP_ERR_INVALID 1     /* bad argument (null pointer, negative size, misalignment) */
#define PP_ERR_UNSUPPORTED 2 /* shape / layout / dtype combination not implemented */
#define PP_ERR_LAUNCH 3      /* HIP reported an error at launch */

typedef void* pp_stream;

int pp_abi_version(void);
const char* pp_last_error(void);

/* ------------------------------------------------------------------------------------------
 * Microbatch split / merge.
 *   split: pippy/microbatch.py:139-141  torch.tensor_split(v, n, dim)   (made contiguous)
 *   merge: pippy/microbatch.py:415      torch.cat(values, dim)
 * Both are row copies: a tensor of shape [outer, dim, inner] is `outer` rows per chunk, each a
 * contiguous run of dim_chunk*inner elements.  Bit-exact for any element type (bytes move).
 * ---------------------------------------------------------------------------------------- */
typedef struct pp_copy_seg {
    const void* src;
    void* dst;
    int64_t n_rows;     /* rows to copy */
    int64_t row_bytes;  /* contiguous bytes per row */
    int64_t src_stride; /* bytes between consecutive source rows */
    int64_t dst_stride; /* bytes between consecutive destination rows */
} pp_copy_seg;

#define PP_COPY_MAX_SEGS 64

/* Copies up to PP_COPY_MAX_SEGS independent row segments in one launch.  `segs` is a HOST array. */
int pp_copy_rows(const pp_copy_seg* segs, int n_segs, pp_stream stream);

/* src: contiguous [outer, dim, inner_bytes]; dsts[i] (host array of device pointers): contiguous
 * [outer, dim_i, inner_bytes] with dim_i from the tensor_split rule (the first dim % n_chunks
 * chunks get ceil(dim / n_chunks), the rest floor).  Requires 1 <= n_chunks <= PP_COPY_MAX_SEGS. */
int pp_split_copy(const void* src, void* const* dsts, int n_chunks, int64_t outer, int64_t dim,
                  int64_t inner_bytes, pp_stream stream);

/* srcs[i] (host array): contiguous [outer, chunk_dims[i], inner_bytes]; dst: contiguous
 * [outer, sum(chunk_dims), inner_bytes]. */
int pp_merge_copy(void* dst, const void* const* srcs, const int64_t* chunk_dims, int n_chunks,
                  int64_t outer, int64_t inner_bytes, pp_stream stream);

/* Generic strided gather of an N-d view (ndim <= 8) into a contiguous destination; one element
 * (elem_bytes in {1,2,4,8,16}) per lane.  Used for inputs that are not contiguous to begin with.
 * `sizes` / `src_strides` (in elements) are HOST arrays. */
int pp_strided_copy_nd(void* dst, const void* src, int ndim, const int64_t* sizes,
                       const int64_t* src_strides, int elem_bytes, pp_stream stream);

/* ------------------------------------------------------------------------------------------
 * Gradient accumulation across microbatches.
 *   pippy/_backward.py:67-69 (autograd AccumulateGrad reached from torch.autograd.backward)
 *   acc[i] = (init ? 0 : acc[i]) + (float)g[i], one IEEE fp32 add per element, so the result is
 *   bit-identical to torch `acc.add_(g.float())` applied in the same microbatch order.
 * ---------------------------------------------------------------------------------------- */
int pp_grad_accum_f32_bf16(float* acc, const uint16_t* g, int64_t n, int init, pp_stream stream);
int pp_grad_accum_f32_f32(float* acc, const float* g, int64_t n, int init, pp_stream stream);
/* fills n bytes with a byte value (used instead of hipMemsetAsync so that callers may capture) */
int pp_fill_bytes(void* dst, int value, int64_t n_bytes, pp_stream stream);

/* ------------------------------------------------------------------------------------------
 * Optimizer step on the fp32 accumulators: what the reference's users run right after
 * schedule.step() (test/test_optim.py:83-99, `optim.SGD(stage.submod.parameters(), ...)`), here as
 * one launch over a stage's flat parameter range.  `param` is bf16 or fp32 (enum pp_dtype), `grad`
 * the fp32 accumulator, state buffers fp32, `master` an optional fp32 copy of bf16 parameters that
 * takes the update (param becomes its rounding) or null.  n % 4 == 0; pointers aligned to 4
 * elements.  Arithmetic follows torch.optim's single-tensor SGD / AdamW operation by operation.
 *   SGD:   d = g + wd p;  buf = first_step ? d : momentum buf + (1 - dampening) d;
 *          d = nesterov ? d + momentum buf : buf  (momentum != 0);  p -= lr d
 *   AdamW: p *= 1 - lr wd;  m += (1 - beta1)(g - m);  v = beta2 v + (1 - beta2) g g;
 *          p -= lr / bias_correction1 * m / (sqrt(v) / bias_correction2_sqrt + eps)
 * ---------------------------------------------------------------------------------------- */
int pp_sgd_step(void* param, int param_dtype, float* master, const float* grad, float* momentum_buf,
                int64_t n, float lr, float momentum, float dampening, float weight_decay, int nesterov,
                int first_step, int maximize, pp_stream stream);
int pp_adamw_step(void* param, int param_dtype, float* master, const float* grad, float* exp_avg,
                  float* exp_avg_sq, int64_t n, float lr, float beta1, float beta2, float eps,
                  float weight_decay, float bias_correction1, float bias_correction2_sqrt, int maximize,
                  pp_stream stream);

/* ------------------------------------------------------------------------------------------
 * bf16 GEMM on MFMA with fp32 accumulation and fused epilogues.
 *   forward  F.linear inside the stage module      pippy/_PipelineStage.py:420-428
 *   backward dI / dW of the same linear            pippy/_backward.py:67-69
 *   C[M,N] = epilogue( sum_k A(m,k) * B(n,k) )
 * ---------------------------------------------------------------------------------------- */
enum pp_gemm_epilogue {
    PP_EPI_NONE = 0,          /* C = acc                                                    */
    PP_EPI_BIAS = 1,          /* C = acc + bias[n]                                          */
    PP_EPI_BIAS_GELU_ERF = 2, /* aux_out = acc + bias[n] (if non-null); C = gelu_erf(that)  */
    PP_EPI_BIAS_GELU_TANH = 3,/* same with the tanh approximation                           */
    PP_EPI_BIAS_RESIDUAL = 4, /* C = acc + bias[n] + aux_in[m,n]   (bias may be null)       */
    PP_EPI_DGELU_ERF = 5,     /* C = acc * gelu_erf'(aux_in[m,n])                           */
    PP_EPI_DGELU_TANH = 6,    /* C = acc * gelu_tanh'(aux_in[m,n])                          */
    PP_EPI_ACCUM_F32 = 7,     /* C(fp32) = (beta ? C : 0) + acc     (fused grad accumulate) */
    PP_EPI_BIAS_RELU = 8,     /* C = max(acc + bias[n], 0)                                  */
    PP_EPI_DRELU = 9,         /* C = aux_in[m,n] > 0 ? acc : 0                              */
    PP_EPI_ACCUM_ROUNDED = 10 /* C(fp32) = (beta ? C : 0) + float(bf16(acc)): bit for bit what a
                                 bf16 C followed by pp_grad_accum_f32_bf16 leaves in C           */
};

enum pp_dtype { PP_BF16 = 0, PP_F32 = 1 };

typedef struct pp_gemm_desc {
    const void* A;  /* a_trans == 0: [M, K] row-major, lda >= K;  a_trans == 1: [K, M], lda >= M */
    const void* B;  /* b_trans == 0: [N, K] row-major, ldb >= K;  b_trans == 1: [K, N], ldb >= N */
    void* C;        /* [M, N] row-major, ldc >= N; bf16 unless c_dtype == PP_F32 */
    int64_t M, N, K;
    int64_t lda, ldb, ldc; /* in elements */
    int32_t a_trans, b_trans;
    int32_t epilogue;      /* enum pp_gemm_epilogue */
    int32_t c_dtype;       /* enum pp_dtype */
    const void* bias;      /* bf16 [N] or null */
    const void* aux_in;    /* bf16 [M, N] with ld_aux (residual / saved pre-activation) */
    void* aux_out;         /* bf16 [M, N] with ld_aux (pre-activation to save) or null */
    int64_t ld_aux;
    int32_t beta;          /* PP_EPI_ACCUM_F32 / _ROUNDED: 0 overwrite, 1 accumulate */
    int32_t reserved;
    float* colsum;         /* PP_EPI_DGELU_* / PP_EPI_DRELU with a bf16 C, or null: fp32
                              [ceil(M / PP_GEMM_COLSUM_ROWS), N], row r receives the column sums of rows
                              32 r .. 32 r + 31 of C as stored: partial sums of the bias gradient of the
                              layer in front of the activation, for pp_colreduce_grouped with
                              n_part_ready = ceil(M / 32) (pp_gemm_bf16 and pp_gemm_bf16_grouped only) */
} pp_gemm_desc;
#define PP_GEMM_COLSUM_ROWS 32

/* Requirements: A, B 16-byte aligned; K % 8 == 0 unless both operands are transposed (then any K: the
 * weight gradient over any number of tokens); lda, ldb % 8 == 0; a transposed operand needs
 * its contiguous extent (M resp. N) % 8 == 0; ldc, ld_aux % 4 == 0 (bf16) . */
int pp_gemm_bf16(const pp_gemm_desc* desc, pp_stream stream);

/* pp_gemm_bf16 with a workspace of `workspace_elems` floats (16-byte aligned) that lets the library
 * split a long reduction: for k-contiguous A and B, a plain bf16 C (epilogue NONE, N and ldc
 * multiples of 4) with at most 64 tiles of 256 x 256 it runs up to 8 splits of K, of at least 4096
 * each, on 256 x 256 tiles (each into its own fp32 copy of C, splits * M * N floats) and adds the copies
 * in split order; any other problem, or a workspace that is too small, runs as pp_gemm_bf16.  The
 * input-gradient GEMM of a vocabulary projection (F.linear backward with K = vocabulary) is the case
 * it is for.  The workspace must not be shared by launches that may overlap. */
int pp_gemm_bf16_splitk(const pp_gemm_desc* desc, float* workspace, int64_t workspace_elems, pp_stream stream);

/* Several independent GEMMs in one launch (longer lists go out as several launches of at most
 * PP_GEMM_MAX_GROUP problems).  All descriptors must agree in a_trans, b_trans and c_dtype.  With a bf16
 * C every problem may bring its own epilogue (any but the accumulating ones); with an fp32 C the
 * problems are either all PP_EPI_NONE or all accumulating (PP_EPI_ACCUM_F32 / _ROUNDED and beta per
 * problem).  The weight-gradient GEMMs of one stage and microbatch (pippy/_backward.py:67-69 reaches
 * them through autograd one by one) are small but independent of each other, and so are the GEMMs that
 * different pipeline stages reach at the same point of their passes (pippy/_PipelineStage.py:420-428 on
 * different ranks): grouped, their tiles fill the GPU together.  A problem computes the same bits
 * alone or in a group. */
#define PP_GEMM_MAX_GROUP 28
int pp_gemm_bf16_grouped(const pp_gemm_desc* descs, int n, pp_stream stream);

/* The weight gradients of several microbatches in one launch.  Problem i is
 *   C_i = (beta ? C_i : 0) + g_0 + g_1 + ... + g_{n_seg-1},   g_s = A_{i,s}^T B_{i,s}
 * with the terms added one at a time in ascending s in fp32 (g_s rounded to bf16 first under
 * PP_EPI_ACCUM_ROUNDED): bit for bit what n_seg accumulating pp_gemm_bf16_grouped launches, one per
 * microbatch in ascending order, leave in C (the reference reaches them through one autograd pass per
 * microbatch, pippy/_backward.py:67-69, accumulating in backward-microbatch order,
 * pippy/PipelineSchedule.py:327,401-438).  A tile keeps its running sum in registers, so C moves once
 * instead of n_seg times.  Every descriptor: a_trans = b_trans = 1, fp32 C, PP_EPI_ACCUM_F32 or _ROUNDED;
 * desc->A and desc->B are DEVICE arrays of n_seg device pointers to the [K, M] and [K, N] operands of the
 * segments (each 16-byte aligned, which the caller vouches for; K, lda, ldb are shared by the segments). */
#define PP_GEMM_MAX_KSEG 1024
int pp_gemm_bf16_grouped_kseg(const pp_gemm_desc* descs, int n, int n_seg, pp_stream stream);

/* One GEMM per segment of a row-partitioned operand, with the segment bounds in DEVICE memory:
 * seg_start[0 .. n_seg] ascending row indices (int32), read by the kernel, so that sizes produced on
 * the device (the token counts of the experts of a mixture-of-experts layer, which the reference
 * would reach as one F.linear per expert inside the stage module, pippy/_PipelineStage.py:420-428)
 * never travel to the host.  seg_ptr[0 .. n_seg) is a device array of device pointers.
 *   PP_SEG_ROWS: for every segment e,  C[r0:r1, :] = epilogue(A[r0:r1, :] * B_e^T)  with
 *     B_e = seg_ptr[e] ([N, K], ldb), r0 = seg_start[e], r1 = seg_start[e + 1]; desc->M is the total
 *     row count (an upper bound for the grid), desc->B is ignored; a_trans = b_trans = 0, bf16 C,
 *     epilogue NONE or BIAS_RESIDUAL with a null bias (C = A B^T + aux_in, rows as in C).
 *   PP_SEG_K: for every segment e,  C_e = A[r0:r1, :]^T * B[r0:r1, :]  with C_e = seg_ptr[e]
 *     ([M, N], ldc): the weight gradient of expert e; desc->K is the total row count, desc->C is
 *     ignored; a_trans = b_trans = 1; bf16 C with NONE (an empty segment writes zeros) or fp32 C
 *     with ACCUM_F32 or ACCUM_ROUNDED / beta. */
enum pp_gemm_seg_mode { PP_SEG_ROWS = 0, PP_SEG_K = 1 };
#define PP_GEMM_MAX_SEGMENTS 1024
int pp_gemm_bf16_segmented(const pp_gemm_desc* desc, const int32_t* seg_start, const void* const* seg_ptr,
                           int n_seg, int mode, pp_stream stream);

/* PP_SEG_K over several microbatches in one launch (the expert weight gradients of a mixture-of-experts
 * layer for all microbatches of a step):  for every segment e,
 *   C_e = (beta ? C_e : 0) + g_{e,0} + ... + g_{e,n_mb-1},   g_{e,m} = A_m[r0:r1, :]^T * B_m[r0:r1, :],
 *   r0 = seg_start_of[m][e], r1 = seg_start_of[m][e + 1]
 * added one term at a time in ascending m in fp32 (g rounded to bf16 first under PP_EPI_ACCUM_ROUNDED): bit
 * for bit what one accumulating PP_SEG_K launch per microbatch, in ascending order, leaves in C_e.  a_of,
 * b_of, seg_start_of ([n_mb]) and seg_ptr ([n_seg]) are DEVICE arrays of device pointers; desc gives M, N,
 * lda, ldb, ldc, epilogue (ACCUM_F32 / ACCUM_ROUNDED) and beta, its A, B, C and K are ignored.  The
 * accumulators C_e, which outweigh a microbatch's operands, move once instead of n_mb times. */
int pp_gemm_bf16_segmented_kseg(const pp_gemm_desc* desc, const void* const* a_of, const void* const* b_of,
                                const int32_t* const* seg_start_of, const void* const* seg_ptr, int n_seg,
                                int n_mb, pp_stream stream);

/* fp32 GEMM with the same descriptor (A, B, C, bias, aux fp32; config 1 of the baseline, the
 * README MLP).  Only a_trans / b_trans, NONE, BIAS, BIAS_RELU, DRELU and ACCUM_F32 epilogues. */
int pp_gemm_f32(const pp_gemm_desc* desc, pp_stream stream);

/* db[n] = sum_m dY[m, n]  (bias gradient of a linear; part of the dW pass).
 * out is bf16 [N] (out_dtype PP_BF16) or fp32 [N]; workspace: fp32 [ws_rows = ceil(M/128), N]. */
int pp_colsum_bf16(const void* dY, int64_t M, int64_t N, int64_t ld, void* out, int out_dtype,
                   float* workspace, pp_stream stream);

/* pp_colsum_bf16 without a workspace argument.  No counterpart in the reference: it exists for
 * callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  The partial sums go to an array that the library itself holds
 * on every GPU it runs on (PP_COLSUM_NOALLOC_MAX_FLOATS floats = 4 MiB per GPU, held until the
 * process ends); the call allocates and frees nothing.  Problems with ceil(M / 128) * N above that
 * limit are rejected with PP_ERR_UNSUPPORTED.  All calls on one GPU share that GPU's array: calls
 * that may overlap on one GPU (different streams, different threads) race and must be serialised
 * by the caller.  Results are bit-identical to pp_colsum_bf16. */
#define PP_COLSUM_NOALLOC_MAX_FLOATS (1 << 20)
int pp_colsum_bf16_noalloc(const void* dY, int64_t M, int64_t N, int64_t ld, void* out, int out_dtype,
                           pp_stream stream);

/* dst[c, r] = src[r, c] for bf16 (any 2-byte type).  Used once per optimizer step to keep a
 * transposed copy of every linear weight, so that the input-gradient GEMM dX = dY W
 * (pippy/_backward.py:67-69) reads both operands k-contiguously. */
int pp_transpose_bf16(const void* src, int64_t rows, int64_t cols, int64_t ld_src, void* dst,
                      int64_t ld_dst, pp_stream stream);

/* dz[i] = dy[i] * act'(aux[i]) for act 0 = relu (aux: the activation's output or input),
 * 1 = gelu (erf form, aux: pre-activation), 2 = gelu (tanh form); dtype PP_BF16 or PP_F32.
 * Backward of an activation that stands between two separately lowered linears
 * (torch.relu in examples/basic/example_train.py:19-22, differentiated by pippy/_backward.py:67-69). */
int pp_activation_bwd(const void* dy, const void* aux, void* dz, int64_t n, int act, int dtype,
                      pp_stream stream);

/* ------------------------------------------------------------------------------------------
 * Element-wise pieces of a Llama-style layer (inside the stage module in the reference; backward
 * through pippy/_backward.py:67-69).  bf16, n % 8 == 0, 16-byte aligned pointers.
 *   SwiGLU:  h = silu(g) * u;   dg = dh * u * silu'(g),  du = dh * silu(g)
 *   RoPE (rotate-half form, in place): for the first n_heads heads of width D of every row of
 *   x [n_tok, ld]:  (x[i], x[i + D/2]) -> (x[i] c - x[i + D/2] s,  x[i + D/2] c + x[i] s)  with
 *   c, s = cos_table / sin_table [seq, D/2] (fp32) at position t % seq;  inverse != 0 applies the
 *   transposed rotation (the backward pass).  A fused [q | k | v] projection is rotated with
 *   n_heads = q heads + k heads.
 * ---------------------------------------------------------------------------------------- */
int pp_swiglu_fwd(const void* g, const void* u, void* h, int64_t n, pp_stream stream);
int pp_swiglu_bwd(const void* g, const void* u, const void* dh, void* dg, void* du, int64_t n,
                  pp_stream stream);
int pp_rope(void* x, const float* cos_table, const float* sin_table, int64_t n_tok, int64_t seq,
            int64_t n_heads, int64_t D, int64_t ld, int inverse, pp_stream stream);

/* SwiGLU fused into the GEMMs on either side of it (the feed-forward of a Llama-style layer inside
 * the stage module: forward through pippy/_PipelineStage.py:420-428, backward through
 * pippy/_backward.py:67-69).  All operands bf16, k-contiguous; x, the weights 16-byte aligned with
 * K, ldx, ldw multiples of 8; N a multiple of 8; gu, h, dgu 8-byte aligned with leading dimensions
 * that are multiples of 4.
 *   pp_gemm_bf16_swiglu:  g = x w_gate^T, u = x w_up^T (x [M, K], w_gate and w_up [N, K] with the same
 *     ldw), both rounded to bf16 and stored side by side in gu [M, 2 N] (g in columns [0, N), u in
 *     [N, 2 N)), and h [M, N] = silu(g) * u from the rounded values: the bits of two pp_gemm_bf16 calls
 *     followed by pp_swiglu_fwd.
 *   pp_gemm_bf16_dswiglu: dh = dy w_down_t^T (dy [M, K], w_down_t [N, K] the transposed down
 *     projection) is rounded to bf16 and never stored; dgu [M, 2 N] receives dg = dh u silu'(g) in
 *     columns [0, N) and du = dh silu(g) in [N, 2 N), g and u read from gu: the bits of pp_gemm_bf16
 *     followed by pp_swiglu_bwd. */
int pp_gemm_bf16_swiglu(const void* x, const void* w_gate, const void* w_up, void* gu, void* h, int64_t M,
                        int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ld_gu, int64_t ldh,
                        pp_stream stream);
int pp_gemm_bf16_dswiglu(const void* dy, const void* w_down_t, const void* gu, void* dgu, int64_t M,
                         int64_t N, int64_t K, int64_t ldy, int64_t ldw, int64_t ld_gu, int64_t ld_dgu,
                         pp_stream stream);
/* The same two calls over rows that are partitioned into n_seg consecutive segments with weights of their
 * own (the experts of a mixture-of-experts feed-forward over its permuted token rows, replacing the per-expert
 * F.linear calls reached from pippy/_PipelineStage.py:420-428 and their backward, pippy/_backward.py:67-69):
 * rows [seg_start[e], seg_start[e+1]) use w_gate_of[e] / w_up_of[e] (forward) or w_down_t_of[e] (backward).
 * seg_start [n_seg + 1] (int32) and the pointer arrays live in DEVICE memory; M is the total number of
 * rows (seg_start[n_seg] <= M), every weight [N, K] with the same ldw.  Rows outside every segment are not
 * written.  Bits as pp_gemm_bf16_segmented (rows mode) followed by pp_swiglu_fwd / pp_swiglu_bwd. */
int pp_gemm_bf16_segmented_swiglu(const void* x, const void* const* w_gate_of, const void* const* w_up_of,
                                  const int32_t* seg_start, int n_seg, void* gu, void* h, int64_t M, int64_t N,
                                  int64_t K, int64_t ldx, int64_t ldw, int64_t ld_gu, int64_t ldh,
                                  pp_stream stream);
int pp_gemm_bf16_segmented_dswiglu(const void* dy, const void* const* w_down_t_of, const int32_t* seg_start,
                                   int n_seg, const void* gu, void* dgu, int64_t M, int64_t N, int64_t K,
                                   int64_t ldy, int64_t ldw, int64_t ld_gu, int64_t ld_dgu, pp_stream stream);

/* ------------------------------------------------------------------------------------------
 * Routing of a top-2 mixture-of-experts layer (a Mixtral-style block inside the stage module;
 * forward through pippy/_PipelineStage.py:420-428, backward through pippy/_backward.py:67-69).
 * T tokens, E experts, topk slots per token; flat slot f = t * topk + k; permuted rows are grouped
 * by expert and ordered by ascending f inside an expert.  All index arrays are int32 in device
 * memory; nothing is read back by the host.
 *   pp_moe_router_top2: logits bf16 [T, ld] -> topk_idx [T, 2] (the two largest logits, the lower
 *     expert index winning a tie) and gate fp32 [T, 2] = softmax over all experts renormalised
 *     over the selected pair.
 *   pp_moe_permute: expert_of_slot [n_slots] -> seg_start [E + 1] (first row of every expert;
 *     seg_start[E] = rows placed), row_src [n_slots] (flat slot of every row), pos [n_slots] (row
 *     of every flat slot; -1 and dropped for an expert id outside [0, E)).  E <= 64.
 *   (pp_moe_gate_bwd writes the columns [E, round_up(E, 8)) of dlogits as zeros: a router whose expert
 *   count is not a multiple of 8 runs its GEMMs on logits padded to one.)
 *   pp_moe_gather: dst[r, :] = scale[f] * src[f / topk, :] with f = row_src[r] for r < *n_rows_dev
 *     (null: r < R); scale null = plain gather.  Tokens -> expert rows, and the weighted
 *     scatter of the output gradient in the backward pass.
 *   pp_moe_combine: out[t, :] = resid[t, :] + sum_k gate[f] * y[pos[f], :] (resid, gate optional),
 *     fp32 sum with one rounding.  Expert rows -> tokens, and the sum of the expert input
 *     gradients in the backward pass.
 *   pp_moe_gate_bwd: dlogits bf16 [T, ld_dl]: gradient of the loss w.r.t. the router logits given
 *     dout [T, C] and the expert outputs y [rows, C]; zero for experts that were not selected.
 * bf16 rows: 16-byte aligned, leading dimensions and C multiples of 8.
 * ---------------------------------------------------------------------------------------- */
int pp_moe_router_top2(const void* logits, int64_t ld, int64_t T, int E, int32_t* topk_idx, float* gate,
                       pp_stream stream);
int pp_moe_permute(const int32_t* expert_of_slot, int64_t n_slots, int E, int32_t* seg_start,
                   int32_t* row_src, int32_t* pos, pp_stream stream);
int pp_moe_gather(const void* src, int64_t ld_src, const int32_t* row_src, const int32_t* n_rows_dev,
                  int topk, const float* scale, void* dst, int64_t ld_dst, int64_t R, int64_t C,
                  pp_stream stream);
int pp_moe_combine(const void* y, int64_t ld_y, const int32_t* pos, const float* gate, int topk,
                   const void* resid, int64_t ld_resid, void* out, int64_t ld_out, int64_t T, int64_t C,
                   pp_stream stream);
int pp_moe_gate_bwd(const void* dout, int64_t ld_dout, const void* y, int64_t ld_y, const int32_t* pos,
                    const int32_t* topk_idx, const float* gate, int topk, int E, void* dlogits,
                    int64_t ld_dl, int64_t T, int64_t C, pp_stream stream);

/* Column reductions of one weight-gradient pass in two launches.  Per descriptor:
 *   out_sum[c] = sum_r dy[r, c]                                   (bias gradient / dbeta), and, if
 *   out_dot is non-null, out_dot[c] = sum_r dy[r, c] * (x[r, c] - mean[r]) * rstd[r]   (dgamma).
 * workspace: fp32 [2, ceil(rows / 128), C] per descriptor, distinct between descriptors.  Sums are
 * formed in a fixed order, so results do not depend on scheduling.
 * n_part_ready = P > 0: the kernel that produced dy has already left P rows of partial sums in the
 * workspace (fp32 [2, P, C]: sums, then dots; pp_layernorm_bwd_input_sums writes that form), so dy
 * and x are not read again (they may be null) and only the final sums are formed. */
typedef struct pp_colreduce_desc {
    const void* dy;      /* bf16 [rows, C] with row stride ld_dy */
    const void* x;       /* bf16 [rows, C] contiguous, or null */
    const float* mean;   /* fp32 [rows] (with x) */
    const float* rstd;   /* fp32 [rows] (with x) */
    void* out_sum;       /* [C] or null */
    void* out_dot;       /* [C] or null */
    float* workspace;
    int64_t ld_dy, rows, C;
    int32_t out_dtype;   /* PP_BF16 or PP_F32 */
    int32_t n_part_ready; /* 0: reduce dy; P > 0: the workspace holds P rows of partial sums */
} pp_colreduce_desc;
#define PP_COLREDUCE_MAX_GROUP 24
int pp_colreduce_grouped(const pp_colreduce_desc* descs, int n, pp_stream stream);

/* ------------------------------------------------------------------------------------------
 * LayerNorm (F.layer_norm inside the stage module; backward via pippy/_backward.py:67-69).
 * x, y, dy, dx: bf16 [rows, C]; gamma, beta: bf16 [C]; mean, rstd: fp32 [rows].
 * A null `mean` selects RMSNorm in all three calls: nothing is subtracted, rstd = 1 / sqrt(mean(x^2)
 * + eps), there is no beta and no dbeta.
 * ---------------------------------------------------------------------------------------- */
int pp_layernorm_fwd(const void* x, const void* gamma, const void* beta, void* y, float* mean,
                     float* rstd, int64_t rows, int64_t C, float eps, pp_stream stream);
/* dx = LN'(dy) (+ dres if non-null): the input-gradient pass */
int pp_layernorm_bwd_input(const void* dy, const void* x, const void* gamma, const float* mean,
                           const float* rstd, const void* dres, void* dx, int64_t rows, int64_t C,
                           pp_stream stream);
/* pp_layernorm_bwd_input that also leaves column sums for the weight-gradient pass, so that dy, x and
 * dx are not read a second time: per block of PP_LN_SUM_ROWS rows one row of partial sums,
 *   ws_weight fp32 [2, P, C]: sum of dy (dbeta), then sum of dy * xhat (dgamma),
 *   ws_dx     fp32 [P, C]:    sum of dx as written (rounded to bf16): the bias gradient of the linear
 *                             layer whose output gradient dx is,
 * with P = ceil(rows / PP_LN_SUM_ROWS); either may be null.  pp_colreduce_grouped with n_part_ready = P
 * forms the final sums.  C <= PP_LN_SUM_MAX_C.  Same reference arithmetic as the two separate passes
 * (F.layer_norm's backward reached from pippy/_backward.py:67-69), in a fixed summation order. */
#define PP_LN_SUM_ROWS 16
#define PP_LN_SUM_MAX_C 1024
int pp_layernorm_bwd_input_sums(const void* dy, const void* x, const void* gamma, const float* mean,
                                const float* rstd, const void* dres, void* dx, int64_t rows, int64_t C,
                                float* ws_weight, float* ws_dx, pp_stream stream);
/* dgamma, dbeta (bf16 [C] or fp32 by out_dtype): the weight-gradient pass.
 * workspace: fp32 [2, ceil(rows/128), C]. */
int pp_layernorm_bwd_weight(const void* dy, const void* x, const float* mean, const float* rstd,
                            void* dgamma, void* dbeta, int out_dtype, float* workspace,
                            int64_t rows, int64_t C, pp_stream stream);

/* ------------------------------------------------------------------------------------------
 * Multi-head attention, flash style (F.scaled_dot_product_attention inside the stage module).
 * q, k, v: bf16, element (b, s, h, d) at base + b*stride_b + s*stride_s + h*head_dim + d, so the
 * three can alias one fused [B, S, 3*H*D] projection output.  o: bf16 [B, S, H*D] contiguous.
 * lse: fp32 [B, H, S] (log-sum-exp of the scaled scores; saved for backward).
 * head_dim in {64, 128}; S % 64 == 0.  A shorter sequence is handed over padded to such an S with zero
 * rows: kv_len = L makes the forward leave keys L .. S-1 out of the softmax (a causal mask does that
 * for the real queries by itself).  The backward needs no mask: with zero key and value rows in the
 * padding and zero d_o rows for the padded queries, the real rows of dq, dk, dv are exact.
 * Grouped-query attention: kv_group = G > 1 query heads share one key / value head, k and v (and dk,
 * dv) then hold H / G heads, query head h reads key / value head h / G, and dk, dv are sums over the
 * group (formed inside one work-group, in ascending query-head order); 0 or 1: one per query head.
 * ---------------------------------------------------------------------------------------- */
typedef struct pp_attn_desc {
    const void* q; const void* k; const void* v;
    void* o; float* lse;
    const void* d_o;       /* backward only: bf16 [B, S, H*D] */
    void* dq; void* dk; void* dv; /* backward only: same addressing as q, k, v */
    float* delta;          /* backward workspace: fp32 [B, H, S] */
    int64_t B, S, H, D;
    int64_t stride_b, stride_s; /* of q/k/v (and dq/dk/dv), in elements */
    float scale;           /* usually 1/sqrt(D) */
    int32_t causal;
    int32_t kv_group;      /* query heads per key / value head; 0 or 1: multi-head attention */
    int32_t kv_len;        /* 0: every key exists; L in 1..S: keys L..S-1 of each sequence are padding */
    int32_t flags;         /* PP_ATTN_* bits */
    float* colsum;         /* backward, head_dim 64, or null: fp32 [B * S / 64, ld_colsum]; row b * (S / 64) + j
                              receives the sums over the 64 tokens of block j of every column of dq, dk and dv
                              as stored, at the column that the element has relative to dq (dq, dk, dv are then
                              sections of one row of a fused projection's gradient, dq first): the partial sums
                              of that projection's bias gradient, for pp_colreduce_grouped with
                              n_part_ready = B * S / 64 */
    int64_t ld_colsum;     /* row length of colsum, in floats */
} pp_attn_desc;
/* Backward: correct dq for the rounding of the forward's output.  The backward starts from
 * delta = rowsum(dO * O) of the bf16 output; the sum of P * dP over the keys is the same number in exact
 * arithmetic and the one under which the rows of dS sum to zero.  The dQ kernel always forms it (it is
 * what `delta` holds afterwards and what the dK / dV kernel uses); with this bit it also corrects its own
 * result, dQ -= (that sum - delta) * (P K), for one more MFMA per key block and tile.  For models whose
 * attention is nearly uniform while their keys share a large common part (an encoder at initialisation),
 * where the query gradients are small differences of large terms. */
#define PP_ATTN_EXACT_DQ 1
int pp_attn_fwd(const pp_attn_desc* desc, pp_stream stream);
int pp_attn_bwd(const pp_attn_desc* desc, pp_stream stream);

/* ------------------------------------------------------------------------------------------
 * Token + position embedding (F.embedding inside the first stage).
 * y[t, :] = wte[ids[t], :] + (wpe ? wpe[t % seq, :] : 0) + (extra_row ? extra_row[:] : 0), summed in
 * fp32 and rounded once;  ids int64 [n_tok]; bf16 tables; extra_row is one bf16 row [C] added to
 * every token (the token-type-0 row of a BERT embedding) or null.
 * ---------------------------------------------------------------------------------------- */
int pp_embed_fwd(const int64_t* ids, const void* wte, const void* wpe, const void* extra_row, void* y,
                 int64_t n_tok, int64_t seq, int64_t C, int64_t vocab, pp_stream stream);
/* The same sum with the position row given per token: wpe[pos_ids[t], :] (pos_ids int64 [n_tok], rows of
 * an [n_pos, C] table; an index out of range reads row 0).  For encoders that count positions over the
 * tokens that are not padding (the embeddings of the model in examples/huggingface/pippy_camemBert.py). */
int pp_embed_fwd_at(const int64_t* ids, const int64_t* pos_ids, const void* wte, const void* wpe,
                    const void* extra_row, void* y, int64_t n_tok, int64_t n_pos, int64_t C, int64_t vocab,
                    pp_stream stream);
/* Those positions: out[b, s] = pad where ids[b, s] == pad, else pad + the number of tokens != pad among
 * ids[b, 0..s]  (ids, out int64 [n_seq, seq]; the position indices that the embeddings of the model in
 * examples/huggingface/pippy_camemBert.py compute with ne / cumsum / mul / add). */
int pp_position_ids_from_padding(const int64_t* ids, int64_t* out, int64_t n_seq, int64_t seq, int64_t pad,
                                 pp_stream stream);
/* Gradient of the lookup, added to fp32 accumulators (F.embedding's backward reached through
 * pippy/_backward.py:67-69, followed by the accumulation into the parameter's gradient):
 *   d_wte[v, :] += g[v, :],  g[v, :] = sum of dy[t, :] over the tokens t with ids[t] == v, formed in
 *   fp32 in ascending t;  d_wpe[p, :] += sum over the batch of dy[b * seq + p, :] in ascending b.
 * round_bf16 != 0 rounds g to bf16 before it is added: bit for bit what a bf16 gradient tensor folded
 * in by pp_grad_accum_f32_bf16 leaves.  No atomics: results do not depend on scheduling.  C <= 8192.
 * padding_idx >= 0: row padding_idx of d_wte is left untouched (nn.Embedding(padding_idx=...) gives that row
 * no gradient) and its tokens are not summed; negative: no such row. */
int pp_embed_bwd(const int64_t* ids, const void* dy, float* d_wte, float* d_wpe, int64_t n_tok,
                 int64_t seq, int64_t C, int64_t vocab, int round_bf16, int64_t padding_idx, pp_stream stream);

/* ------------------------------------------------------------------------------------------
 * Cross-entropy loss of one microbatch (loss_fn at pippy/PipelineSchedule.py:154-155 when it is
 * torch cross_entropy with mean reduction) fused with its gradient.
 * logits bf16 [rows, ld] (first V columns valid); target int64 [rows] (ignore_index skipped; so is a
 * target outside [0, V), which torch rejects: callers that cannot trust their targets check them on the
 * host); loss: fp32 [1], NaN when every row is skipped (the mean over no rows, as torch returns it; the
 * gradient is zero then); dlogits bf16 [rows, ld] (columns >= V written as 0) or null (loss only);
 * workspace: fp32 [rows + 2].
 * ---------------------------------------------------------------------------------------- */
int pp_ce_loss(const void* logits, const int64_t* target, float* loss, void* dlogits,
               float* workspace, int64_t rows, int64_t V, int64_t ld, int64_t ignore_index,
               int logits_dtype, pp_stream stream);

/* ------------------------------------------------------------------------------------------
 * Launch list: a host array of tagged descriptors executed in order on one stream.  One call
 * replays a whole stage forward / input-gradient / weight-gradient pass for one microbatch
 * (pippy/_PipelineStage.py:452-550) without returning to Python between kernels.
 * ---------------------------------------------------------------------------------------- */
enum pp_op_kind {
    PP_OP_GEMM_BF16 = 1, PP_OP_GEMM_F32 = 2, PP_OP_COLSUM = 3, PP_OP_LN_FWD = 4,
    PP_OP_LN_BWD_INPUT = 5, PP_OP_LN_BWD_WEIGHT = 6, PP_OP_ATTN_FWD = 7, PP_OP_ATTN_BWD = 8,
    PP_OP_EMBED_FWD = 9, PP_OP_EMBED_BWD = 10, PP_OP_CE_LOSS = 11, PP_OP_ACCUM_BF16 = 12,
    PP_OP_ACCUM_F32 = 13, PP_OP_COPY_ROWS = 14, PP_OP_FILL = 15, PP_OP_ACT_BWD = 16,
    PP_OP_SWIGLU_FWD = 17, PP_OP_SWIGLU_BWD = 18, PP_OP_ROPE = 19, PP_OP_GEMM_SEG = 20,
    PP_OP_MOE_ROUTER = 21, PP_OP_MOE_PERMUTE = 22, PP_OP_MOE_GATHER = 23, PP_OP_MOE_COMBINE = 24,
    PP_OP_MOE_GATE_BWD = 25, PP_OP_GEMM_SWIGLU = 26, PP_OP_GEMM_DSWIGLU = 27, PP_OP_POSITION_IDS = 28,
    PP_OP_GEMM_KSEG = 29, PP_OP_GEMM_SEG_KSEG = 30, PP_OP_GEMM_SEG_SWIGLU = 31, PP_OP_GEMM_SEG_DSWIGLU = 32
};

/* Field use per kind (unused fields are ignored):
 *   GEMM_*        p: A B C bias aux_in aux_out | i: M N K lda ldb ldc ld_aux | j: a_trans b_trans
 *                 epilogue c_dtype beta; GEMM_BF16 also p[8]: split-K workspace or null, i[10]: its
 *                 size in floats (then the op is pp_gemm_bf16_splitk), p[9]: colsum or null
 *   COLSUM        p: dY out workspace | i: M N ld | j: out_dtype n_part_ready
 *   LN_FWD        p: x gamma beta y mean rstd | i: rows C | f: eps
 *   LN_BWD_INPUT  p: dy x gamma mean rstd dres dx ws_weight ws_dx | i: rows C  (a non-null ws_weight or
 *                 ws_dx: pp_layernorm_bwd_input_sums)
 *   LN_BWD_WEIGHT p: dy x mean rstd dgamma dbeta workspace | i: rows C | j: out_dtype n_part_ready
 *                 (n_part_ready > 0, here and for COLSUM: the op runs through pp_colreduce_grouped)
 *   ATTN_*        p: q k v o lse d_o dq dk dv delta colsum | i: B S H D stride_b stride_s ld_colsum | f: scale
 *                 | j: causal kv_group kv_len flags
 *   EMBED_FWD     p: ids wte wpe y extra_row pos_ids | i: n_tok seq C vocab n_pos  (pos_ids non-null:
 *                 pp_embed_fwd_at)
 *   POSITION_IDS  p: ids out | i: n_seq seq pad
 *   EMBED_BWD     p: ids dy d_wte d_wpe | i: n_tok seq C vocab padding_idx+1 (0: none) | j: round_bf16
 *   CE_LOSS       p: logits target loss dlogits workspace | i: rows V ld ignore_index | j: dtype
 *   ACCUM_*       p: acc g | i: n | j: init
 *   COPY_ROWS     p: src dst | i: n_rows row_bytes src_stride dst_stride
 *   FILL          p: dst | i: n_bytes | j: value
 *   ACT_BWD       p: dy aux dz | i: n | j: act dtype
 *   SWIGLU_FWD    p: g u h | i: n
 *   SWIGLU_BWD    p: g u dh dg du | i: n
 *   ROPE          p: x cos sin | i: n_tok seq n_heads D ld | j: inverse
 *   GEMM_SEG      as GEMM_BF16, and p[6]: seg_start p[7]: seg_ptr | i[7]: n_seg | j[5]: mode
 *   MOE_ROUTER    p: logits topk_idx gate | i: ld T E
 *   MOE_PERMUTE   p: expert_of_slot seg_start row_src pos | i: n_slots E
 *   MOE_GATHER    p: src row_src n_rows_dev scale dst | i: ld_src topk ld_dst R C
 *   MOE_COMBINE   p: y pos gate resid out | i: ld_y topk ld_resid ld_out T C
 *   MOE_GATE_BWD  p: dout y pos topk_idx gate dlogits | i: ld_dout ld_y topk E ld_dl T C
 *   GEMM_SWIGLU   p: x w_gate w_up gu h | i: M N K ldx ldw ld_gu ldh
 *   GEMM_DSWIGLU  p: dy w_down_t gu dgu | i: M N K ldy ldw ld_gu ld_dgu
 *   GEMM_KSEG     as GEMM_BF16 with p[0], p[1]: device arrays of the segments' A and B pointers
 *                 | i[7]: n_seg; consecutive GEMM_KSEG ops with the same n_seg go out as ONE
 *                 pp_gemm_bf16_grouped_kseg call (they must not depend on each other)
 *   GEMM_SEG_KSEG as GEMM_SEG in k mode with p[0], p[1]: device arrays of the microbatches' A and B, p[6]:
 *                 device array of their seg_start arrays | i[7]: n_seg, i[8]: n_mb
 *   GEMM_SEG_SWIGLU  p: x w_gate_of w_up_of gu h seg_start | i: M N K ldx ldw ld_gu ldh n_seg
 *   GEMM_SEG_DSWIGLU p: dy w_down_t_of gu dgu seg_start | i: M N K ldy ldw ld_gu ld_dgu n_seg
 * flags bit 0 (PP_OP_SKIP): the op is stepped over.
 * flags bit 1 (PP_OP_GROUPED): a GEMM_BF16 op that may be launched together with the grouped
 * GEMM_BF16 ops next to it (they must not depend on each other); likewise consecutive grouped
 * COLSUM / LN_BWD_WEIGHT ops run as one pp_colreduce_grouped call (distinct workspaces needed). */
#define PP_OP_SKIP 1
#define PP_OP_GROUPED 2

typedef struct pp_op {
    int32_t kind;   /* enum pp_op_kind */
    int32_t flags;
    void* p[12];
    int64_t i[12];
    float f[2];
    int32_t j[6];
} pp_op;

/* Runs ops[0..n) in order; stops at the first failure and returns its code (the index of the
 * failing op is in pp_last_error()). */
int pp_run_ops(const pp_op* ops, int n_ops, pp_stream stream);

/* ------------------------------------------------------------------------------------------
 * Per-launch timing of launch-list ops (measurement aid; no reference counterpart).  Between
 * pp_profile_start and pp_profile_stop every op run by pp_run_ops is bracketed by two HIP events on
 * its stream (host-side event objects only; no device memory).  pp_profile_read waits for the
 * recorded events and returns, for one op kind, the summed elapsed milliseconds, the summed
 * algorithmic work (FLOPs for GEMM and attention kinds, bytes for the HBM-bound kinds) and the
 * number of launches.  Not thread-safe.
 * ---------------------------------------------------------------------------------------- */
int pp_profile_start(int max_records);
int pp_profile_stop(void);
int pp_profile_read(int kind, double* total_ms, double* total_work, int64_t* count);

#ifdef __cplusplus
}
#endif
#endif /* PIPPY_AMD_H */
