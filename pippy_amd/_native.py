"""ctypes binding of ``libpippy_amd.so`` (the C ABI declared in ``include/pippy_amd.h``).

There is no CPU fallback: if the library is missing, every kernel call raises.  Tensors are passed
as raw device pointers and launches go to torch's current HIP stream, so they order with torch
work on that stream.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import torch

from ._build import LIB_PATH

PP_OK = 0
PP_ERR_INVALID, PP_ERR_UNSUPPORTED, PP_ERR_LAUNCH = 1, 2, 3
PP_COLSUM_NOALLOC_MAX_FLOATS = 1 << 20
PP_BF16, PP_F32 = 0, 1

# enum pp_gemm_epilogue
EPI_NONE, EPI_BIAS, EPI_BIAS_GELU_ERF, EPI_BIAS_GELU_TANH, EPI_BIAS_RESIDUAL = 0, 1, 2, 3, 4
EPI_DGELU_ERF, EPI_DGELU_TANH, EPI_ACCUM_F32, EPI_BIAS_RELU, EPI_DRELU, EPI_ACCUM_ROUNDED = 5, 6, 7, 8, 9, 10

# enum pp_op_kind
(OP_GEMM_BF16, OP_GEMM_F32, OP_COLSUM, OP_LN_FWD, OP_LN_BWD_INPUT, OP_LN_BWD_WEIGHT, OP_ATTN_FWD,
 OP_ATTN_BWD, OP_EMBED_FWD, OP_EMBED_BWD, OP_CE_LOSS, OP_ACCUM_BF16, OP_ACCUM_F32, OP_COPY_ROWS,
 OP_FILL, OP_ACT_BWD, OP_SWIGLU_FWD, OP_SWIGLU_BWD, OP_ROPE, OP_GEMM_SEG, OP_MOE_ROUTER, OP_MOE_PERMUTE,
 OP_MOE_GATHER, OP_MOE_COMBINE, OP_MOE_GATE_BWD, OP_GEMM_SWIGLU, OP_GEMM_DSWIGLU, OP_POSITION_IDS,
 OP_GEMM_KSEG, OP_GEMM_SEG_KSEG, OP_GEMM_SEG_SWIGLU, OP_GEMM_SEG_DSWIGLU) = range(1, 33)
SEG_ROWS, SEG_K = 0, 1
OP_SKIP = 1
OP_GROUPED = 2
ATTN_EXACT_DQ = 1
ACT_RELU, ACT_GELU_ERF, ACT_GELU_TANH = 0, 1, 2

PP_COPY_MAX_SEGS = 64

# every symbol include/pippy_amd.h declares
EXPORTED_SYMBOLS = (
    "pp_abi_version", "pp_last_error", "pp_copy_rows", "pp_split_copy", "pp_merge_copy",
    "pp_strided_copy_nd", "pp_grad_accum_f32_bf16", "pp_grad_accum_f32_f32", "pp_fill_bytes",
    "pp_gemm_bf16", "pp_gemm_bf16_splitk", "pp_gemm_bf16_grouped", "pp_gemm_bf16_grouped_kseg", "pp_gemm_bf16_segmented_kseg", "pp_gemm_f32", "pp_colsum_bf16", "pp_colreduce_grouped", "pp_layernorm_fwd", "pp_layernorm_bwd_input", "pp_layernorm_bwd_input_sums",
    "pp_layernorm_bwd_weight", "pp_attn_fwd", "pp_attn_bwd", "pp_embed_fwd", "pp_embed_bwd",
    "pp_ce_loss", "pp_run_ops", "pp_activation_bwd", "pp_transpose_bf16", "pp_profile_start", "pp_profile_stop",
    "pp_profile_read", "pp_sgd_step", "pp_adamw_step", "pp_swiglu_fwd", "pp_swiglu_bwd", "pp_rope",
    "pp_gemm_bf16_segmented", "pp_moe_router_top2", "pp_moe_permute", "pp_moe_gather", "pp_moe_combine",
    "pp_moe_gate_bwd", "pp_colsum_bf16_noalloc", "pp_gemm_bf16_swiglu", "pp_gemm_bf16_dswiglu",
    "pp_embed_fwd_at", "pp_position_ids_from_padding", "pp_gemm_bf16_segmented_swiglu",
    "pp_gemm_bf16_segmented_dswiglu",
)


class CopySeg(C.Structure):
    _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("n_rows", C.c_int64),
                ("row_bytes", C.c_int64), ("src_stride", C.c_int64), ("dst_stride", C.c_int64)]


class GemmDesc(C.Structure):
    _fields_ = [("A", C.c_void_p), ("B", C.c_void_p), ("C", C.c_void_p),
                ("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64),
                ("lda", C.c_int64), ("ldb", C.c_int64), ("ldc", C.c_int64),
                ("a_trans", C.c_int32), ("b_trans", C.c_int32),
                ("epilogue", C.c_int32), ("c_dtype", C.c_int32),
                ("bias", C.c_void_p), ("aux_in", C.c_void_p), ("aux_out", C.c_void_p),
                ("ld_aux", C.c_int64), ("beta", C.c_int32), ("reserved", C.c_int32), ("colsum", C.c_void_p)]


class ColReduceDesc(C.Structure):
    _fields_ = [("dy", C.c_void_p), ("x", C.c_void_p), ("mean", C.c_void_p), ("rstd", C.c_void_p),
                ("out_sum", C.c_void_p), ("out_dot", C.c_void_p), ("workspace", C.c_void_p),
                ("ld_dy", C.c_int64), ("rows", C.c_int64), ("C", C.c_int64),
                ("out_dtype", C.c_int32), ("n_part_ready", C.c_int32)]


class AttnDesc(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p),
                ("o", C.c_void_p), ("lse", C.c_void_p), ("d_o", C.c_void_p),
                ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p),
                ("delta", C.c_void_p),
                ("B", C.c_int64), ("S", C.c_int64), ("H", C.c_int64), ("D", C.c_int64),
                ("stride_b", C.c_int64), ("stride_s", C.c_int64),
                ("scale", C.c_float), ("causal", C.c_int32), ("kv_group", C.c_int32), ("kv_len", C.c_int32),
                ("flags", C.c_int32), ("colsum", C.c_void_p), ("ld_colsum", C.c_int64)]


class Op(C.Structure):
    _fields_ = [("kind", C.c_int32), ("flags", C.c_int32), ("p", C.c_void_p * 12),
                ("i", C.c_int64 * 12), ("f", C.c_float * 2), ("j", C.c_int32 * 6)]


_lib: Optional[C.CDLL] = None


class NativeLibraryError(RuntimeError):
    pass


def lib() -> C.CDLL:
    """Loads the kernel library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise NativeLibraryError(
            f"{LIB_PATH} is missing: build it with `python -m pippy_amd._build` "
            "(there is no CPU fallback for the pipeline-stage kernels)")
    L = C.CDLL(str(LIB_PATH))
    L.pp_last_error.restype = C.c_char_p
    L.pp_abi_version.restype = C.c_int
    vp, i64, i32, f32 = C.c_void_p, C.c_int64, C.c_int, C.c_float
    sigs = {
        "pp_copy_rows": [C.POINTER(CopySeg), i32, vp],
        "pp_split_copy": [vp, C.POINTER(vp), i32, i64, i64, i64, vp],
        "pp_merge_copy": [vp, C.POINTER(vp), C.POINTER(i64), i32, i64, i64, vp],
        "pp_strided_copy_nd": [vp, vp, i32, C.POINTER(i64), C.POINTER(i64), i32, vp],
        "pp_grad_accum_f32_bf16": [vp, vp, i64, i32, vp],
        "pp_grad_accum_f32_f32": [vp, vp, i64, i32, vp],
        "pp_fill_bytes": [vp, i32, i64, vp],
        "pp_gemm_bf16": [C.POINTER(GemmDesc), vp],
        "pp_gemm_f32": [C.POINTER(GemmDesc), vp],
        "pp_gemm_bf16_splitk": [C.POINTER(GemmDesc), vp, i64, vp],
        "pp_gemm_bf16_grouped": [C.POINTER(GemmDesc), i32, vp],
        "pp_gemm_bf16_grouped_kseg": [C.POINTER(GemmDesc), i32, i32, vp],
        "pp_gemm_bf16_segmented_kseg": [C.POINTER(GemmDesc), vp, vp, vp, vp, i32, i32, vp],
        "pp_colsum_bf16": [vp, i64, i64, i64, vp, i32, vp, vp],
        "pp_colsum_bf16_noalloc": [vp, i64, i64, i64, vp, i32, vp],
        "pp_colreduce_grouped": [C.POINTER(ColReduceDesc), i32, vp],
        "pp_layernorm_fwd": [vp, vp, vp, vp, vp, vp, i64, i64, f32, vp],
        "pp_layernorm_bwd_input": [vp, vp, vp, vp, vp, vp, vp, i64, i64, vp],
        "pp_layernorm_bwd_input_sums": [vp, vp, vp, vp, vp, vp, vp, i64, i64, vp, vp, vp],
        "pp_layernorm_bwd_weight": [vp, vp, vp, vp, vp, vp, i32, vp, i64, i64, vp],
        "pp_attn_fwd": [C.POINTER(AttnDesc), vp],
        "pp_attn_bwd": [C.POINTER(AttnDesc), vp],
        "pp_embed_fwd": [vp, vp, vp, vp, vp, i64, i64, i64, i64, vp],
        "pp_embed_bwd": [vp, vp, vp, vp, i64, i64, i64, i64, i32, i64, vp],
        "pp_embed_fwd_at": [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, vp],
        "pp_position_ids_from_padding": [vp, vp, i64, i64, i64, vp],
        "pp_ce_loss": [vp, vp, vp, vp, vp, i64, i64, i64, i64, i32, vp],
        "pp_run_ops": [C.POINTER(Op), i32, vp],
        "pp_activation_bwd": [vp, vp, vp, i64, i32, i32, vp],
        "pp_transpose_bf16": [vp, i64, i64, i64, vp, i64, vp],
        "pp_profile_start": [i32],
        "pp_profile_stop": [],
        "pp_profile_read": [i32, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(i64)],
        "pp_swiglu_fwd": [vp, vp, vp, i64, vp],
        "pp_swiglu_bwd": [vp, vp, vp, vp, vp, i64, vp],
        "pp_rope": [vp, vp, vp, i64, i64, i64, i64, i64, i32, vp],
        "pp_gemm_bf16_swiglu": [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, vp],
        "pp_gemm_bf16_dswiglu": [vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, vp],
        "pp_gemm_bf16_segmented_swiglu": [vp, vp, vp, vp, i32, vp, vp, i64, i64, i64, i64, i64, i64, i64, vp],
        "pp_gemm_bf16_segmented_dswiglu": [vp, vp, vp, i32, vp, vp, i64, i64, i64, i64, i64, i64, i64, vp],
        "pp_gemm_bf16_segmented": [C.POINTER(GemmDesc), vp, vp, i32, i32, vp],
        "pp_moe_router_top2": [vp, i64, i64, i32, vp, vp, vp],
        "pp_moe_permute": [vp, i64, i32, vp, vp, vp, vp],
        "pp_moe_gather": [vp, i64, vp, vp, i32, vp, vp, i64, i64, i64, vp],
        "pp_moe_combine": [vp, i64, vp, vp, i32, vp, i64, vp, i64, i64, i64, vp],
        "pp_moe_gate_bwd": [vp, i64, vp, i64, vp, vp, vp, i32, i32, vp, i64, i64, i64, vp],
        "pp_sgd_step": [vp, i32, vp, vp, vp, i64, f32, f32, f32, f32, i32, i32, i32, vp],
        "pp_adamw_step": [vp, i32, vp, vp, vp, vp, i64, f32, f32, f32, f32, f32, f32, f32, i32, vp],
    }
    for name, argtypes in sigs.items():
        fn = getattr(L, name)
        fn.argtypes = argtypes
        fn.restype = C.c_int
    _lib = L
    return L


def check(rc: int, what: str) -> None:
    if rc != PP_OK:
        msg = lib().pp_last_error()
        raise RuntimeError(f"{what} failed with code {rc}: {msg.decode() if msg else ''}")


def current_stream() -> int:
    """Raw handle of torch's current HIP stream (what ``torch.cuda.current_stream().cuda_stream``
    returns, without building the Python wrapper objects: this is called once per launch list)."""
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def require_cuda(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "pippy_amd kernels take device tensors; got a tensor on "
                f"{t.device} (there is no CPU path)")


# ---- microbatch copies ----------------------------------------------------------------------
def copy_rows(segs: Sequence[tuple]) -> None:
    """segs: (src_ptr, dst_ptr, n_rows, row_bytes, src_stride, dst_stride) tuples."""
    if not segs:
        return
    arr = (CopySeg * len(segs))()
    for a, s in zip(arr, segs):
        a.src, a.dst, a.n_rows, a.row_bytes, a.src_stride, a.dst_stride = s
    for i0 in range(0, len(segs), PP_COPY_MAX_SEGS):
        n = min(PP_COPY_MAX_SEGS, len(segs) - i0)
        sub = C.cast(C.byref(arr, i0 * C.sizeof(CopySeg)), C.POINTER(CopySeg))
        check(lib().pp_copy_rows(sub, n, current_stream()), "pp_copy_rows")


def split_copy(src: torch.Tensor, dsts: Sequence[torch.Tensor], dim: int) -> None:
    require_cuda(src, *dsts)
    assert src.is_contiguous() and all(d.is_contiguous() for d in dsts)
    outer = 1
    for s in src.shape[:dim]:
        outer *= s
    inner = src.element_size()
    for s in src.shape[dim + 1:]:
        inner *= s
    arr = (C.c_void_p * len(dsts))(*[d.data_ptr() for d in dsts])
    check(lib().pp_split_copy(src.data_ptr(), arr, len(dsts), outer, src.shape[dim], inner,
                              current_stream()), "pp_split_copy")


def merge_copy(dst: torch.Tensor, srcs: Sequence[torch.Tensor], dim: int) -> None:
    require_cuda(dst, *srcs)
    assert dst.is_contiguous() and all(s.is_contiguous() for s in srcs)
    outer = 1
    for s in dst.shape[:dim]:
        outer *= s
    inner = dst.element_size()
    for s in dst.shape[dim + 1:]:
        inner *= s
    n = len(srcs)
    ptrs = (C.c_void_p * n)(*[s.data_ptr() for s in srcs])
    dims = (C.c_int64 * n)(*[s.shape[dim] for s in srcs])
    check(lib().pp_merge_copy(dst.data_ptr(), ptrs, dims, n, outer, inner, current_stream()),
          "pp_merge_copy")


def strided_copy_nd(dst: torch.Tensor, src: torch.Tensor) -> None:
    """dst (contiguous) <- src (any strides), same shape and dtype."""
    require_cuda(dst, src)
    assert dst.is_contiguous() and dst.shape == src.shape and dst.dtype == src.dtype
    nd = src.dim()
    sizes = (C.c_int64 * max(nd, 1))(*src.shape)
    strides = (C.c_int64 * max(nd, 1))(*src.stride())
    check(lib().pp_strided_copy_nd(dst.data_ptr(), src.data_ptr(), nd, sizes, strides,
                                   src.element_size(), current_stream()), "pp_strided_copy_nd")


# ---- gradient accumulation ------------------------------------------------------------------
def grad_accum(acc: torch.Tensor, g: torch.Tensor, init: bool = False) -> None:
    require_cuda(acc, g)
    assert acc.dtype == torch.float32 and acc.is_contiguous() and g.is_contiguous()
    assert acc.numel() == g.numel()
    if g.dtype == torch.bfloat16:
        check(lib().pp_grad_accum_f32_bf16(acc.data_ptr(), g.data_ptr(), acc.numel(), int(init),
                                           current_stream()), "pp_grad_accum_f32_bf16")
    elif g.dtype == torch.float32:
        check(lib().pp_grad_accum_f32_f32(acc.data_ptr(), g.data_ptr(), acc.numel(), int(init),
                                          current_stream()), "pp_grad_accum_f32_f32")
    else:
        raise TypeError(f"grad_accum: unsupported gradient dtype {g.dtype}")


# ---- optimizer step ---------------------------------------------------------------------------
def _pp_dtype(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return 0
    if t.dtype == torch.float32:
        return 1
    raise TypeError(f"unsupported parameter dtype {t.dtype}")


def sgd_step(param, grad, buf, *, master=None, lr, momentum=0.0, dampening=0.0, weight_decay=0.0,
             nesterov=False, first_step=False, maximize=False) -> None:
    """Flat tensors: ``param`` bf16/fp32, ``grad`` / ``buf`` / ``master`` fp32 of the same length."""
    require_cuda(param, grad)
    assert grad.dtype == torch.float32 and param.is_contiguous() and grad.is_contiguous()
    assert grad.numel() == param.numel()
    for t in (buf, master):
        assert t is None or (t.dtype == torch.float32 and t.numel() == param.numel() and t.is_contiguous())
    check(lib().pp_sgd_step(param.data_ptr(), _pp_dtype(param), _p_or_none(master), grad.data_ptr(),
                            _p_or_none(buf), param.numel(), lr, momentum, dampening, weight_decay,
                            int(nesterov), int(first_step), int(maximize), current_stream()), "pp_sgd_step")


def adamw_step(param, grad, exp_avg, exp_avg_sq, *, master=None, lr, beta1, beta2, eps, weight_decay,
               bias_correction1, bias_correction2_sqrt, maximize=False) -> None:
    require_cuda(param, grad, exp_avg, exp_avg_sq)
    assert grad.dtype == torch.float32 and param.is_contiguous() and grad.is_contiguous()
    for t in (grad, exp_avg, exp_avg_sq, master):
        assert t is None or (t.dtype == torch.float32 and t.numel() == param.numel() and t.is_contiguous())
    check(lib().pp_adamw_step(param.data_ptr(), _pp_dtype(param), _p_or_none(master), grad.data_ptr(),
                              exp_avg.data_ptr(), exp_avg_sq.data_ptr(), param.numel(), lr, beta1, beta2, eps,
                              weight_decay, bias_correction1, bias_correction2_sqrt, int(maximize),
                              current_stream()), "pp_adamw_step")


def _p_or_none(t):
    return None if t is None else t.data_ptr()


# ---- Llama-style element-wise pieces ----------------------------------------------------------
def swiglu_fwd(g, u, h) -> None:
    require_cuda(g, u, h)
    assert g.is_contiguous() and u.is_contiguous() and h.is_contiguous() and g.numel() == u.numel() == h.numel()
    check(lib().pp_swiglu_fwd(g.data_ptr(), u.data_ptr(), h.data_ptr(), g.numel(), current_stream()), "pp_swiglu_fwd")


def swiglu_bwd(g, u, dh, dg, du) -> None:
    require_cuda(g, u, dh, dg, du)
    for t in (g, u, dh, dg, du):
        assert t.is_contiguous() and t.numel() == g.numel()
    check(lib().pp_swiglu_bwd(g.data_ptr(), u.data_ptr(), dh.data_ptr(), dg.data_ptr(), du.data_ptr(), g.numel(),
                              current_stream()), "pp_swiglu_bwd")


def gemm_swiglu(x, w_gate, w_up, gu, h) -> None:
    """gu [M, 2 N] = [x w_gate^T | x w_up^T] (bf16) and h [M, N] = silu(gate) * up, in one kernel."""
    require_cuda(x, w_gate, w_up, gu, h)
    M, K = x.shape
    Nn = w_gate.shape[0]
    assert w_gate.shape == w_up.shape == (Nn, K) and gu.shape == (M, 2 * Nn) and h.shape == (M, Nn)
    assert x.stride(1) == w_gate.stride(1) == w_up.stride(1) == gu.stride(1) == h.stride(1) == 1
    assert w_gate.stride(0) == w_up.stride(0)
    check(lib().pp_gemm_bf16_swiglu(x.data_ptr(), w_gate.data_ptr(), w_up.data_ptr(), gu.data_ptr(), h.data_ptr(),
                                    M, Nn, K, x.stride(0), w_gate.stride(0), gu.stride(0), h.stride(0),
                                    current_stream()), "pp_gemm_bf16_swiglu")


def gemm_dswiglu(dy, w_down_t, gu, dgu) -> None:
    """dgu [M, 2 N] = [dg | du] from dh = dy w_down_t^T (never stored) and the saved gu = [g | u]."""
    require_cuda(dy, w_down_t, gu, dgu)
    M, K = dy.shape
    Nn = w_down_t.shape[0]
    assert w_down_t.shape == (Nn, K) and gu.shape == dgu.shape == (M, 2 * Nn)
    assert dy.stride(1) == w_down_t.stride(1) == gu.stride(1) == dgu.stride(1) == 1
    check(lib().pp_gemm_bf16_dswiglu(dy.data_ptr(), w_down_t.data_ptr(), gu.data_ptr(), dgu.data_ptr(), M, Nn, K,
                                     dy.stride(0), w_down_t.stride(0), gu.stride(0), dgu.stride(0),
                                     current_stream()), "pp_gemm_bf16_dswiglu")


def rope(x2d, cos, sin, seq: int, n_heads: int, D: int, inverse: bool = False) -> None:
    """In-place rotation of the first ``n_heads`` heads of every row of ``x2d`` [tokens, ld]."""
    require_cuda(x2d, cos, sin)
    assert x2d.dim() == 2 and x2d.stride(1) == 1 and cos.dtype == torch.float32 and sin.dtype == torch.float32
    assert cos.shape == sin.shape == (seq, D // 2) and cos.is_contiguous() and sin.is_contiguous()
    check(lib().pp_rope(x2d.data_ptr(), cos.data_ptr(), sin.data_ptr(), x2d.shape[0], seq, n_heads, D,
                        x2d.stride(0), int(inverse), current_stream()), "pp_rope")


# ---- mixture-of-experts routing and segmented GEMMs ---------------------------------------------
def gemm_segmented_swiglu(x, w_gate_list: torch.Tensor, w_up_list: torch.Tensor, seg_start: torch.Tensor, gu, h, *,
                          ld: Optional[int] = None) -> None:
    """``gemm_swiglu`` over row segments with weights of their own: rows [seg_start[e], seg_start[e + 1]) of
    ``x`` [R, K] use the [N, K] weights (leading dimension ``ld``) whose addresses are entry e of the int64
    device tensors ``w_gate_list`` and ``w_up_list``; ``gu`` [R, 2 N], ``h`` [R, N]."""
    require_cuda(x, w_gate_list, w_up_list, seg_start, gu, h)
    assert seg_start.dtype == torch.int32 and w_gate_list.dtype == w_up_list.dtype == torch.int64
    n_seg = seg_start.numel() - 1
    assert w_gate_list.numel() == w_up_list.numel() == n_seg
    R, K = x.shape
    Nn = h.shape[1]
    assert gu.shape == (R, 2 * Nn) and h.shape[0] == R and x.stride(1) == gu.stride(1) == h.stride(1) == 1
    check(lib().pp_gemm_bf16_segmented_swiglu(x.data_ptr(), w_gate_list.data_ptr(), w_up_list.data_ptr(),
                                              seg_start.data_ptr(), n_seg, gu.data_ptr(), h.data_ptr(), R, Nn, K,
                                              x.stride(0), ld if ld is not None else K, gu.stride(0), h.stride(0),
                                              current_stream()), "pp_gemm_bf16_segmented_swiglu")


def gemm_segmented_dswiglu(dy, w_down_t_list: torch.Tensor, seg_start: torch.Tensor, gu, dgu, *,
                           ld: Optional[int] = None) -> None:
    """``gemm_dswiglu`` over row segments: rows [seg_start[e], seg_start[e + 1]) of ``dy`` [R, K] use the
    transposed down projection [N, K] (leading dimension ``ld``) at entry e of ``w_down_t_list``."""
    require_cuda(dy, w_down_t_list, seg_start, gu, dgu)
    assert seg_start.dtype == torch.int32 and w_down_t_list.dtype == torch.int64
    n_seg = seg_start.numel() - 1
    assert w_down_t_list.numel() == n_seg
    R, K = dy.shape
    Nn = gu.shape[1] // 2
    assert gu.shape == dgu.shape == (R, 2 * Nn) and dy.stride(1) == gu.stride(1) == dgu.stride(1) == 1
    check(lib().pp_gemm_bf16_segmented_dswiglu(dy.data_ptr(), w_down_t_list.data_ptr(), seg_start.data_ptr(), n_seg,
                                               gu.data_ptr(), dgu.data_ptr(), R, Nn, K, dy.stride(0),
                                               ld if ld is not None else K, gu.stride(0), dgu.stride(0),
                                               current_stream()), "pp_gemm_bf16_segmented_dswiglu")


def gemm_bf16_segmented(A, B_or_C_list: torch.Tensor, Cm, seg_start: torch.Tensor, mode: int, *, other=None,
                        N: Optional[int] = None, ld: Optional[int] = None, epilogue: int = EPI_NONE,
                        aux_in=None, beta: int = 0, c_dtype=None) -> None:
    """Segmented GEMM (see ``pp_gemm_bf16_segmented``).

    rows mode: ``A`` [R, K], ``Cm`` [R, N]; ``B_or_C_list`` is an int64 device tensor of per-segment B
    pointers ([N, K] each, leading dimension ``ld``).
    k mode: ``A`` [R, M] and ``other`` [R, N] are the transposed operands; ``B_or_C_list`` holds the
    per-segment C pointers ([M, N], leading dimension ``ld``, dtype ``c_dtype``); ``Cm`` is None."""
    require_cuda(A, B_or_C_list, seg_start, Cm, other, aux_in)
    assert seg_start.dtype == torch.int32 and B_or_C_list.dtype == torch.int64
    n_seg = seg_start.numel() - 1
    assert B_or_C_list.numel() == n_seg
    if mode not in (SEG_ROWS, SEG_K):
        raise ValueError(f"unknown mode {mode}: SEG_ROWS or SEG_K")
    d = GemmDesc()
    if mode == SEG_ROWS:
        assert A.stride(1) == 1 and Cm.stride(1) == 1 and A.shape[0] == Cm.shape[0]
        d.A, d.B, d.C = A.data_ptr(), None, Cm.data_ptr()
        d.M, d.N, d.K = A.shape[0], Cm.shape[1], A.shape[1]
        d.lda, d.ldb, d.ldc = A.stride(0), ld if ld is not None else A.shape[1], Cm.stride(0)
        d.a_trans = d.b_trans = 0
        d.c_dtype = PP_BF16
        if aux_in is not None:
            assert aux_in.shape == Cm.shape and aux_in.stride(1) == 1
            d.aux_in, d.ld_aux = aux_in.data_ptr(), aux_in.stride(0)
    else:
        assert other is not None and A.shape[0] == other.shape[0] and A.stride(1) == 1 and other.stride(1) == 1
        d.A, d.B, d.C = A.data_ptr(), other.data_ptr(), None
        d.M, d.N, d.K = A.shape[1], other.shape[1], A.shape[0]
        d.lda, d.ldb, d.ldc = A.stride(0), other.stride(0), ld if ld is not None else other.shape[1]
        d.a_trans = d.b_trans = 1
        d.c_dtype = PP_F32 if c_dtype == torch.float32 else PP_BF16
    d.epilogue, d.beta = epilogue, beta
    check(lib().pp_gemm_bf16_segmented(C.byref(d), seg_start.data_ptr(), B_or_C_list.data_ptr(), n_seg, mode,
                                       current_stream()), "pp_gemm_bf16_segmented")


def moe_router_top2(logits, topk_idx, gate) -> None:
    require_cuda(logits, topk_idx, gate)
    T, E = logits.shape
    assert logits.dtype == torch.bfloat16 and logits.stride(1) == 1
    assert topk_idx.dtype == torch.int32 and topk_idx.is_contiguous() and topk_idx.numel() == 2 * T
    assert gate.dtype == torch.float32 and gate.is_contiguous() and gate.numel() == 2 * T
    check(lib().pp_moe_router_top2(logits.data_ptr(), logits.stride(0), T, E, topk_idx.data_ptr(), gate.data_ptr(),
                                   current_stream()), "pp_moe_router_top2")


def moe_permute(expert_of_slot, E: int, seg_start, row_src, pos) -> None:
    require_cuda(expert_of_slot, seg_start, row_src, pos)
    n = expert_of_slot.numel()
    for t in (expert_of_slot, seg_start, row_src, pos):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert seg_start.numel() == E + 1 and row_src.numel() == n and pos.numel() == n
    check(lib().pp_moe_permute(expert_of_slot.data_ptr(), n, E, seg_start.data_ptr(), row_src.data_ptr(),
                               pos.data_ptr(), current_stream()), "pp_moe_permute")


def moe_gather(src, row_src, topk: int, dst, *, scale=None, n_rows=None) -> None:
    require_cuda(src, row_src, dst, scale, n_rows)
    assert src.stride(1) == 1 and dst.stride(1) == 1 and src.shape[1] == dst.shape[1]
    assert row_src.dtype == torch.int32 and row_src.numel() == dst.shape[0]
    assert scale is None or (scale.dtype == torch.float32 and scale.is_contiguous())
    check(lib().pp_moe_gather(src.data_ptr(), src.stride(0), row_src.data_ptr(), _p_or_none(n_rows), topk,
                              _p_or_none(scale), dst.data_ptr(), dst.stride(0), dst.shape[0], dst.shape[1],
                              current_stream()), "pp_moe_gather")


def moe_combine(y, pos, topk: int, out, *, gate=None, resid=None) -> None:
    require_cuda(y, pos, out, gate, resid)
    T, Cc = out.shape
    assert y.stride(1) == 1 and out.stride(1) == 1 and y.shape[1] == Cc
    assert pos.dtype == torch.int32 and pos.numel() == T * topk
    assert gate is None or (gate.dtype == torch.float32 and gate.is_contiguous() and gate.numel() == T * topk)
    assert resid is None or (resid.shape == out.shape and resid.stride(1) == 1)
    check(lib().pp_moe_combine(y.data_ptr(), y.stride(0), pos.data_ptr(), _p_or_none(gate), topk,
                               _p_or_none(resid), resid.stride(0) if resid is not None else 0, out.data_ptr(),
                               out.stride(0), T, Cc, current_stream()), "pp_moe_combine")


def moe_gate_bwd(dout, y, pos, topk_idx, gate, E: int, dlogits) -> None:
    require_cuda(dout, y, pos, topk_idx, gate, dlogits)
    T, Cc = dout.shape
    topk = pos.numel() // T
    assert dlogits.shape == (T, (E + 7) // 8 * 8) and dlogits.dtype == torch.bfloat16 and dlogits.stride(1) == 1
    check(lib().pp_moe_gate_bwd(dout.data_ptr(), dout.stride(0), y.data_ptr(), y.stride(0), pos.data_ptr(),
                                topk_idx.data_ptr(), gate.data_ptr(), topk, E, dlogits.data_ptr(),
                                dlogits.stride(0), T, Cc, current_stream()), "pp_moe_gate_bwd")


def fill_bytes(t: torch.Tensor, value: int = 0) -> None:
    require_cuda(t)
    assert t.is_contiguous()
    check(lib().pp_fill_bytes(t.data_ptr(), value, t.numel() * t.element_size(),
                              current_stream()), "pp_fill_bytes")


# ---- GEMM -------------------------------------------------------------------------------------
def gemm_desc(A: torch.Tensor, B: torch.Tensor, Cm: torch.Tensor, *, a_trans: bool = False,
              b_trans: bool = False, epilogue: int = EPI_NONE, bias: Optional[torch.Tensor] = None,
              aux_in: Optional[torch.Tensor] = None, aux_out: Optional[torch.Tensor] = None,
              beta: int = 0, colsum: Optional[torch.Tensor] = None) -> GemmDesc:
    """A: [M,K] (or [K,M] if a_trans); B: [N,K] (or [K,N] if b_trans); Cm: [M,N].
    Row-major 2-d tensors whose last stride is 1 (a row stride larger than the row is fine)."""
    require_cuda(A, B, Cm, bias, aux_in, aux_out)
    for t in (A, B, Cm, aux_in, aux_out):
        if t is not None:
            assert t.dim() == 2 and t.stride(1) == 1, "GEMM operands are row-major 2-d"
    M, N = Cm.shape
    K = A.shape[0] if a_trans else A.shape[1]
    assert (A.shape[1] if a_trans else A.shape[0]) == M, "A does not match C"
    assert (B.shape[1] if b_trans else B.shape[0]) == N, "B does not match C"
    assert (B.shape[0] if b_trans else B.shape[1]) == K, "A and B disagree on K"
    d = GemmDesc()
    d.A, d.B, d.C = A.data_ptr(), B.data_ptr(), Cm.data_ptr()
    d.M, d.N, d.K = M, N, K
    d.lda, d.ldb, d.ldc = A.stride(0), B.stride(0), Cm.stride(0)
    d.a_trans, d.b_trans = int(a_trans), int(b_trans)
    d.epilogue = epilogue
    d.c_dtype = PP_F32 if Cm.dtype == torch.float32 else PP_BF16
    d.bias = ptr(bias)
    d.aux_in = ptr(aux_in)
    d.aux_out = ptr(aux_out)
    ld_aux = 0
    for t in (aux_in, aux_out):
        if t is not None:
            assert t.shape == Cm.shape
            assert ld_aux in (0, t.stride(0)), "aux_in and aux_out share one leading dimension"
            ld_aux = t.stride(0)
    d.ld_aux = ld_aux
    d.beta = beta
    if colsum is not None:
        require_cuda(colsum)
        assert colsum.dtype == torch.float32 and colsum.numel() >= ((M + GEMM_COLSUM_ROWS - 1) // GEMM_COLSUM_ROWS) * N
    d.colsum = ptr(colsum)
    return d


def gemm_bf16(A, B, Cm, **kw) -> None:
    assert A.dtype == torch.bfloat16 and B.dtype == torch.bfloat16
    d = gemm_desc(A, B, Cm, **kw)
    check(lib().pp_gemm_bf16(C.byref(d), current_stream()), "pp_gemm_bf16")


def gemm_bf16_splitk(A, B, Cm, workspace: torch.Tensor, **kw) -> None:
    """``gemm_bf16`` that may split a long K over several work-groups per tile, through ``workspace``
    (fp32, up to 8 copies of C)."""
    require_cuda(workspace)
    assert workspace.dtype == torch.float32 and workspace.is_contiguous()
    d = gemm_desc(A, B, Cm, **kw)
    check(lib().pp_gemm_bf16_splitk(C.byref(d), workspace.data_ptr(), workspace.numel(), current_stream()),
          "pp_gemm_bf16_splitk")


def gemm_bf16_grouped(problems) -> None:
    """problems: list of (A, B, C, kwargs) sharing layout flags, epilogue and output dtype."""
    arr = (GemmDesc * len(problems))()
    for k, (A, B, Cm, kw) in enumerate(problems):
        d = gemm_desc(A, B, Cm, **kw)
        C.memmove(C.byref(arr, k * C.sizeof(GemmDesc)), C.byref(d), C.sizeof(GemmDesc))
    check(lib().pp_gemm_bf16_grouped(arr, len(problems), current_stream()), "pp_gemm_bf16_grouped")


class KsegLaunch:
    """Descriptors and device pointer tables of one ``pp_gemm_bf16_grouped_kseg`` launch, built once.

    problems: list of (As, Bs, C, kwargs): the weight gradient C (fp32) over the segments (microbatches)
    s of As[s]^T Bs[s], added in ascending s, all problems in one launch."""

    def __init__(self, problems):
        self.n_seg = len(problems[0][0])
        self.n = len(problems)
        self.arr = (GemmDesc * self.n)()
        ptrs = []
        for As, Bs, Cm, kw in problems:
            assert len(As) == len(Bs) == self.n_seg
            for t in list(As) + list(Bs):
                assert t.data_ptr() % 16 == 0 and t.dtype == torch.bfloat16
            assert all(a.shape == As[0].shape and a.stride() == As[0].stride() for a in As)
            assert all(b.shape == Bs[0].shape and b.stride() == Bs[0].stride() for b in Bs)
            ptrs += [a.data_ptr() for a in As] + [b.data_ptr() for b in Bs]
        # one table for the whole launch: problem k's A pointers at [2 k n_seg, ...), its B pointers after them
        self.table = torch.tensor(ptrs, dtype=torch.int64, device=problems[0][2].device)
        for k, (As, Bs, Cm, kw) in enumerate(problems):
            d = gemm_desc(As[0], Bs[0], Cm, a_trans=True, b_trans=True, **kw)
            d.A = self.table.data_ptr() + 8 * (2 * k * self.n_seg)
            d.B = self.table.data_ptr() + 8 * ((2 * k + 1) * self.n_seg)
            C.memmove(C.byref(self.arr, k * C.sizeof(GemmDesc)), C.byref(d), C.sizeof(GemmDesc))
        self.keep = problems

    def run(self) -> None:
        check(lib().pp_gemm_bf16_grouped_kseg(self.arr, self.n, self.n_seg, current_stream()),
              "pp_gemm_bf16_grouped_kseg")


def gemm_bf16_grouped_kseg(problems, keep=None) -> None:
    """One launch of ``KsegLaunch(problems)``; ``keep`` (a list) receives the launch object, whose pointer
    table must outlive the kernel (without it the call waits for the stream)."""
    launch = KsegLaunch(problems)
    launch.run()
    if keep is not None:
        keep.append(launch)
    else:
        torch.cuda.current_stream().synchronize()


def gemm_f32(A, B, Cm, **kw) -> None:
    assert A.dtype == torch.float32 and B.dtype == torch.float32 and Cm.dtype == torch.float32
    d = gemm_desc(A, B, Cm, **kw)
    check(lib().pp_gemm_f32(C.byref(d), current_stream()), "pp_gemm_f32")


def colsum(dY: torch.Tensor, out: torch.Tensor, workspace: torch.Tensor) -> None:
    require_cuda(dY, out, workspace)
    M, N = dY.shape
    assert dY.stride(1) == 1 and out.numel() == N and workspace.dtype == torch.float32
    assert workspace.numel() >= ((M + 127) // 128) * N
    check(lib().pp_colsum_bf16(dY.data_ptr(), M, N, dY.stride(0), out.data_ptr(),
                               PP_F32 if out.dtype == torch.float32 else PP_BF16,
                               workspace.data_ptr(), current_stream()), "pp_colsum_bf16")


def colreduce_grouped(items) -> None:
    """items: dicts with dy, out_sum and/or out_dot, workspace and, for out_dot, x, mean, rstd; with
    ``n_part_ready`` = P the workspace already holds P rows of partial sums and dy only gives the shape."""
    arr = (ColReduceDesc * len(items))()
    for d, it in zip(arr, items):
        dy = it["dy"]
        require_cuda(dy, it.get("x"), it.get("out_sum"), it.get("out_dot"), it["workspace"])
        d.dy, d.ld_dy, d.rows, d.C = dy.data_ptr(), dy.stride(0), dy.shape[0], dy.shape[1]
        d.x, d.mean, d.rstd = ptr(it.get("x")), ptr(it.get("mean")), ptr(it.get("rstd"))
        d.out_sum, d.out_dot = ptr(it.get("out_sum")), ptr(it.get("out_dot"))
        d.workspace = it["workspace"].data_ptr()
        d.n_part_ready = int(it.get("n_part_ready", 0))
        assert it["workspace"].numel() >= (d.n_part_ready or 2 * ((dy.shape[0] + 127) // 128)) * dy.shape[1]
        out = it.get("out_sum") if it.get("out_sum") is not None else it.get("out_dot")
        d.out_dtype = PP_F32 if out.dtype == torch.float32 else PP_BF16
    check(lib().pp_colreduce_grouped(arr, len(items), current_stream()), "pp_colreduce_grouped")


# ---- LayerNorm --------------------------------------------------------------------------------
def layernorm_fwd(x, gamma, beta, y, mean, rstd, eps: float) -> None:
    require_cuda(x, gamma, beta, y, mean, rstd)
    rows, Cc = x.shape
    check(lib().pp_layernorm_fwd(x.data_ptr(), gamma.data_ptr(), ptr(beta), y.data_ptr(),
                                 ptr(mean), rstd.data_ptr(), rows, Cc, eps,
                                 current_stream()), "pp_layernorm_fwd")


def layernorm_bwd_input(dy, x, gamma, mean, rstd, dres, dx) -> None:
    require_cuda(dy, x, gamma, mean, rstd, dres, dx)
    rows, Cc = x.shape
    check(lib().pp_layernorm_bwd_input(dy.data_ptr(), x.data_ptr(), gamma.data_ptr(),
                                       ptr(mean), rstd.data_ptr(), ptr(dres), dx.data_ptr(),
                                       rows, Cc, current_stream()), "pp_layernorm_bwd_input")


GEMM_COLSUM_ROWS = 32  # PP_GEMM_COLSUM_ROWS: rows of C per row of column sums that a GEMM epilogue leaves
LN_SUM_ROWS = 16     # PP_LN_SUM_ROWS: rows per partial-sum row of pp_layernorm_bwd_input_sums
LN_SUM_MAX_C = 1024  # PP_LN_SUM_MAX_C


def layernorm_bwd_input_sums(dy, x, gamma, mean, rstd, dres, dx, ws_weight=None, ws_dx=None) -> int:
    """The input gradient plus rows of partial column sums (one per ``LN_SUM_ROWS`` rows): ``ws_weight``
    fp32 [2, P, C] (sum of dy, sum of dy * xhat), ``ws_dx`` fp32 [P, C] (sum of dx).  Returns P."""
    require_cuda(dy, x, gamma, mean, rstd, dres, dx, ws_weight, ws_dx)
    rows, Cc = x.shape
    n_part = (rows + LN_SUM_ROWS - 1) // LN_SUM_ROWS
    assert ws_weight is None or (ws_weight.dtype == torch.float32 and ws_weight.numel() >= 2 * n_part * Cc)
    assert ws_dx is None or (ws_dx.dtype == torch.float32 and ws_dx.numel() >= n_part * Cc)
    check(lib().pp_layernorm_bwd_input_sums(dy.data_ptr(), x.data_ptr(), gamma.data_ptr(), ptr(mean),
                                            rstd.data_ptr(), ptr(dres), dx.data_ptr(), rows, Cc, ptr(ws_weight),
                                            ptr(ws_dx), current_stream()), "pp_layernorm_bwd_input_sums")
    return n_part


def layernorm_bwd_weight(dy, x, mean, rstd, dgamma, dbeta, workspace) -> None:
    require_cuda(dy, x, mean, rstd, dgamma, dbeta, workspace)
    rows, Cc = x.shape
    assert workspace.numel() >= 2 * ((rows + 127) // 128) * Cc
    check(lib().pp_layernorm_bwd_weight(dy.data_ptr(), x.data_ptr(), ptr(mean),
                                        rstd.data_ptr(), dgamma.data_ptr(), ptr(dbeta),
                                        PP_F32 if dgamma.dtype == torch.float32 else PP_BF16,
                                        workspace.data_ptr(), rows, Cc, current_stream()),
          "pp_layernorm_bwd_weight")


# ---- attention --------------------------------------------------------------------------------
def attn_desc(qkv: torch.Tensor, o: torch.Tensor, lse: torch.Tensor, H: int, causal: bool,
              scale: Optional[float] = None, d_o: Optional[torch.Tensor] = None,
              dqkv: Optional[torch.Tensor] = None, delta: Optional[torch.Tensor] = None,
              n_kv_heads: Optional[int] = None, kv_len: Optional[int] = None, exact_dq: bool = False,
              colsum: Optional[torch.Tensor] = None) -> AttnDesc:
    """qkv: [B, S, (H + 2 H_kv) * D] fused projection output (q | k | v along the last dim);
    ``n_kv_heads`` < H: grouped-query attention (H / n_kv_heads query heads per key / value head);
    ``kv_len`` < S: rows kv_len .. S-1 of every sequence are (zero) padding that the forward masks;
    ``exact_dq``: the backward corrects dq for the rounding of the forward's output (PP_ATTN_EXACT_DQ);
    ``colsum`` (backward, head size 64): fp32 [B * S / 64, width], receives the column sums of every block of
    64 tokens of dqkv as stored."""
    require_cuda(qkv, o, lse, d_o, dqkv, delta)
    B, S, width = qkv.shape
    Hkv = H if n_kv_heads is None else n_kv_heads
    assert 0 < Hkv <= H and H % Hkv == 0 and width % (H + 2 * Hkv) == 0
    D = width // (H + 2 * Hkv)
    HD, KD = H * D, Hkv * D
    assert qkv.stride(2) == 1 and o.is_contiguous() and o.shape == (B, S, HD)
    es = qkv.element_size()
    d = AttnDesc()
    base = qkv.data_ptr()
    d.q, d.k, d.v = base, base + HD * es, base + (HD + KD) * es
    d.kv_group = H // Hkv
    d.o, d.lse = o.data_ptr(), lse.data_ptr()
    d.B, d.S, d.H, d.D = B, S, H, D
    d.stride_b, d.stride_s = qkv.stride(0), qkv.stride(1)
    d.scale = scale if scale is not None else D ** -0.5
    d.causal = int(causal)
    assert kv_len is None or 0 < kv_len <= S
    d.kv_len = 0 if kv_len is None else kv_len
    d.flags = ATTN_EXACT_DQ if exact_dq else 0
    if d_o is not None:
        assert dqkv is not None and delta is not None
        assert dqkv.shape == qkv.shape and dqkv.stride() == qkv.stride() and d_o.is_contiguous()
        gb = dqkv.data_ptr()
        d.d_o = d_o.data_ptr()
        d.dq, d.dk, d.dv = gb, gb + HD * es, gb + (HD + KD) * es
        d.delta = delta.data_ptr()
        if colsum is not None:
            require_cuda(colsum)
            assert colsum.dtype == torch.float32 and colsum.is_contiguous() and colsum.shape == (B * S // 64, width)
            d.colsum, d.ld_colsum = colsum.data_ptr(), width
    return d


def attn_fwd(qkv, o, lse, H, causal, scale=None, n_kv_heads=None, kv_len=None) -> None:
    d = attn_desc(qkv, o, lse, H, causal, scale, n_kv_heads=n_kv_heads, kv_len=kv_len)
    check(lib().pp_attn_fwd(C.byref(d), current_stream()), "pp_attn_fwd")


def attn_bwd(qkv, o, lse, d_o, dqkv, delta, H, causal, scale=None, n_kv_heads=None, kv_len=None,
             exact_dq=False, colsum=None) -> None:
    d = attn_desc(qkv, o, lse, H, causal, scale, d_o=d_o, dqkv=dqkv, delta=delta, n_kv_heads=n_kv_heads,
                  kv_len=kv_len, exact_dq=exact_dq, colsum=colsum)
    check(lib().pp_attn_bwd(C.byref(d), current_stream()), "pp_attn_bwd")


# ---- embedding / loss -------------------------------------------------------------------------
def embed_fwd(ids, wte, wpe, y, seq: int, extra_row=None) -> None:
    require_cuda(ids, wte, wpe, y)
    assert ids.dtype == torch.int64 and ids.is_contiguous() and y.is_contiguous()
    vocab, Cc = wte.shape
    assert extra_row is None or (extra_row.numel() == Cc and extra_row.is_contiguous())
    check(lib().pp_embed_fwd(ids.data_ptr(), wte.data_ptr(), ptr(wpe), ptr(extra_row), y.data_ptr(),
                             ids.numel(), seq, Cc, vocab, current_stream()), "pp_embed_fwd")


def embed_fwd_at(ids, pos_ids, wte, wpe, y, extra_row=None) -> None:
    """As ``embed_fwd`` with the row of the position table given per token (``pos_ids`` int64, like ``ids``)."""
    require_cuda(ids, pos_ids, wte, wpe, y)
    assert ids.dtype == pos_ids.dtype == torch.int64 and ids.is_contiguous() and pos_ids.is_contiguous()
    assert pos_ids.numel() == ids.numel() and y.is_contiguous() and wpe.shape[1] == wte.shape[1]
    vocab, Cc = wte.shape
    assert extra_row is None or (extra_row.numel() == Cc and extra_row.is_contiguous())
    check(lib().pp_embed_fwd_at(ids.data_ptr(), pos_ids.data_ptr(), wte.data_ptr(), wpe.data_ptr(), ptr(extra_row),
                                y.data_ptr(), ids.numel(), wpe.shape[0], Cc, vocab, current_stream()),
          "pp_embed_fwd_at")


def position_ids_from_padding(ids, out, pad: int) -> None:
    """out[b, s] = pad where ids[b, s] == pad, else pad + the count of tokens != pad among ids[b, :s + 1]."""
    require_cuda(ids, out)
    assert ids.dtype == out.dtype == torch.int64 and ids.dim() == 2 and out.shape == ids.shape
    assert ids.is_contiguous() and out.is_contiguous()
    check(lib().pp_position_ids_from_padding(ids.data_ptr(), out.data_ptr(), ids.shape[0], ids.shape[1], pad,
                                             current_stream()), "pp_position_ids_from_padding")


def embed_bwd(ids, dy, d_wte, d_wpe, seq: int, round_bf16: bool = False, padding_idx: Optional[int] = None) -> None:
    """``padding_idx``: the row of ``d_wte`` that receives no gradient (its tokens are skipped)."""
    require_cuda(ids, dy, d_wte, d_wpe)
    vocab, Cc = d_wte.shape
    pad = -1 if padding_idx is None else padding_idx % vocab
    check(lib().pp_embed_bwd(ids.data_ptr(), dy.data_ptr(), d_wte.data_ptr(), ptr(d_wpe),
                             ids.numel(), seq, Cc, vocab, int(round_bf16), pad, current_stream()), "pp_embed_bwd")


def ce_loss(logits, target, loss, dlogits, workspace, V: int, ignore_index: int = -100) -> None:
    """logits: [rows, ld] with the first V columns valid (ld = logits.stride(0))."""
    require_cuda(logits, target, loss, dlogits, workspace)
    rows = logits.shape[0]
    assert logits.stride(1) == 1 and target.numel() == rows and workspace.numel() >= rows + 2
    if dlogits is not None:
        assert dlogits.stride() == logits.stride()
    check(lib().pp_ce_loss(logits.data_ptr(), target.data_ptr(), loss.data_ptr(), ptr(dlogits),
                           workspace.data_ptr(), rows, V, logits.stride(0), ignore_index,
                           PP_F32 if logits.dtype == torch.float32 else PP_BF16,
                           current_stream()), "pp_ce_loss")


def activation_bwd(dy, aux, dz, act: int) -> None:
    require_cuda(dy, aux, dz)
    assert dy.is_contiguous() and aux.is_contiguous() and dz.is_contiguous()
    assert dy.numel() == aux.numel() == dz.numel() and dy.dtype == aux.dtype == dz.dtype
    check(lib().pp_activation_bwd(dy.data_ptr(), aux.data_ptr(), dz.data_ptr(), dy.numel(), act,
                                  PP_F32 if dy.dtype == torch.float32 else PP_BF16,
                                  current_stream()), "pp_activation_bwd")


def transpose_bf16(src: torch.Tensor, dst: torch.Tensor) -> None:
    """dst[c, r] = src[r, c]; 2-d, 2-byte elements, unit inner strides."""
    require_cuda(src, dst)
    assert src.dim() == 2 and dst.dim() == 2 and src.stride(1) == 1 and dst.stride(1) == 1
    assert dst.shape == (src.shape[1], src.shape[0]) and src.element_size() == 2 == dst.element_size()
    check(lib().pp_transpose_bf16(src.data_ptr(), src.shape[0], src.shape[1], src.stride(0),
                                  dst.data_ptr(), dst.stride(0), current_stream()), "pp_transpose_bf16")


def run_ops(ops, n: int) -> None:
    check(lib().pp_run_ops(ops, n, current_stream()), "pp_run_ops")


# ---- per-launch timing ---------------------------------------------------------------------------
def profile_start(max_records: int = 1 << 16) -> None:
    check(lib().pp_profile_start(max_records), "pp_profile_start")


def profile_stop() -> None:
    check(lib().pp_profile_stop(), "pp_profile_stop")


def profile_read(kind: int):
    """(total_ms, total_work, count) of the ops of one kind recorded since profile_start."""
    ms, work, cnt = C.c_double(), C.c_double(), C.c_int64()
    check(lib().pp_profile_read(kind, C.byref(ms), C.byref(work), C.byref(cnt)), "pp_profile_read")
    return ms.value, work.value, cnt.value
