"""Stage programs: a stage module lowered to launch lists of HIP kernels.

The reference executes a stage by calling the user's ``nn.Module`` (``_PipelineStage.py:420-428``)
and one fused ``torch.autograd.backward`` (``_backward.py:67-69``).  Here a stage whose module is
built from the blocks in ``stage_modules.py`` is *lowered* once per microbatch slot into three
launch lists over pre-allocated device buffers:

* ``F``  forward;
* ``I``  input-gradient pass (dI): gradients w.r.t. the stage input;
* ``W``  weight-gradient pass (dW): parameter gradients, then their fp32 accumulation.

A fused backward is ``I`` followed by ``W``; a zero-bubble schedule runs them apart.  Lists are
replayed with one ``pp_run_ops`` call each, so the host language is left once per pass.

HBM layout per stage: one flat parameter arena (module parameters are views into it, names
unchanged), one flat staging arena for the per-microbatch parameter gradients in the parameter
dtype, and one flat fp32 accumulator arena; per microbatch slot, the activations saved for
backward and the stage output plus the gradient buffer of that output (the next stage writes its
input gradient straight into it: the hand-off is a pointer, not a copy).
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from . import _native as N

_ALIGN_ELEMS = 128  # every arena entry starts on a 256-byte boundary


def _round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


class ParamArena:
    """Flat storage of one stage's parameters, gradient staging and fp32 accumulators."""

    def __init__(self, module: nn.Module, device: torch.device, blocks: Sequence[nn.Module] = ()):
        params = [(n, p) for n, p in module.named_parameters()]
        if not params:
            self.dtype = torch.bfloat16
        else:
            dts = {p.dtype for _, p in params}
            if len(dts) != 1:
                raise RuntimeError(f"a native stage needs one parameter dtype, found {dts}")
            self.dtype = dts.pop()
        if self.dtype not in (torch.bfloat16, torch.float32):
            raise RuntimeError(f"native stages support bf16 or fp32 parameters, not {self.dtype}")
        pad_rows: Dict[int, int] = {}
        direct = set()
        # the blocks may be wrappers around the module's layers that are not part of the module itself
        holders = {id(m): m for m in module.modules()}
        for blk in blocks:
            holders.update({id(m): m for m in blk.modules()})
        for mod in holders.values():
            for p, rows in getattr(mod, "_pp_padded_rows", lambda: [])():
                pad_rows[id(p)] = rows
            for p in getattr(mod, "_pp_direct_acc_params", lambda: [])():
                direct.add(id(p))
        # parameters whose gradient goes through the staging arena come first; the single
        # accumulate op of a W pass covers [0, staged_total)
        # and among them matrices before vectors: the weight-gradient GEMMs add into the accumulators
        # themselves, so what is left for the accumulate op is (normally) one range of small tensors
        params = [q for q in params if id(q[1]) not in direct and q[1].dim() >= 2] + \
                 [q for q in params if id(q[1]) not in direct and q[1].dim() < 2] + \
                 [q for q in params if id(q[1]) in direct]
        self.entries: Dict[int, Tuple[int, int, Tuple[int, ...]]] = {}  # id(p) -> (off, numel, padded shape)
        off = 0
        self.staged_total = 0
        for _, p in params:
            if id(p) in direct and self.staged_total == 0:
                self.staged_total = off
            shape = tuple(p.shape)
            if id(p) in pad_rows:
                shape = (pad_rows[id(p)],) + shape[1:]
            numel = 1
            for s in shape:
                numel *= s
            self.entries[id(p)] = (off, numel, shape)
            off = _round_up(off + numel, _ALIGN_ELEMS)
        self.total = off
        if not direct:
            self.staged_total = off
        elif all(id(p) in direct for _, p in params):
            self.staged_total = 0
        self.device = device
        self.params = torch.zeros(max(off, 1), dtype=self.dtype, device=device)
        self.staging = torch.zeros(max(off, 1), dtype=self.dtype, device=device)
        self.acc = torch.zeros(max(off, 1), dtype=torch.float32, device=device)
        for _, p in params:
            o, _n, _shape = self.entries[id(p)]
            view = self.params[o:o + p.numel()].view(p.shape)
            view.copy_(p.detach().to(device))
            p.data = view
        self.named = params
        # transposed copies of linear weights ([in, out]) for the input-gradient GEMMs
        self._transposed: Dict[int, Tuple[nn.Parameter, torch.Tensor]] = {}
        self._stacked: Dict[Tuple[int, ...], Tuple[torch.Tensor, List[Tuple[nn.Parameter, torch.Tensor]]]] = {}
        self._versions = None
        self._epoch = 0  # bumped by updates that write the arena directly (fused optimizers)

    def weight_t(self, p: nn.Parameter) -> torch.Tensor:
        """[in, out_padded] copy of a 2-d weight, kept in step with the parameter by
        ``refresh_transposed``."""
        ent = self._transposed.get(id(p))
        if ent is None:
            w = self.weight(p, padded=True)
            t = torch.empty((w.shape[1], w.shape[0]), dtype=w.dtype, device=self.device)
            N.transpose_bf16(w, t)
            ent = (p, t)
            self._transposed[id(p)] = ent
        return ent[1]

    def weight_t_cat(self, *ps: nn.Parameter) -> torch.Tensor:
        """[in, out1 + out2 + ...]: the transposed copies of weights with the same input width side by
        side, so that dY1 W1 + dY2 W2 + ... is ONE product of [dY1 | dY2 | ...] with this matrix.  Kept in
        step with the parameters by ``refresh_transposed``."""
        key = ("cat",) + tuple(id(p) for p in ps)
        ent = self._transposed.get(key)
        if ent is None:
            ws = [self.weight(p, padded=True) for p in ps]
            assert all(w.shape[1] == ws[0].shape[1] for w in ws)
            t = torch.empty((ws[0].shape[1], sum(w.shape[0] for w in ws)), dtype=ws[0].dtype, device=self.device)
            lo = 0
            for k, (p, w) in enumerate(zip(ps, ws)):
                view = t[:, lo:lo + w.shape[0]]
                lo += w.shape[0]
                N.transpose_bf16(w, view)
                self._transposed[key + (k,)] = (p, view)
            ent = (None, t)
            self._transposed[key] = ent
        return ent[1]

    def weight_t_stack(self, p: nn.Parameter) -> torch.Tensor:
        """[E, in, out]: the transposed copy of every [out, in] matrix of a stacked 3-d weight, kept in
        step with the parameter by ``refresh_transposed``."""
        key = ("stack", id(p))
        ent = self._transposed.get(key)
        if ent is None:
            w = self.weight(p, padded=True)
            t = torch.empty((w.shape[0], w.shape[2], w.shape[1]), dtype=w.dtype, device=self.device)
            for e in range(w.shape[0]):
                N.transpose_bf16(w[e], t[e])
                self._transposed[key + (e,)] = (p, t[e], e)
            ent = (None, t)
            self._transposed[key] = ent
        return ent[1]

    def rows_cat(self, *ps: nn.Parameter) -> torch.Tensor:
        """[out1 + out2 + ..., in] (or the 1-d analogue for biases): copies of parameters with the same
        trailing shape stacked along dimension 0, so that projections which read the same input run as
        ONE GEMM.  Kept in step with the parameters by ``refresh_transposed``."""
        key = tuple(id(p) for p in ps)
        ent = self._stacked.get(key)
        if ent is None:
            ws = [self.weight(p, padded=True) for p in ps]
            t = torch.cat(ws, dim=0)
            parts, lo = [], 0
            for p, w in zip(ps, ws):
                parts.append((p, t[lo:lo + w.shape[0]]))
                lo += w.shape[0]
            ent = (t, parts)
            self._stacked[key] = ent
        return ent[0]

    def refresh_transposed(self) -> None:
        """Re-transposes (re-copies) the weights whose parameter changed since the last call (an
        optimizer step bumps the parameter's version counter)."""
        if not self._transposed and not self._stacked:
            return
        live = [ent for ent in self._transposed.values() if ent[0] is not None]
        stacked = [(p, view) for _, parts in self._stacked.values() for p, view in parts]
        versions = (self._epoch,) + tuple(ent[0]._version for ent in live) + tuple(p._version for p, _ in stacked)
        if versions == self._versions:
            return
        self._versions = versions
        for ent in live:      # (parameter, copy[, index of the matrix inside a stacked parameter])
            src = self.weight(ent[0], padded=True)
            N.transpose_bf16(src if len(ent) == 2 else src[ent[2]], ent[1])
        for p, view in stacked:
            view.copy_(self.weight(p, padded=True))

    def mark_updated(self) -> None:
        """The parameter arena was written behind the parameters' version counters."""
        self._epoch += 1

    def _slice(self, flat: torch.Tensor, p: nn.Parameter, padded: bool) -> torch.Tensor:
        o, numel, shape = self.entries[id(p)]
        if padded:
            return flat[o:o + numel].view(shape)
        return flat[o:o + p.numel()].view(p.shape)

    def staged_ranges(self, skip_ids) -> List[Tuple[int, int]]:
        """[begin, end) element ranges of the staging arena that hold gradients, leaving out the
        parameters in ``skip_ids``; neighbours are merged (alignment gaps hold zeros)."""
        ranges: List[Tuple[int, int]] = []
        for _, p in self.named:
            o, numel, _shape = self.entries[id(p)]
            if o >= self.staged_total or id(p) in skip_ids:
                continue
            end = min(_round_up(o + numel, _ALIGN_ELEMS), self.staged_total)
            if ranges and ranges[-1][1] == o:
                ranges[-1] = (ranges[-1][0], end)
            else:
                ranges.append((o, end))
        return ranges

    def weight(self, p, padded=True):
        return self._slice(self.params, p, padded)

    def grad_staging(self, p, padded=True):
        return self._slice(self.staging, p, padded)

    def grad_acc(self, p, padded=True):
        return self._slice(self.acc, p, padded)


# ---- op constructors (host-side shape checks happen here, before anything is launched) ----------
def _p(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def op_gemm(A, B, Cm, *, a_trans=False, b_trans=False, epilogue=N.EPI_NONE, bias=None, aux_in=None,
            aux_out=None, beta=0, splitk_workspace=None) -> N.Op:
    """``splitk_workspace`` (fp32) lets the library split a long reduction (``pp_gemm_bf16_splitk``)."""
    f32 = A.dtype == torch.float32
    d = N.gemm_desc(A, B, Cm, a_trans=a_trans, b_trans=b_trans, epilogue=epilogue, bias=bias,
                    aux_in=aux_in, aux_out=aux_out, beta=beta)
    if bias is not None:
        assert bias.numel() == Cm.shape[1] and bias.dtype == A.dtype
    op = N.Op()
    op.kind = N.OP_GEMM_F32 if f32 else N.OP_GEMM_BF16
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4], op.p[5] = d.A, d.B, d.C, d.bias, d.aux_in, d.aux_out
    op.i[0], op.i[1], op.i[2], op.i[3], op.i[4], op.i[5], op.i[6] = d.M, d.N, d.K, d.lda, d.ldb, d.ldc, d.ld_aux
    op.j[0], op.j[1], op.j[2], op.j[3], op.j[4] = d.a_trans, d.b_trans, d.epilogue, d.c_dtype, d.beta
    if splitk_workspace is not None:
        assert not f32 and splitk_workspace.dtype == torch.float32 and splitk_workspace.is_contiguous()
        op.p[8], op.i[10] = splitk_workspace.data_ptr(), splitk_workspace.numel()
    return op


def splitk_copies(M: int, Nn: int, K: int) -> int:
    """How many fp32 copies of an [M, Nn] output a k-split of this problem can use (0: none): at most
    64 tiles of 256 x 256, splits of at least 4096 along K, at most 8 (the library's own rule)."""
    tiles = ((M + 255) // 256) * ((Nn + 255) // 256)
    if tiles > 64:
        return 0
    splits = min(256 // tiles, ((K + 63) // 64) // 64, 8)
    return splits if splits >= 2 else 0


def op_colsum(dY, out, ws) -> N.Op:
    M, Nn = dY.shape
    assert dY.stride(1) == 1 and out.numel() == Nn and ws.numel() >= 2 * ((M + 127) // 128) * Nn
    op = N.Op()
    op.kind = N.OP_COLSUM
    op.p[0], op.p[1], op.p[2] = dY.data_ptr(), out.data_ptr(), ws.data_ptr()
    op.i[0], op.i[1], op.i[2] = M, Nn, dY.stride(0)
    op.j[0] = N.PP_F32 if out.dtype == torch.float32 else N.PP_BF16
    return op


def op_act_bwd(dy, aux, dz, act) -> N.Op:
    assert dy.is_contiguous() and aux.is_contiguous() and dz.is_contiguous()
    assert dy.numel() == aux.numel() == dz.numel() and dy.dtype == aux.dtype == dz.dtype
    op = N.Op()
    op.kind = N.OP_ACT_BWD
    op.p[0], op.p[1], op.p[2] = dy.data_ptr(), aux.data_ptr(), dz.data_ptr()
    op.i[0] = dy.numel()
    op.j[0] = act
    op.j[1] = N.PP_F32 if dy.dtype == torch.float32 else N.PP_BF16
    return op


def op_swiglu_fwd(g, u, h) -> N.Op:
    assert g.is_contiguous() and u.is_contiguous() and h.is_contiguous()
    assert g.numel() == u.numel() == h.numel() and g.numel() % 8 == 0 and g.dtype == torch.bfloat16
    op = N.Op()
    op.kind = N.OP_SWIGLU_FWD
    op.p[0], op.p[1], op.p[2] = g.data_ptr(), u.data_ptr(), h.data_ptr()
    op.i[0] = g.numel()
    return op


def op_swiglu_bwd(g, u, dh, dg, du) -> N.Op:
    for t in (g, u, dh, dg, du):
        assert t.is_contiguous() and t.numel() == g.numel() and t.dtype == torch.bfloat16
    op = N.Op()
    op.kind = N.OP_SWIGLU_BWD
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4] = (g.data_ptr(), u.data_ptr(), dh.data_ptr(), dg.data_ptr(),
                                                   du.data_ptr())
    op.i[0] = g.numel()
    return op


def op_gemm_swiglu(x, w_gate, w_up, gu, h) -> N.Op:
    """gu [T, 2 F] = [x w_gate^T | x w_up^T] and h [T, F] = silu(gate) * up in one GEMM kernel."""
    T, K = x.shape
    Fn = w_gate.shape[0]
    assert w_gate.shape == w_up.shape == (Fn, K) and gu.shape == (T, 2 * Fn) and h.shape == (T, Fn)
    for t in (x, w_gate, w_up, gu, h):
        assert t.dtype == torch.bfloat16 and t.stride(1) == 1
    assert w_gate.stride(0) == w_up.stride(0) and Fn % 8 == 0 and K % 8 == 0
    op = N.Op()
    op.kind = N.OP_GEMM_SWIGLU
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4] = (x.data_ptr(), w_gate.data_ptr(), w_up.data_ptr(), gu.data_ptr(),
                                                   h.data_ptr())
    op.i[0], op.i[1], op.i[2] = T, Fn, K
    op.i[3], op.i[4], op.i[5], op.i[6] = x.stride(0), w_gate.stride(0), gu.stride(0), h.stride(0)
    return op


def op_gemm_dswiglu(dy, w_down_t, gu, dgu) -> N.Op:
    """dgu [T, 2 F] = [dg | du] from dh = dy w_down_t^T (not stored) and the saved gu = [g | u]."""
    T, K = dy.shape
    Fn = w_down_t.shape[0]
    assert w_down_t.shape == (Fn, K) and gu.shape == dgu.shape == (T, 2 * Fn)
    for t in (dy, w_down_t, gu, dgu):
        assert t.dtype == torch.bfloat16 and t.stride(1) == 1
    assert Fn % 8 == 0 and K % 8 == 0
    op = N.Op()
    op.kind = N.OP_GEMM_DSWIGLU
    op.p[0], op.p[1], op.p[2], op.p[3] = dy.data_ptr(), w_down_t.data_ptr(), gu.data_ptr(), dgu.data_ptr()
    op.i[0], op.i[1], op.i[2] = T, Fn, K
    op.i[3], op.i[4], op.i[5], op.i[6] = dy.stride(0), w_down_t.stride(0), gu.stride(0), dgu.stride(0)
    return op


def op_rope(x2d, cos, sin, seq, n_heads, D, inverse=False) -> N.Op:
    assert x2d.dim() == 2 and x2d.stride(1) == 1 and x2d.dtype == torch.bfloat16
    assert cos.shape == sin.shape == (seq, D // 2) and cos.dtype == sin.dtype == torch.float32
    assert n_heads * D <= x2d.stride(0) and x2d.shape[0] % seq == 0
    op = N.Op()
    op.kind = N.OP_ROPE
    op.p[0], op.p[1], op.p[2] = x2d.data_ptr(), cos.data_ptr(), sin.data_ptr()
    op.i[0], op.i[1], op.i[2], op.i[3], op.i[4] = x2d.shape[0], seq, n_heads, D, x2d.stride(0)
    op.j[0] = int(inverse)
    return op


def op_gemm_seg_swiglu(x, w_gate_list, w_up_list, seg_start, gu, h, *, ld=None) -> N.Op:
    """``op_gemm_swiglu`` over the expert segments of permuted rows: the [F, K] weights of segment e (leading
    dimension ``ld``) are entry e of the int64 device tensors ``w_gate_list`` / ``w_up_list``."""
    T, K = x.shape
    Fn = h.shape[1]
    assert gu.shape == (T, 2 * Fn) and h.shape == (T, Fn) and Fn % 8 == 0 and K % 8 == 0
    for t in (x, gu, h):
        assert t.dtype == torch.bfloat16 and t.stride(1) == 1
    assert seg_start.dtype == torch.int32 and w_gate_list.dtype == w_up_list.dtype == torch.int64
    assert w_gate_list.numel() == w_up_list.numel() == seg_start.numel() - 1
    op = N.Op()
    op.kind = N.OP_GEMM_SEG_SWIGLU
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4], op.p[5] = (x.data_ptr(), w_gate_list.data_ptr(), w_up_list.data_ptr(),
                                                            gu.data_ptr(), h.data_ptr(), seg_start.data_ptr())
    op.i[0], op.i[1], op.i[2] = T, Fn, K
    op.i[3], op.i[4], op.i[5], op.i[6] = x.stride(0), ld if ld is not None else K, gu.stride(0), h.stride(0)
    op.i[7] = w_gate_list.numel()
    return op


def op_gemm_seg_dswiglu(dy, w_down_t_list, seg_start, gu, dgu, *, ld=None) -> N.Op:
    """``op_gemm_dswiglu`` over the expert segments: the transposed down projection [F, K] of segment e is
    entry e of ``w_down_t_list``."""
    T, K = dy.shape
    Fn = gu.shape[1] // 2
    assert gu.shape == dgu.shape == (T, 2 * Fn) and Fn % 8 == 0 and K % 8 == 0
    for t in (dy, gu, dgu):
        assert t.dtype == torch.bfloat16 and t.stride(1) == 1
    assert seg_start.dtype == torch.int32 and w_down_t_list.dtype == torch.int64
    assert w_down_t_list.numel() == seg_start.numel() - 1
    op = N.Op()
    op.kind = N.OP_GEMM_SEG_DSWIGLU
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4] = (dy.data_ptr(), w_down_t_list.data_ptr(), gu.data_ptr(),
                                                   dgu.data_ptr(), seg_start.data_ptr())
    op.i[0], op.i[1], op.i[2] = T, Fn, K
    op.i[3], op.i[4], op.i[5], op.i[6] = dy.stride(0), ld if ld is not None else K, gu.stride(0), dgu.stride(0)
    op.i[7] = w_down_t_list.numel()
    return op


def op_gemm_seg(mode, A, ptr_list, seg_start, *, Cm=None, other=None, n_cols=None, ld=None,
                epilogue=N.EPI_NONE, aux_in=None, beta=0, c_f32=False) -> N.Op:
    """Segmented GEMM over the expert segments of permuted rows (sizes read on the device).
    rows mode: Cm[r0:r1] = A[r0:r1] B_e^T (+ aux_in), B_e [n_cols = Cm.shape[1], K] with leading
    dimension ``ld`` from ``ptr_list``.  k mode: C_e = A[r0:r1]^T other[r0:r1], C_e [A.shape[1],
    other.shape[1]] with leading dimension ``ld`` from ``ptr_list``."""
    assert seg_start.dtype == torch.int32 and ptr_list.dtype == torch.int64
    assert ptr_list.numel() == seg_start.numel() - 1
    op = N.Op()
    op.kind = N.OP_GEMM_SEG
    if mode == N.SEG_ROWS:
        assert A.stride(1) == 1 and Cm.stride(1) == 1 and A.shape[0] == Cm.shape[0]
        assert A.dtype == torch.bfloat16 and Cm.dtype == torch.bfloat16
        op.p[0], op.p[1], op.p[2] = A.data_ptr(), None, Cm.data_ptr()
        op.i[0], op.i[1], op.i[2] = A.shape[0], Cm.shape[1], A.shape[1]
        op.i[3], op.i[4], op.i[5] = A.stride(0), ld if ld is not None else A.shape[1], Cm.stride(0)
        if aux_in is not None:
            assert aux_in.shape == Cm.shape and aux_in.stride(1) == 1
            op.p[4], op.i[6] = aux_in.data_ptr(), aux_in.stride(0)
        op.j[0], op.j[1], op.j[3] = 0, 0, N.PP_BF16
    else:
        assert A.stride(1) == 1 and other.stride(1) == 1 and A.shape[0] == other.shape[0]
        op.p[0], op.p[1], op.p[2] = A.data_ptr(), other.data_ptr(), None
        op.i[0], op.i[1], op.i[2] = A.shape[1], other.shape[1], A.shape[0]
        op.i[3], op.i[4], op.i[5] = A.stride(0), other.stride(0), ld if ld is not None else other.shape[1]
        op.j[0], op.j[1], op.j[3] = 1, 1, N.PP_F32 if c_f32 else N.PP_BF16
    op.j[2], op.j[4], op.j[5] = epilogue, beta, mode
    op.p[6], op.p[7] = seg_start.data_ptr(), ptr_list.data_ptr()
    op.i[7] = ptr_list.numel()
    return op


def op_moe_router(logits, topk_idx, gate, E=None) -> N.Op:
    """``E``: number of experts when ``logits`` carries padding columns after them."""
    T = logits.shape[0]
    E = logits.shape[1] if E is None else E
    assert logits.dtype == torch.bfloat16 and logits.stride(1) == 1 and E <= logits.shape[1]
    assert topk_idx.dtype == torch.int32 and topk_idx.numel() == 2 * T and topk_idx.is_contiguous()
    assert gate.dtype == torch.float32 and gate.numel() == 2 * T and gate.is_contiguous()
    op = N.Op()
    op.kind = N.OP_MOE_ROUTER
    op.p[0], op.p[1], op.p[2] = logits.data_ptr(), topk_idx.data_ptr(), gate.data_ptr()
    op.i[0], op.i[1], op.i[2] = logits.stride(0), T, E
    return op


def op_moe_permute(expert_of_slot, E, seg_start, row_src, pos) -> N.Op:
    n = expert_of_slot.numel()
    for t in (expert_of_slot, seg_start, row_src, pos):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert seg_start.numel() == E + 1 and row_src.numel() == n and pos.numel() == n
    op = N.Op()
    op.kind = N.OP_MOE_PERMUTE
    op.p[0], op.p[1], op.p[2], op.p[3] = (expert_of_slot.data_ptr(), seg_start.data_ptr(), row_src.data_ptr(),
                                          pos.data_ptr())
    op.i[0], op.i[1] = n, E
    return op


def op_moe_gather(src, row_src, topk, dst, scale=None, n_rows=None) -> N.Op:
    assert src.stride(1) == 1 and dst.stride(1) == 1 and src.shape[1] == dst.shape[1]
    assert row_src.dtype == torch.int32 and row_src.numel() == dst.shape[0]
    assert scale is None or (scale.dtype == torch.float32 and scale.is_contiguous())
    op = N.Op()
    op.kind = N.OP_MOE_GATHER
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4] = src.data_ptr(), row_src.data_ptr(), _p(n_rows), _p(scale), dst.data_ptr()
    op.i[0], op.i[1], op.i[2], op.i[3], op.i[4] = src.stride(0), topk, dst.stride(0), dst.shape[0], dst.shape[1]
    return op


def op_moe_combine(y, pos, topk, out, gate=None, resid=None) -> N.Op:
    T, Cc = out.shape
    assert y.stride(1) == 1 and out.stride(1) == 1 and y.shape[1] == Cc
    assert pos.dtype == torch.int32 and pos.numel() == T * topk
    assert gate is None or (gate.dtype == torch.float32 and gate.numel() == T * topk and gate.is_contiguous())
    assert resid is None or (resid.shape == out.shape and resid.stride(1) == 1)
    op = N.Op()
    op.kind = N.OP_MOE_COMBINE
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4] = y.data_ptr(), pos.data_ptr(), _p(gate), _p(resid), out.data_ptr()
    op.i[0], op.i[1], op.i[2], op.i[3], op.i[4], op.i[5] = (y.stride(0), topk, resid.stride(0) if resid is not None else 0,
                                                          out.stride(0), T, Cc)
    return op


def op_moe_gate_bwd(dout, y, pos, topk_idx, gate, E, dlogits) -> N.Op:
    T, Cc = dout.shape
    topk = pos.numel() // T
    assert dlogits.shape == (T, (E + 7) // 8 * 8) and dlogits.dtype == torch.bfloat16 and dlogits.stride(1) == 1
    assert dout.stride(1) == 1 and y.stride(1) == 1 and y.shape[1] == Cc
    op = N.Op()
    op.kind = N.OP_MOE_GATE_BWD
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4], op.p[5] = (dout.data_ptr(), y.data_ptr(), pos.data_ptr(),
                                                          topk_idx.data_ptr(), gate.data_ptr(), dlogits.data_ptr())
    op.i[0], op.i[1], op.i[2], op.i[3], op.i[4], op.i[5], op.i[6] = (dout.stride(0), y.stride(0), topk, E,
                                                                     dlogits.stride(0), T, Cc)
    return op


def op_ln_fwd(x, gamma, beta, y, mean, rstd, eps) -> N.Op:
    rows, Cc = x.shape
    assert x.is_contiguous() and y.is_contiguous() and y.shape == x.shape
    assert gamma.numel() == Cc and rstd.numel() == rows and (mean is None or mean.numel() == rows)
    assert mean is not None or beta is None, "RMSNorm (mean=None) has no beta"
    op = N.Op()
    op.kind = N.OP_LN_FWD
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4], op.p[5] = (x.data_ptr(), gamma.data_ptr(), _p(beta),
                                                            y.data_ptr(), _p(mean), rstd.data_ptr())
    op.i[0], op.i[1] = rows, Cc
    op.f[0] = eps
    return op


def op_ln_bwd_input(dy, x, gamma, mean, rstd, dres, dx) -> N.Op:
    rows, Cc = x.shape
    for t in (dy, x, dx) + ((dres,) if dres is not None else ()):
        assert t.is_contiguous() and t.shape == x.shape
    op = N.Op()
    op.kind = N.OP_LN_BWD_INPUT
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4], op.p[5], op.p[6] = (
        dy.data_ptr(), x.data_ptr(), gamma.data_ptr(), _p(mean), rstd.data_ptr(), _p(dres),
        dx.data_ptr())
    op.i[0], op.i[1] = rows, Cc
    return op


def op_ln_bwd_weight(dy, x, mean, rstd, dgamma, dbeta, ws) -> N.Op:
    rows, Cc = x.shape
    assert dy.is_contiguous() and x.is_contiguous() and dy.shape == x.shape
    assert dgamma.numel() == Cc and ws.numel() >= 2 * ((rows + 127) // 128) * Cc
    op = N.Op()
    op.kind = N.OP_LN_BWD_WEIGHT
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4], op.p[5], op.p[6] = (
        dy.data_ptr(), x.data_ptr(), _p(mean), rstd.data_ptr(), dgamma.data_ptr(), _p(dbeta),
        ws.data_ptr())
    op.i[0], op.i[1] = rows, Cc
    op.j[0] = N.PP_F32 if dgamma.dtype == torch.float32 else N.PP_BF16
    return op


def op_attn(kind, qkv, o, lse, H, causal, d_o=None, dqkv=None, delta=None, n_kv_heads=None, kv_len=None,
            scale=None, exact_dq=False) -> N.Op:
    """``scale``: the factor on the scores (None: 1 / sqrt(head size)); ``exact_dq``: see ``N.attn_desc``."""
    if qkv.shape[1] % 64:
        raise RuntimeError(f"the attention kernels take sequence lengths that are multiples of 64, got "
                           f"{qkv.shape[1]} (stage_modules.lower_attention pads)")
    d = N.attn_desc(qkv, o, lse, H, causal, scale, d_o=d_o, dqkv=dqkv, delta=delta, n_kv_heads=n_kv_heads,
                    kv_len=kv_len, exact_dq=exact_dq)
    op = N.Op()
    op.kind = kind
    for k, v in enumerate((d.q, d.k, d.v, d.o, d.lse, d.d_o, d.dq, d.dk, d.dv, d.delta)):
        op.p[k] = v
    op.i[0], op.i[1], op.i[2], op.i[3], op.i[4], op.i[5] = d.B, d.S, d.H, d.D, d.stride_b, d.stride_s
    op.f[0] = d.scale
    op.j[0] = d.causal
    op.j[1] = d.kv_group
    op.j[2] = d.kv_len
    op.j[3] = d.flags
    return op


def op_embed_fwd(ids, wte, wpe, y, seq, extra_row=None, pos_ids=None) -> N.Op:
    """``pos_ids`` (int64, one per token): the row of ``wpe`` each token reads, instead of its index in
    the sequence."""
    vocab, Cc = wte.shape
    assert ids.dtype == torch.int64 and y.shape == (ids.numel(), Cc) and y.is_contiguous()
    assert extra_row is None or (extra_row.numel() == Cc and extra_row.is_contiguous())
    op = N.Op()
    op.kind = N.OP_EMBED_FWD
    op.p[0], op.p[1], op.p[2], op.p[3] = ids.data_ptr(), wte.data_ptr(), _p(wpe), y.data_ptr()
    op.p[4] = _p(extra_row)
    op.i[0], op.i[1], op.i[2], op.i[3] = ids.numel(), seq, Cc, vocab
    if pos_ids is not None:
        assert wpe is not None and pos_ids.dtype == torch.int64 and pos_ids.numel() == ids.numel() \
            and pos_ids.is_contiguous()
        op.p[5] = pos_ids.data_ptr()
        op.i[4] = wpe.shape[0]
    return op


def op_position_ids(ids, out, pad: int) -> N.Op:
    assert ids.dtype == out.dtype == torch.int64 and ids.dim() == 2 and out.shape == ids.shape
    assert ids.is_contiguous() and out.is_contiguous()
    op = N.Op()
    op.kind = N.OP_POSITION_IDS
    op.p[0], op.p[1] = ids.data_ptr(), out.data_ptr()
    op.i[0], op.i[1], op.i[2] = ids.shape[0], ids.shape[1], pad
    return op


def op_embed_bwd(ids, dy, d_wte, d_wpe, seq, round_bf16=False, padding_idx=None) -> N.Op:
    """``round_bf16``: the per-microbatch row sums are rounded to bf16 before they are added (the bits
    of a bf16 gradient tensor folded into the fp32 accumulator).  ``padding_idx``: the row of ``d_wte``
    that gets no gradient, as ``nn.Embedding(padding_idx=...)`` has it."""
    vocab, Cc = d_wte.shape
    assert d_wte.dtype == torch.float32 and dy.shape == (ids.numel(), Cc) and dy.is_contiguous()
    op = N.Op()
    op.kind = N.OP_EMBED_BWD
    op.p[0], op.p[1], op.p[2], op.p[3] = ids.data_ptr(), dy.data_ptr(), d_wte.data_ptr(), _p(d_wpe)
    op.i[0], op.i[1], op.i[2], op.i[3] = ids.numel(), seq, Cc, vocab
    op.i[4] = 0 if padding_idx is None else padding_idx % vocab + 1
    op.j[0] = int(round_bf16)
    return op


def op_ce_loss(logits, target, loss, dlogits, ws, V, ignore_index) -> N.Op:
    rows = logits.shape[0]
    assert logits.stride(1) == 1 and ws.numel() >= rows + 2 and target.numel() == rows
    if dlogits is not None:
        assert dlogits.stride() == logits.stride() and dlogits.shape[0] == rows
    op = N.Op()
    op.kind = N.OP_CE_LOSS
    op.p[0], op.p[1], op.p[2], op.p[3], op.p[4] = (logits.data_ptr(), target.data_ptr(),
                                                   loss.data_ptr(), _p(dlogits), ws.data_ptr())
    op.i[0], op.i[1], op.i[2], op.i[3] = rows, V, logits.stride(0), ignore_index
    op.j[0] = N.PP_F32 if logits.dtype == torch.float32 else N.PP_BF16
    return op


def op_accum(acc, g, init=False) -> N.Op:
    assert acc.dtype == torch.float32 and acc.numel() == g.numel()
    op = N.Op()
    op.kind = N.OP_ACCUM_F32 if g.dtype == torch.float32 else N.OP_ACCUM_BF16
    op.p[0], op.p[1] = acc.data_ptr(), g.data_ptr()
    op.i[0] = acc.numel()
    op.j[0] = int(init)
    return op


def op_copy_rows(src, dst, n_rows, row_bytes, src_stride, dst_stride) -> N.Op:
    """``n_rows`` runs of ``row_bytes`` bytes from ``src`` to ``dst`` with byte strides between runs."""
    def room(t):    # bytes from the tensor's first element to the end of its storage (t may be a strided view)
        return t.untyped_storage().nbytes() - t.storage_offset() * t.element_size()
    assert src_stride >= row_bytes and dst_stride >= row_bytes
    assert (n_rows - 1) * src_stride + row_bytes <= room(src), "op_copy_rows: reads past the source"
    assert (n_rows - 1) * dst_stride + row_bytes <= room(dst), "op_copy_rows: writes past the destination"
    op = N.Op()
    op.kind = N.OP_COPY_ROWS
    op.p[0], op.p[1] = src.data_ptr(), dst.data_ptr()
    op.i[0], op.i[1], op.i[2], op.i[3] = n_rows, row_bytes, src_stride, dst_stride
    return op


def op_fill(t, value=0) -> N.Op:
    assert t.is_contiguous()
    op = N.Op()
    op.kind = N.OP_FILL
    op.p[0] = t.data_ptr()
    op.i[0] = t.numel() * t.element_size()
    op.j[0] = value
    return op


OP_SKIP = N.OP_SKIP  # pp_op.flags bit: the runner steps over the op


class OpList:
    """A growable list of descriptors, frozen into one ctypes array before its first replay."""

    def __init__(self):
        self.ops: List[N.Op] = []
        self._arr = None

    def append(self, op: N.Op) -> int:
        assert self._arr is None, "list is frozen"
        self.ops.append(op)
        return len(self.ops) - 1

    def freeze(self):
        n = len(self.ops)
        arr = (N.Op * max(n, 1))()
        for k, op in enumerate(self.ops):
            C.memmove(C.byref(arr, k * C.sizeof(N.Op)), C.byref(op), C.sizeof(N.Op))
        self._arr = arr
        self.n = n

    def run(self):
        if self._arr is None:
            self.freeze()
        if self.n:
            N.run_ops(self._arr, self.n)

    def __getitem__(self, k) -> N.Op:
        if self._arr is None:
            self.freeze()
        return self._arr[k]

    def find_pointer(self, ptr: int) -> List[Tuple[int, int]]:
        if self._arr is None:
            self.freeze()
        hits = []
        for k in range(self.n):
            for q in range(12):
                if self._arr[k].p[q] == ptr:
                    hits.append((k, q))
        return hits


class MicrobatchProgram:
    """Launch lists and buffers of one (stage, microbatch slot)."""

    def __init__(self):
        self.F = OpList()
        self.I = OpList()
        self.W = OpList()
        self.acts: Dict[str, torch.Tensor] = {}
        self.input_slot: Optional[torch.Tensor] = None
        self.output: Optional[torch.Tensor] = None       # what the next stage (or the user) sees
        self.output_grad: Optional[torch.Tensor] = None  # gradient of `output`, same layout
        self.input_grad: Optional[torch.Tensor] = None
        self.in_key = None
        self.input_patches: List[Tuple[OpList, int, int]] = []
        self.init_toggle_fill: List[int] = []   # W ops that run only on the first accumulation
        self.init_toggle_accum: List[int] = []  # W ops whose init flag follows the stage state
        self.init_toggle_beta: List[int] = []   # W GEMMs that accumulate in their epilogue
        self.loss_ops: Dict[int, Tuple[OpList, torch.Tensor, torch.Tensor]] = {}
        self.w_tags: List[Optional[str]] = []   # per W op: how it follows the accumulation state


class Builder:
    """Handed to ``block.lower``: allocates buffers and records ops for one microbatch slot."""

    def __init__(self, stage_prog: "StageProgram", mb: int, prog: MicrobatchProgram):
        self.sp = stage_prog
        self.mb = mb
        self.prog = prog
        self.training = stage_prog.training
        self.fused_accumulate = stage_prog.fused_accumulate
        self._scope: List[str] = []
        self._backward: List[Callable] = []
        self._w_gemm: List[Tuple[N.Op, Optional[str]]] = []
        self._w_reduce: List[Tuple[N.Op, Optional[str]]] = []
        self._w_other: List[Tuple[N.Op, Optional[str]]] = []
        self.device = stage_prog.device

    # -- naming
    def scope(self, name: str):
        b = self

        class _S:
            def __enter__(self_inner):
                b._scope.append(name)

            def __exit__(self_inner, *exc):
                b._scope.pop()
        return _S()

    def _key(self, name: str) -> str:
        return ".".join(self._scope + [name])

    # -- buffers
    def act(self, name, shape, dtype=None) -> torch.Tensor:
        """Per-microbatch buffer that lives from forward until the matching backward."""
        t = torch.empty(tuple(shape), dtype=dtype or self.sp.act_dtype, device=self.device)
        self.prog.acts[self._key(name)] = t
        return t

    def grad(self, name, shape, dtype=None) -> torch.Tensor:
        """Gradient buffer written in the I pass and read in the W pass.  Shared by all
        microbatches of the stage when I and W run back to back; per microbatch when the schedule
        may defer W (zero-bubble)."""
        if self.sp.split_backward:
            return self.act("grad:" + name, shape, dtype)
        return self.sp.shared(self._key("grad:" + name), shape, dtype or self.sp.act_dtype)

    def workspace(self, name, shape, dtype) -> torch.Tensor:
        """Stage-shared workspace with a name of its own (for ops that run concurrently with
        others in a grouped launch and therefore cannot share scratch)."""
        return self.sp.shared("ws:" + name, shape, dtype)

    def w_reduce(self, op):
        """Queues a column reduction of the weight-gradient pass; all of them run grouped, after
        the grouped dW GEMMs."""
        op.flags |= N.OP_GROUPED
        self._w_reduce.append((op, None))

    def scratch(self, name, shape, dtype) -> torch.Tensor:
        """Workspace valid inside one kernel sequence (never carried across passes)."""
        return self.sp.shared("scratch:" + name, shape, dtype, exact=False)

    # -- parameters
    def weight(self, p, padded=True):
        return self.sp.arena.weight(p, padded)

    def weight_t(self, p):
        return self.sp.arena.weight_t(p)

    def weight_t_cat(self, *ps):
        return self.sp.arena.weight_t_cat(*ps)

    def rows_cat(self, *ps):
        return self.sp.arena.rows_cat(*ps)

    def grad_target(self, p, padded=True):
        """Where the W pass writes a microbatch gradient that no GEMM epilogue accumulates: the
        staging arena, which the accumulate ops at the end of the pass fold into fp32."""
        return self.sp.arena.grad_staging(p, padded)

    def grad_acc(self, p, padded=True):
        return self.sp.arena.grad_acc(p, padded)

    # -- ops
    def f(self, op):
        return self.prog.F.append(op)

    def i(self, op):
        return self.prog.I.append(op)

    def w(self, op, tag: Optional[str] = None):
        """Queues an op of the weight-gradient pass.  ``tag`` names how the op follows the
        accumulation state: "accum" (its init flag), "beta" (GEMM epilogue accumulate), "fill"
        (runs only when an accumulation starts)."""
        self._w_other.append((op, tag))

    def w_weight_gemm(self, dY2d, X2d, p, padded=True):
        """dW[out, in] = dY^T X for a linear weight ``p``: bf16/fp32 into staging, or fused fp32
        accumulation."""
        # all dW GEMMs of a pass only read buffers that the input-gradient pass has finished, so
        # they are independent of each other: they go first and are marked for grouped launch
        epi = self.weight_grad_epilogue(p)
        if epi is not None:
            op = op_gemm(dY2d, X2d, self.grad_acc(p, padded), a_trans=True, b_trans=True, epilogue=epi, beta=1)
            op.flags |= N.OP_GROUPED
            self._w_gemm.append((op, "beta"))
        else:
            op = op_gemm(dY2d, X2d, self.grad_target(p, padded), a_trans=True, b_trans=True)
            op.flags |= N.OP_GROUPED
            self._w_gemm.append((op, None))

    def weight_grad_epilogue(self, p) -> Optional[int]:
        """The GEMM epilogue that adds the gradient of weight ``p`` to its fp32 accumulator, or None
        when the gradient goes through the staging arena.  ``fused_accumulate`` adds the fp32 sums;
        the default adds them rounded to the parameter dtype, which leaves bit for bit what a
        gradient written in that dtype and folded in by the accumulate kernel would."""
        if self.sp.staged_weight_grads:
            return None
        self.sp.epilogue_accumulated.add(id(p))
        if self.fused_accumulate or p.dtype == torch.float32:
            return N.EPI_ACCUM_F32
        return N.EPI_ACCUM_ROUNDED

    def on_backward(self, fn: Callable):
        """Registers the block's backward emitter ``fn(dy, need_dx, dx_out) -> dx``; it runs later,
        in reverse block order, under the naming scope that is current now."""
        scope = list(self._scope)

        def scoped(dy, need_dx, dx_out):
            saved, self._scope = self._scope, list(scope)
            try:
                return fn(dy, need_dx, dx_out)
            finally:
                self._scope = saved

        self._backward.append(scoped)


# Pointer fields that an op of the input-gradient pass writes, by kind (kinds that are absent write through
# fields that never hold a gradient tensor which a column reduction reads).
_WRITTEN_FIELDS = {
    N.OP_GEMM_BF16: (2, 5), N.OP_GEMM_F32: (2, 5), N.OP_GEMM_SEG: (2, 5), N.OP_LN_BWD_INPUT: (6,),
    N.OP_ATTN_BWD: (6, 7, 8, 9), N.OP_ACT_BWD: (2,), N.OP_SWIGLU_BWD: (3, 4), N.OP_ROPE: (0,),
    N.OP_COPY_ROWS: (1,), N.OP_FILL: (0,), N.OP_ACCUM_BF16: (0,), N.OP_ACCUM_F32: (0,),
    N.OP_MOE_GATHER: (4,), N.OP_MOE_COMBINE: (4,), N.OP_MOE_GATE_BWD: (5,), N.OP_GEMM_DSWIGLU: (3,),
    N.OP_GEMM_SEG_DSWIGLU: (3,),
    N.OP_EMBED_BWD: (2, 3), N.OP_CE_LOSS: (2, 3),
}


def _fuse_column_sums(b: "Builder", prog: MicrobatchProgram) -> None:
    """Lets the kernels of the I pass that produce a gradient tensor leave the partial column sums that the W
    pass needs of it, so that its column reductions do not read the tensor from memory a second time:

    * the dgamma / dbeta reduction of a LayerNorm takes them from that LayerNorm's own input-gradient op;
    * a bias-gradient column sum over a tensor that a LayerNorm input-gradient op wrote as its ``dx`` (the
      gradient of the residual stream, which is the output gradient of the linear layer in front of the
      norm) takes the sums of ``dx`` from that op;
    * a bias-gradient column sum over the output of a GEMM with an activation-derivative epilogue (the
      gradient in front of a GELU or ReLU) takes them from that GEMM's epilogue;
    * the bias gradient of a fused q | k | v projection takes them from the attention backward kernels (head
      size 64), which write that projection's output gradient.

    Only exact matches are rewired: same pointers, same shape, and no other op of the I pass writing anywhere
    into the tensor."""
    if os.environ.get("PIPPY_AMD_TWO_PASS_COLUMN_SUMS") == "1":  # for A / B measurements of this rewiring
        return
    I = prog.I.ops
    ln_ops = [op for op in I if op.kind == N.OP_LN_BWD_INPUT and 0 < op.i[1] <= N.LN_SUM_MAX_C]
    act_ops = [op for op in I if op.kind == N.OP_GEMM_BF16 and op.j[3] == N.PP_BF16 and not op.p[8]
               and op.j[2] in (N.EPI_DGELU_ERF, N.EPI_DGELU_TANH, N.EPI_DRELU)]
    attn_ops = [op for op in I if op.kind == N.OP_ATTN_BWD and op.i[3] == 64 and not op.p[10]]
    if not ln_ops and not act_ops and not attn_ops:
        return
    writes = [(op.p[q], op) for op in I for q in _WRITTEN_FIELDS.get(op.kind, range(12)) if op.p[q]]

    def only_writer(src, lo: int, n_bytes: int) -> bool:
        """No op of the pass other than ``src`` writes through a pointer into [lo, lo + n_bytes): the tensor
        that the reduction reads is what ``src`` left there (an in-place rotary embedding or a row copy into
        a part of it, which start inside the range, rule the rewiring out)."""
        return not any(lo <= ptr < lo + n_bytes and op is not src for ptr, op in writes)

    for k, (op, _tag) in enumerate(b._w_reduce):
        if op.j[1]:
            continue
        if op.kind == N.OP_LN_BWD_WEIGHT:
            src = [l for l in ln_ops if l.p[0] == op.p[0] and l.p[1] == op.p[1] and l.i[0] == op.i[0]
                   and l.i[1] == op.i[1] and not l.p[7]]
            if len(src) != 1:
                continue
            rows, Cc = op.i[0], op.i[1]
            n_part = (rows + N.LN_SUM_ROWS - 1) // N.LN_SUM_ROWS
            ws = b.grad(f"colsums.{k}", (2 * n_part * Cc,), torch.float32)
            src[0].p[7] = ws.data_ptr()
            op.p[6], op.j[1] = ws.data_ptr(), n_part
        elif op.kind == N.OP_COLSUM:
            rows, Cc, ld = op.i[0], op.i[1], op.i[2]
            n_bytes = 2 * ((rows - 1) * ld + Cc) if rows else 0
            src = [l for l in ln_ops if l.p[6] == op.p[0] and l.i[0] == rows and l.i[1] == Cc and not l.p[8]]
            if len(src) == 1 and ld == Cc and only_writer(src[0], op.p[0], n_bytes):
                n_part = (rows + N.LN_SUM_ROWS - 1) // N.LN_SUM_ROWS
                ws = b.grad(f"colsums.{k}", (n_part * Cc,), torch.float32)
                src[0].p[8] = ws.data_ptr()
                op.p[2], op.j[1] = ws.data_ptr(), n_part
                continue
            # the input gradient of an activation, written by the epilogue of the GEMM in front of it
            src = [g for g in act_ops if g.p[2] == op.p[0] and g.i[0] == rows and g.i[1] == Cc and g.i[5] == ld
                   and not g.p[9]]
            if len(src) == 1 and only_writer(src[0], op.p[0], n_bytes):
                n_part = (rows + N.GEMM_COLSUM_ROWS - 1) // N.GEMM_COLSUM_ROWS
                ws = b.grad(f"colsums.{k}", (n_part * Cc,), torch.float32)
                src[0].p[9] = ws.data_ptr()
                op.p[2], op.j[1] = ws.data_ptr(), n_part
                continue
            # the gradient of a fused q | k | v projection, written by the attention backward: dq at the head
            # of every row, dk and dv behind it, the rows of all sequences back to back
            def fused(a):
                Bn, S, H, D, sb, ss = (a.i[q] for q in range(6))
                Hkv = H // max(a.j[1], 1)
                return (a.p[6] == op.p[0] and a.p[7] == a.p[6] + 2 * H * D and a.p[8] == a.p[7] + 2 * Hkv * D
                        and Cc == (H + 2 * Hkv) * D and ss == ld and sb == S * ss and rows == Bn * S)
            src = [a for a in attn_ops if fused(a)]
            if len(src) == 1 and only_writer(src[0], op.p[0], n_bytes):
                n_part = rows // 64
                ws = b.grad(f"colsums.{k}", (n_part * Cc,), torch.float32)
                src[0].p[10], src[0].i[6] = ws.data_ptr(), Cc
                op.p[2], op.j[1] = ws.data_ptr(), n_part


class StageProgram:
    """All microbatch programs of one stage plus its arenas and shared buffers."""

    def __init__(self, blocks: Sequence[nn.Module], module: nn.Module, device, training: bool,
                 split_backward: bool, fused_accumulate: bool, is_first: bool, is_last: bool):
        self.blocks = list(blocks)
        self.device = device
        self.training = training
        self.split_backward = split_backward
        # fused_accumulate: False - weight-gradient GEMMs add their sums, rounded to the parameter
        # dtype, to the fp32 accumulators (the same bits as the staged form); True - they add the
        # unrounded fp32 sums; "staged" - every gradient is written to the staging arena in the
        # parameter dtype and folded in by the accumulate kernel (the literal form of the contract)
        if isinstance(fused_accumulate, str) and fused_accumulate != "staged":
            raise ValueError(f"fused_accumulate must be False, True or 'staged', not {fused_accumulate!r}")
        self.staged_weight_grads = fused_accumulate == "staged"
        self.fused_accumulate = bool(fused_accumulate) and not self.staged_weight_grads
        self.epilogue_accumulated = set()  # ids of the parameters whose GEMM epilogue accumulates
        self.is_first = is_first
        self.is_last = is_last
        self.arena = ParamArena(module, device, self.blocks)
        self.act_dtype = self.arena.dtype
        self._shared: Dict[str, torch.Tensor] = {}
        self.zeroed_once = set()   # addresses of shared buffers whose padding a block cleared when it was built
        self.mbs: Dict[int, MicrobatchProgram] = {}
        self._batched_w: Dict[Tuple[int, ...], "BatchedW"] = {}
        self.acc_initialized = False  # False: the next W pass overwrites the accumulators
        # True once ``materialize_grads`` has set ``param.grad`` from the accumulators: a ``.grad`` that
        # is None afterwards was cleared by the user's optimizer
        self.grads_handed_over = False

    def shared(self, key, shape, dtype, exact=True) -> torch.Tensor:
        # Launch lists hold raw pointers into these buffers, so a buffer is never replaced or
        # freed once handed out: the size is part of the key.
        shape = tuple(shape)
        numel = 1
        for s in shape:
            numel *= s
        full_key = (key, numel, dtype)
        t = self._shared.get(full_key)
        if t is None:
            t = torch.empty(max(numel, 1), dtype=dtype, device=self.device)
            self._shared[full_key] = t
        return t[:numel].view(shape)

    def ones_f32(self, n: int) -> torch.Tensor:
        """A [1, n] row of ones (the left operand that turns an fp32 GEMM into a column sum)."""
        t = self._shared.get(("ones_f32", n))
        if t is None:
            t = torch.ones(max(n, 1), dtype=torch.float32, device=self.device)
            self._shared[("ones_f32", n)] = t
        return t.view(1, n)

    def build(self, mb: int, x: torch.Tensor, dx_target: Optional[torch.Tensor]) -> MicrobatchProgram:
        """Lowers every block for microbatch slot ``mb`` with input ``x`` (a real buffer: the
        previous stage's output slot, or this stage's own input slot on the first stage).
        ``dx_target`` is the buffer the gradient w.r.t. ``x`` must be written to (the previous
        stage's output-gradient slot) or None when nobody consumes it."""
        prog = MicrobatchProgram()
        b = Builder(self, mb, prog)
        prog.in_key = (tuple(x.shape), x.dtype, x.data_ptr(), _p(dx_target))
        prog.input_slot = x
        h = x
        for k, blk in enumerate(self.blocks):
            with b.scope(f"{k}"):
                h = blk.lower(b, h)
        prog.output = h
        if self.training:
            # gradient of the output, in the (possibly padded) layout of the buffer behind it;
            # zero-filled once so that padding columns stay zero for every later use
            out_buf = getattr(h, "_pp_padded", None)
            if out_buf is None:
                gbuf = torch.zeros(h.shape, dtype=h.dtype, device=self.device)
                prog.output_grad = gbuf
            else:
                gbuf = torch.zeros(out_buf.shape, dtype=out_buf.dtype, device=self.device)
                prog.output_grad = _like_view(gbuf, h, out_buf)
            prog.output_grad_buf = gbuf
            dy = gbuf
            fns = b._backward
            assert len(fns) == len(self.blocks), "every block registers exactly one backward emitter"
            for idx in reversed(range(len(fns))):
                first = idx == 0
                need_dx = (not first) or (dx_target is not None)
                dy = fns[idx](dy, need_dx, dx_target if first else None)
            if dx_target is not None:
                assert dy is not None and dy.data_ptr() == dx_target.data_ptr()
            prog.input_grad = dy
            _fuse_column_sums(b, prog)
            toggles = {"accum": prog.init_toggle_accum, "beta": prog.init_toggle_beta,
                       "fill": prog.init_toggle_fill}
            for op, tag in b._w_gemm + b._w_reduce + b._w_other:
                k = prog.W.append(op)
                prog.w_tags.append(tag)
                if tag is not None:
                    toggles[tag].append(k)
            # fold this microbatch's staged parameter gradients into the fp32 accumulators
            # (those that no GEMM epilogue has added already)
            for lo, hi in self.arena.staged_ranges(self.epilogue_accumulated):
                k = prog.W.append(op_accum(self.arena.acc[lo:hi], self.arena.staging[lo:hi], init=False))
                prog.w_tags.append("accum")
                prog.init_toggle_accum.append(k)
        prog.F.freeze()
        prog.I.freeze()
        prog.W.freeze()
        self.mbs[mb] = prog
        return prog

    def batched_w(self, mbs: Tuple[int, ...]) -> "BatchedW":
        """The weight-gradient passes of the microbatches ``mbs`` (ascending) as ONE launch list in which
        every weight-gradient GEMM runs once over all of them (see ``BatchedW``)."""
        key = tuple(mbs)
        got = self._batched_w.get(key)
        if got is None or any(self.mbs[m] is not p for m, p in zip(key, got.progs)):
            got = self._batched_w[key] = BatchedW(self, key)
        return got

    def set_accumulate_mode(self, prog: MicrobatchProgram, init: bool) -> None:
        """Patches the W list for the first (init) or a later microbatch of an accumulation."""
        for k in prog.init_toggle_accum:
            prog.W[k].j[0] = int(init)
        for k in prog.init_toggle_beta:
            prog.W[k].j[4] = 0 if init else 1
        for k in prog.init_toggle_fill:
            if init:
                prog.W[k].flags &= ~OP_SKIP
            else:
                prog.W[k].flags |= OP_SKIP


class BatchedW:
    """The weight-gradient passes of several microbatches of a stage as one launch list.

    The reference accumulates parameter gradients microbatch by microbatch (one autograd pass each,
    ``pippy/_backward.py:67-69``, in backward-microbatch order, ``pippy/PipelineSchedule.py:327,401-438``).
    With every microbatch's operands still resident, a weight-gradient GEMM can instead run ONCE over all of
    them: a tile walks the microbatches in ascending order, rounds each microbatch's product as the
    single-microbatch kernel would, and adds it to a running fp32 sum in registers - the same additions in
    the same order, so the accumulators end up bit-identical, but they are read and written once instead of
    once per microbatch (``pp_gemm_bf16_grouped_kseg``; ``pp_gemm_bf16_segmented_kseg`` for the expert
    weights of a mixture-of-experts layer, whose accumulators outweigh a microbatch's operands by far).
    Everything else of the passes (column reductions, embedding gradients, the accumulate op over the small
    tensors) follows per microbatch, in order."""

    def __init__(self, sp: "StageProgram", mbs: Tuple[int, ...]):
        self.progs = [sp.mbs[m] for m in mbs]
        first = self.progs[0]
        n_ops = first.W.n if first.W._arr is not None else len(first.W.ops)
        for p in self.progs:
            assert (p.W.n if p.W._arr is not None else len(p.W.ops)) == n_ops and p.w_tags == first.w_tags
        dev = sp.device
        self.list = OpList()
        self.beta_ops: List[int] = []                     # batched GEMMs: beta follows the accumulation state
        self.rest: List[Tuple[int, int, str]] = []        # (index, position of its microbatch, tag) of the others
        batched = set()
        dense, seg = [], []
        for k in range(n_ops):
            op = first.W[k]
            accumulating = op.j[2] in (N.EPI_ACCUM_F32, N.EPI_ACCUM_ROUNDED) and op.j[3] == N.PP_F32
            if op.kind == N.OP_GEMM_BF16 and op.j[0] and op.j[1] and accumulating and first.w_tags[k] == "beta" \
                    and not op.p[8]:
                dense.append(k)
            elif op.kind == N.OP_GEMM_SEG and op.j[5] == N.SEG_K and accumulating and first.w_tags[k] == "beta":
                seg.append(k)
        n_mb = len(self.progs)
        # where the copies of this list hold a pointer that a forward pass re-points at the stage's current
        # input (a first stage reads the caller's tensors): (position of the microbatch, op, pointer slot)
        patched = [(pos, k, q) for pos, p in enumerate(self.progs) for (lst, k, q) in p.input_patches if lst is p.W]
        self._tables: Dict[int, Tuple[torch.Tensor, List[int]]] = {}   # op -> (device table, its host copy)
        self._copy_of: Dict[Tuple[int, int], int] = {}                 # (position, op) -> index in this list
        for k in dense:
            ops = [p.W[k] for p in self.progs]
            assert all(o.p[2] == ops[0].p[2] and tuple(o.i[:6]) == tuple(ops[0].i[:6]) for o in ops)
            host = [o.p[0] for o in ops] + [o.p[1] for o in ops]
            table = torch.tensor(host, dtype=torch.int64, device=dev)
            self._tables[k] = (table, host)
            op = N.Op()
            C.memmove(C.byref(op), C.byref(ops[0]), C.sizeof(N.Op))
            op.kind = N.OP_GEMM_KSEG
            op.flags = 0
            op.p[0], op.p[1] = table.data_ptr(), table.data_ptr() + 8 * n_mb
            op.i[7] = n_mb
            self.beta_ops.append(self.list.append(op))
            batched.add(k)
        for k in seg:
            ops = [p.W[k] for p in self.progs]
            assert all(o.p[7] == ops[0].p[7] and tuple(o.i[:2]) == tuple(ops[0].i[:2]) and
                       tuple(o.i[3:6]) == tuple(ops[0].i[3:6]) and o.i[7] == ops[0].i[7] for o in ops)
            host = [o.p[0] for o in ops] + [o.p[1] for o in ops] + [o.p[6] for o in ops]
            table = torch.tensor(host, dtype=torch.int64, device=dev)
            self._tables[k] = (table, host)
            op = N.Op()
            C.memmove(C.byref(op), C.byref(ops[0]), C.sizeof(N.Op))
            op.kind = N.OP_GEMM_SEG_KSEG
            op.flags = 0
            op.p[0], op.p[1] = table.data_ptr(), table.data_ptr() + 8 * n_mb
            op.p[6] = table.data_ptr() + 16 * n_mb
            op.i[8] = n_mb
            self.beta_ops.append(self.list.append(op))
            batched.add(k)
        for pos, p in enumerate(self.progs):
            for k in range(n_ops):
                if k in batched:
                    continue
                op = N.Op()
                C.memmove(C.byref(op), C.byref(p.W[k]), C.sizeof(N.Op))
                idx = self.list.append(op)
                self._copy_of[(pos, k)] = idx
                if p.w_tags[k] is not None:
                    self.rest.append((idx, pos, p.w_tags[k]))
        self.list.freeze()
        self.n_batched = len(batched)
        self._patched = patched
        self._table_slot = {0: 0, 1: 1, 6: 2}     # pointer slot of an op -> which third of its table

    def _follow_input_patches(self) -> None:
        """Re-points the copies at what the per-microbatch lists point at now."""
        n_mb = len(self.progs)
        for pos, k, q in self._patched:
            ptr = self.progs[pos].W[k].p[q]
            if k in self._tables:
                table, host = self._tables[k]
                at = self._table_slot[q] * n_mb + pos
                if host[at] != ptr:
                    host[at] = ptr
                    table[at] = ptr
            else:
                self.list[self._copy_of[(pos, k)]].p[q] = ptr

    def run(self, init: bool) -> None:
        """``init``: the accumulation starts with this batch (the accumulators are overwritten)."""
        lst = self.list
        self._follow_input_patches()
        for k in self.beta_ops:
            lst[k].j[4] = 0 if init else 1
        for k, pos, tag in self.rest:
            first = init and pos == 0
            if tag == "accum":
                lst[k].j[0] = int(first)
            elif tag == "beta":
                lst[k].j[4] = 0 if first else 1
            elif tag == "fill":
                if first:
                    lst[k].flags &= ~OP_SKIP
                else:
                    lst[k].flags |= OP_SKIP
        lst.run()


def _like_view(padded_grad: torch.Tensor, out_view: torch.Tensor, padded_out: torch.Tensor) -> torch.Tensor:
    """The view of ``padded_grad`` that corresponds to ``out_view`` inside ``padded_out``."""
    off = (out_view.data_ptr() - padded_out.data_ptr()) // out_view.element_size()
    return torch.as_strided(padded_grad, out_view.shape, out_view.stride(), off)
