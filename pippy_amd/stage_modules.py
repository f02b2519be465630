"""Stage building blocks that lower to HIP launch lists.

Each block is an ordinary ``nn.Module``: its ``forward`` is the torch statement of what it
computes (used for tracing, for un-pipelined comparison runs and by the CPU oracle), and its
``lower`` emits the kernels that compute the same thing on the GPU for one microbatch slot,
registering one backward emitter that produces the input-gradient (I) and weight-gradient (W)
ops.  These are the modules the reference would run through ``submod(*args)``
(``pippy/_PipelineStage.py:420-428``) and differentiate with ``torch.autograd.backward``
(``pippy/_backward.py:67-69``).
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _native as N
from . import _program as P


class NativeBlock(nn.Module):
    """Base class of lowerable blocks."""

    def lower(self, b: "P.Builder", x: torch.Tensor) -> torch.Tensor:  # pragma: no cover
        raise NotImplementedError

    def _pp_padded_rows(self) -> List[Tuple[nn.Parameter, int]]:
        """(parameter, padded leading size) pairs for parameters stored with padding."""
        return []

    def _pp_direct_acc_params(self) -> List[nn.Parameter]:
        """Parameters whose gradient is added straight into the fp32 accumulator."""
        return []


def _as2d(t: torch.Tensor) -> torch.Tensor:
    return t.reshape(-1, t.shape[-1])


# ---- lowering helpers for standard layers ------------------------------------------------------
def lower_linear(b: "P.Builder", name: str, lin: nn.Linear, x2d: torch.Tensor, *, epilogue=N.EPI_BIAS,
                 aux_in=None, save_pre=False, out: Optional[torch.Tensor] = None):
    """y = epilogue(x W^T + bias).  Returns (y, pre_activation or None)."""
    if getattr(lin, "weight_in_out", False):
        if lin.weight.dtype != torch.bfloat16:
            raise RuntimeError("a linear layer that stores its weight as [in, out] lowers in bf16 only")
        W = b.weight_t(lin.weight)     # the [out, in] copy: both GEMM operands k-contiguous
    else:
        W = b.weight(lin.weight)
    bias = b.weight(lin.bias) if lin.bias is not None else None
    T = x2d.shape[0]
    y = out if out is not None else b.act(name, (T, W.shape[0]))
    pre = b.act(name + ".pre", (T, W.shape[0])) if save_pre else None
    if bias is None and epilogue == N.EPI_BIAS:
        epilogue = N.EPI_NONE
    b.f(P.op_gemm(x2d, W, y, epilogue=epilogue, bias=bias, aux_in=aux_in, aux_out=pre))
    return y, pre


def lower_stacked_linears(b: "P.Builder", name: str, layers, x2d: torch.Tensor) -> torch.Tensor:
    """[y1 | y2 | ...] for ``nn.Linear`` layers that read the same input, as one GEMM with the arena's
    stacked copy of their weights (and biases); three GEMMs into column ranges of the buffer when only
    some of them have a bias."""
    T = x2d.shape[0]
    y = b.act(name, (T, sum(lin.out_features for lin in layers)))
    biases = [lin.bias for lin in layers]
    if all(bias is None for bias in biases) or all(bias is not None for bias in biases):
        bias = b.rows_cat(*biases) if biases[0] is not None else None
        b.f(P.op_gemm(x2d, b.rows_cat(*(lin.weight for lin in layers)), y,
                      epilogue=N.EPI_BIAS if bias is not None else N.EPI_NONE, bias=bias))
        return y
    lo = 0
    for k, lin in enumerate(layers):
        lower_linear(b, f"{name}{k}", lin, x2d, out=y[:, lo:lo + lin.out_features])
        lo += lin.out_features
    return y


def bias_grad(b: "P.Builder", lin: nn.Linear, dY2d: torch.Tensor):
    """db = column sum of dY (W pass)."""
    if lin.bias is None:
        return
    if dY2d.dtype == torch.float32:
        # fp32 stages are small: ones[1, T] @ dY through the fp32 GEMM is an ordered column sum
        ones = b.sp.ones_f32(dY2d.shape[0])
        epi = b.weight_grad_epilogue(lin.bias)
        if epi is not None:
            b.w(P.op_gemm(ones, dY2d, b.grad_acc(lin.bias).view(1, -1), b_trans=True, epilogue=epi, beta=1),
                tag="beta")
        else:
            b.w(P.op_gemm(ones, dY2d, b.grad_target(lin.bias).view(1, -1), b_trans=True))
        return
    M, Nn = dY2d.shape
    # reductions of one pass run as one grouped launch: every op needs a workspace of its own
    ws = b.workspace("colsum:" + str(id(lin)), (2 * ((M + 127) // 128) * Nn,), torch.float32)
    b.w_reduce(P.op_colsum(dY2d, b.grad_target(lin.bias), ws))


def linear_backward(b: "P.Builder", name: str, lin: nn.Linear, x2d: torch.Tensor, dY2d: torch.Tensor, *,
                    need_dx=True, dx_out=None, dx_epilogue=N.EPI_NONE, dx_aux=None, padded=True):
    """I: dX = epilogue(dY W); W: dW = dY^T X, db = colsum(dY)."""
    if getattr(lin, "weight_in_out", False):
        # the stored [in, out] weight is what the input-gradient GEMM reads; its gradient is X^T dY
        Wio = b.weight(lin.weight)
        dx = None
        if need_dx:
            dx = dx_out if dx_out is not None else b.grad(name + ".dx", (dY2d.shape[0], Wio.shape[0]))
            ws = None
            copies = P.splitk_copies(dY2d.shape[0], Wio.shape[0], dY2d.shape[1])
            if copies and dx_epilogue == N.EPI_NONE:
                ws = b.workspace("splitk", (copies * dY2d.shape[0] * Wio.shape[0],), torch.float32)
            b.i(P.op_gemm(dY2d, Wio, dx, epilogue=dx_epilogue, aux_in=dx_aux, splitk_workspace=ws))
        b.w_weight_gemm(x2d, dY2d, lin.weight)
        bias_grad(b, lin, dY2d)
        return dx
    W = b.weight(lin.weight, padded)
    dx = None
    if need_dx:
        dx = dx_out if dx_out is not None else b.grad(name + ".dx", (dY2d.shape[0], W.shape[1]))
        if W.dtype == torch.bfloat16:
            # dX = dY W with the transposed weight copy: both operands k-contiguous; a long reduction
            # into a small output (the vocabulary projection) is split along K through a workspace
            ws = None
            copies = P.splitk_copies(dY2d.shape[0], W.shape[1], dY2d.shape[1])
            if copies and dx_epilogue == N.EPI_NONE:
                ws = b.workspace("splitk", (copies * dY2d.shape[0] * W.shape[1],), torch.float32)
            b.i(P.op_gemm(dY2d, b.weight_t(lin.weight), dx, epilogue=dx_epilogue, aux_in=dx_aux,
                          splitk_workspace=ws))
        else:
            b.i(P.op_gemm(dY2d, W, dx, b_trans=True, epilogue=dx_epilogue, aux_in=dx_aux))
    b.w_weight_gemm(dY2d, x2d, lin.weight, padded)
    bias_grad(b, lin, dY2d)
    return dx


def lower_attention(b: "P.Builder", qkv: torch.Tensor, Bn: int, S: int, H: int, causal: bool,
                    n_kv_heads: Optional[int] = None, scale: Optional[float] = None):
    """Emits attention over the q|k|v rows ``qkv`` [Bn * S, W].  Returns the output [Bn * S, H * D] and the
    emitter of the backward, ``d_att -> dqkv`` ([Bn * S, W]).

    The kernels take sequence lengths that are multiples of 64.  Any other length runs on copies padded
    to the next multiple with zero rows: the forward leaves the keys past the end out of the softmax
    (``kv_len``; under a causal mask no real query sees them anyway), and in the backward a query past
    the end has no output gradient while a key past the end has zero key and value rows, so the real
    rows come out exactly as without padding, forward and backward."""
    T, W = qkv.shape
    Hkv = H if n_kv_heads is None else n_kv_heads
    D = W // (H + 2 * Hkv)
    Cc = H * D
    # Without a causal mask every query sees every key: at initialisation attention is then nearly uniform
    # over the whole sequence and the query gradients are small differences of large terms, which the
    # rounding of the forward's output would swamp (the dQ kernel corrects for it at one more MFMA per
    # block).  Under a causal mask the early queries see few keys and the effect stays below the rounding
    # of the operands themselves.
    exact_dq = not causal
    att = b.act("att", (T, Cc))
    if S % 64 == 0:
        lse = b.act("lse", (Bn, H, S), torch.float32)
        b.f(P.op_attn(N.OP_ATTN_FWD, qkv.view(Bn, S, W), att.view(Bn, S, Cc), lse, H, causal, n_kv_heads=Hkv,
                      scale=scale))

        def backward(d_att):
            dqkv = b.grad("dqkv", (T, W))
            delta = b.scratch("attn_delta", (Bn, H, S), torch.float32)
            b.i(P.op_attn(N.OP_ATTN_BWD, qkv.view(Bn, S, W), att.view(Bn, S, Cc), lse, H, causal,
                          d_o=d_att.view(Bn, S, Cc), dqkv=dqkv.view(Bn, S, W), delta=delta, n_kv_heads=Hkv,
                          scale=scale, exact_dq=exact_dq))
            return dqkv

        return att, backward
    Sp = (S + 63) // 64 * 64
    es = qkv.element_size()
    qkv_p = b.act("qkv_padded", (Bn, Sp, W))
    att_p = b.act("att_padded", (Bn, Sp, Cc))
    lse = b.act("lse", (Bn, H, Sp), torch.float32)
    qkv_p.zero_()       # once: the launch lists only ever write the real rows
    b.f(P.op_copy_rows(qkv, qkv_p, Bn, S * W * es, S * W * es, Sp * W * es))
    b.f(P.op_attn(N.OP_ATTN_FWD, qkv_p, att_p, lse, H, causal, n_kv_heads=Hkv, kv_len=S, scale=scale))
    b.f(P.op_copy_rows(att_p, att, Bn, S * Cc * es, Sp * Cc * es, S * Cc * es))

    def backward(d_att):
        d_att_p = b.grad("d_att_padded", (Bn, Sp, Cc))
        dqkv_p = b.grad("dqkv_padded", (Bn, Sp, W))
        dqkv = b.grad("dqkv", (T, W))
        delta = b.scratch("attn_delta", (Bn, H, Sp), torch.float32)
        if d_att_p.data_ptr() not in b.sp.zeroed_once:      # (shared by the microbatches of a stage)
            d_att_p.zero_()
            b.sp.zeroed_once.add(d_att_p.data_ptr())
        b.i(P.op_copy_rows(d_att, d_att_p, Bn, S * Cc * es, S * Cc * es, Sp * Cc * es))
        b.i(P.op_attn(N.OP_ATTN_BWD, qkv_p, att_p, lse, H, causal, d_o=d_att_p, dqkv=dqkv_p, delta=delta,
                      n_kv_heads=Hkv, kv_len=S, scale=scale, exact_dq=exact_dq))
        b.i(P.op_copy_rows(dqkv_p, dqkv, Bn, S * W * es, Sp * W * es, S * W * es))
        return dqkv

    return att, backward


def lower_layernorm(b: "P.Builder", name: str, ln: nn.LayerNorm, x2d: torch.Tensor):
    T, Cc = x2d.shape
    y = b.act(name, (T, Cc))
    mean = b.act(name + ".mean", (T,), torch.float32)
    rstd = b.act(name + ".rstd", (T,), torch.float32)
    b.f(P.op_ln_fwd(x2d, b.weight(ln.weight), b.weight(ln.bias) if ln.bias is not None else None, y,
                    mean, rstd, ln.eps))
    return y, mean, rstd


def layernorm_backward(b: "P.Builder", name: str, ln: nn.LayerNorm, x2d, mean, rstd, dy2d, dres=None,
                       dx_out=None):
    """I: dx = LN'(dy) + dres; W: dgamma, dbeta."""
    T, Cc = x2d.shape
    dx = dx_out if dx_out is not None else b.grad(name + ".dx", (T, Cc))
    b.i(P.op_ln_bwd_input(dy2d, x2d, b.weight(ln.weight), mean, rstd, dres, dx))
    ws = b.workspace("ln_bwd:" + str(id(ln)), (2 * ((T + 127) // 128) * Cc,), torch.float32)
    has_bias = ln.bias is not None
    b.w_reduce(P.op_ln_bwd_weight(dy2d, x2d, mean, rstd, b.grad_target(ln.weight),
                                  b.grad_target(ln.bias) if has_bias else None, ws))
    return dx


_ACT_EPI = {None: N.EPI_BIAS, "relu": N.EPI_BIAS_RELU, "gelu_erf": N.EPI_BIAS_GELU_ERF,
            "gelu_tanh": N.EPI_BIAS_GELU_TANH}
_ACT_DEPI = {"gelu_erf": N.EPI_DGELU_ERF, "gelu_tanh": N.EPI_DGELU_TANH, "relu": N.EPI_DRELU}
_ACT_KIND = {"relu": N.ACT_RELU, "gelu_erf": N.ACT_GELU_ERF, "gelu_tanh": N.ACT_GELU_TANH}


def _torch_act(y, activation):
    if activation == "silu":
        return F.silu(y)
    if activation == "relu":
        return torch.relu(y)
    if activation == "gelu_erf":
        return F.gelu(y)
    if activation == "gelu_tanh":
        return F.gelu(y, approximate="tanh")
    return y


# ---- blocks ---------------------------------------------------------------------------------------
class LinearAct(NativeBlock):
    """``activation(linear(x))`` around a standard ``nn.Linear`` (activation: None, "relu",
    "gelu_erf", "gelu_tanh").  The stage lowering builds it from an ``nn.Linear`` followed by an
    activation; it wraps the original module, so parameter names stay those of the user's model."""

    def __init__(self, lin: nn.Linear, activation: Optional[str] = None):
        super().__init__()
        assert activation in _ACT_EPI
        self.lin = lin
        self.activation = activation

    def forward(self, x):
        return _torch_act(self.lin(x), self.activation)

    def lower(self, b, x):
        x2d = _as2d(x)
        act = self.activation
        save_pre = b.training and act in ("gelu_erf", "gelu_tanh")
        y, pre = lower_linear(b, "y", self.lin, x2d, epilogue=_ACT_EPI[act], save_pre=save_pre)
        out = y.view(x.shape[:-1] + (y.shape[-1],))

        def bwd(dy, need_dx, dx_out):
            dy2d = _as2d(dy)
            if act is not None:
                dz = b.grad("dz", dy2d.shape, dy2d.dtype)
                # relu' can be read off the output; gelu' needs the pre-activation
                b.i(P.op_act_bwd(dy2d, y if act == "relu" else pre, dz, _ACT_KIND[act]))
                dy2d = dz
            dx = linear_backward(b, "lin", self.lin, x2d, dy2d, need_dx=need_dx,
                                 dx_out=_as2d(dx_out) if dx_out is not None else None)
            return None if dx is None else dx.view(x.shape)

        b.on_backward(bwd)
        return out


class LayerNormBlock(NativeBlock):
    """A stand-alone ``nn.LayerNorm`` over the last dimension."""

    def __init__(self, ln: nn.LayerNorm):
        super().__init__()
        self.ln = ln

    def forward(self, x):
        return self.ln(x)

    def lower(self, b, x):
        x2d = _as2d(x)
        y, mean, rstd = lower_layernorm(b, "y", self.ln, x2d)

        def bwd(dy, need_dx, dx_out):
            dx = layernorm_backward(b, "ln", self.ln, x2d, mean, rstd, _as2d(dy),
                                    dx_out=_as2d(dx_out) if dx_out is not None else None)
            return dx.view(x.shape)

        b.on_backward(bwd)
        return y.view(x.shape)


def _padding_idx(table: nn.Embedding) -> Optional[int]:
    """``nn.Embedding(padding_idx=i)`` gives row i no gradient: the embedding backward leaves that row of the
    accumulator (zero since the accumulation started) alone."""
    return getattr(table, "padding_idx", None)


class TokenEmbedding(NativeBlock):
    """Token + learned position embedding: ``wte[ids] + wpe[:S]`` (GPT-2 style);
    ``positions=False`` leaves the position table out (models with rotary embeddings)."""

    def __init__(self, vocab: int, max_seq: int, dim: int, dtype=torch.bfloat16, init_std=0.02,
                 positions: bool = True):
        super().__init__()
        self.wte = nn.Embedding(vocab, dim, dtype=dtype)
        nn.init.normal_(self.wte.weight, std=init_std)
        self.wpe = None
        if positions:
            self.wpe = nn.Embedding(max_seq, dim, dtype=dtype)
            nn.init.normal_(self.wpe.weight, std=init_std)

    position_offset = 0      # position p reads row p + position_offset of the table (OPT keeps two spare rows)

    def forward(self, ids):
        if self.wpe is None:
            return self.wte(ids)
        S = ids.shape[-1]
        pos = torch.arange(S, device=ids.device) + self.position_offset
        return self.wte(ids) + self.wpe(pos)

    def _pp_direct_acc_params(self):
        return [self.wte.weight] + ([self.wpe.weight] if self.wpe is not None else [])

    def lower(self, b, ids):
        if ids.dtype != torch.int64 or ids.dim() != 2:
            raise RuntimeError(f"TokenEmbedding expects int64 ids of shape [batch, seq], got "
                               f"{ids.dtype} {tuple(ids.shape)}")
        Bn, S = ids.shape
        wte = b.weight(self.wte.weight)
        first = self.position_offset
        wpe = b.weight(self.wpe.weight)[first:] if self.wpe is not None else None
        if wpe is not None and S > wpe.shape[0]:
            raise RuntimeError(f"sequence length {S} exceeds the position table ({wpe.shape[0]} rows from row {first})")
        Cc = wte.shape[1]
        y = b.act("y", (Bn, S, Cc))
        b.f(P.op_embed_fwd(ids, wte, wpe, y.view(Bn * S, Cc), S))

        def bwd(dy, need_dx, dx_out):
            # added straight into the fp32 accumulators (zeroed on the first accumulation): per row the
            # sum over its tokens in ascending order, rounded to bf16 first unless the stage adds
            # unrounded sums (``fused_accumulate=True``)
            acc_wte = b.grad_acc(self.wte.weight)
            acc_wpe = b.grad_acc(self.wpe.weight) if self.wpe is not None else None
            b.w(P.op_fill(acc_wte), tag="fill")
            if acc_wpe is not None:
                b.w(P.op_fill(acc_wpe), tag="fill")
            b.w(P.op_embed_bwd(ids, dy.view(Bn * S, Cc), acc_wte, acc_wpe[first:] if acc_wpe is not None else None,
                               S, round_bf16=not b.fused_accumulate, padding_idx=_padding_idx(self.wte)))
            return None

        b.on_backward(bwd)
        return y


class EncoderEmbedding(NativeBlock):
    """BERT-style embedding: ``LayerNorm(word[ids] + position[:S] + token_type[0])``.  All tokens
    are of type 0, which is what the encoder computes when no ``token_type_ids`` are passed.  A
    wrapper around a user's layers may have no token-type table (``token_type_embeddings = None``) or no
    LayerNorm (``LayerNorm = None``: an encoder that normalises inside its layers)."""

    def __init__(self, vocab: int, max_seq: int, dim: int, n_types: int = 2, eps: float = 1e-12,
                 dtype=torch.bfloat16, init_std=0.02):
        super().__init__()
        self.word_embeddings = nn.Embedding(vocab, dim, dtype=dtype)
        self.position_embeddings = nn.Embedding(max_seq, dim, dtype=dtype)
        self.token_type_embeddings = nn.Embedding(n_types, dim, dtype=dtype)
        self.LayerNorm = nn.LayerNorm(dim, eps=eps, dtype=dtype)
        for emb in (self.word_embeddings, self.position_embeddings, self.token_type_embeddings):
            nn.init.normal_(emb.weight, std=init_std)

    # None: position s reads row s.  A token id: the positions are counted over the tokens that are not
    # that (padding) id, starting one past it, and padding tokens read row ``padding_positions`` (RoBERTa)
    padding_positions = None

    def _positions(self, ids):
        if self.padding_positions is None:
            return torch.arange(ids.shape[-1], device=ids.device)
        real = (ids != self.padding_positions).long()
        return torch.cumsum(real, dim=-1) * real + self.padding_positions

    def forward(self, ids):
        pos = self._positions(ids)
        # one rounding of the three-term sum, as the lowered kernel does
        e = self.word_embeddings(ids).float() + self.position_embeddings(pos).float()
        if self.token_type_embeddings is not None:
            e = e + self.token_type_embeddings.weight[0].float()
        e = e.to(self.word_embeddings.weight.dtype)
        return self.LayerNorm(e) if self.LayerNorm is not None else e

    def _pp_direct_acc_params(self):
        return [self.word_embeddings.weight, self.position_embeddings.weight]

    def lower(self, b, ids):
        if ids.dtype != torch.int64 or ids.dim() != 2:
            raise RuntimeError(f"EncoderEmbedding expects int64 ids of shape [batch, seq], got "
                               f"{ids.dtype} {tuple(ids.shape)}")
        Bn, S = ids.shape
        wte, wpe = b.weight(self.word_embeddings.weight), b.weight(self.position_embeddings.weight)
        wtt = b.weight(self.token_type_embeddings.weight) if self.token_type_embeddings is not None else None
        pad = self.padding_positions
        if S + (0 if pad is None else pad + 1) > wpe.shape[0]:
            raise RuntimeError(f"sequence length {S} exceeds the position table ({wpe.shape[0]} rows"
                               f"{'' if pad is None else f', the first {pad + 1} not for positions'})")
        Cc = wte.shape[1]
        T = Bn * S
        e = b.act("e", (T, Cc))
        pos_ids = None
        if pad is not None:
            pos_ids = b.act("pos_ids", (Bn, S), torch.int64)
            b.f(P.op_position_ids(ids, pos_ids, pad))
        b.f(P.op_embed_fwd(ids, wte, wpe, e, S, extra_row=wtt[0] if wtt is not None else None,
                           pos_ids=pos_ids.view(-1) if pos_ids is not None else None))
        if self.LayerNorm is not None:
            y, mean, rstd = lower_layernorm(b, "ln", self.LayerNorm, e)
        else:
            y = e

        def bwd(dy, need_dx, dx_out):
            de = dy.view(T, Cc)
            if self.LayerNorm is not None:
                de = layernorm_backward(b, "ln", self.LayerNorm, e, mean, rstd, de)
            acc_wte = b.grad_acc(self.word_embeddings.weight)
            acc_wpe = b.grad_acc(self.position_embeddings.weight)
            b.w(P.op_fill(acc_wte), tag="fill")
            b.w(P.op_fill(acc_wpe), tag="fill")
            pad_w = _padding_idx(self.word_embeddings)
            if pos_ids is None:
                b.w(P.op_embed_bwd(ids, de, acc_wte, acc_wpe, S, round_bf16=not b.fused_accumulate, padding_idx=pad_w))
            else:   # the position table is one more table read at computed indices
                b.w(P.op_embed_bwd(ids, de, acc_wte, None, S, round_bf16=not b.fused_accumulate, padding_idx=pad_w))
                b.w(P.op_embed_bwd(pos_ids.view(-1), de, acc_wpe, None, S, round_bf16=not b.fused_accumulate,
                                   padding_idx=_padding_idx(self.position_embeddings)))
            if wtt is not None:
                # the type-0 row receives the gradient of every token; the other rows none
                g_tt = b.grad_target(self.token_type_embeddings.weight)
                ws = b.workspace("colsum:tt", (2 * ((T + 127) // 128) * Cc,), torch.float32)
                b.w_reduce(P.op_colsum(de, g_tt[0], ws))
            return None

        b.on_backward(bwd)
        return y.view(Bn, S, Cc)


class TransformerLayer(NativeBlock):
    """One transformer layer: multi-head self-attention and a GELU feed-forward, pre-LayerNorm
    (GPT-2) or post-LayerNorm (BERT).  Parameter names follow GPT-2 (``ln_1``, ``attn.c_attn``,
    ``attn.c_proj``, ``ln_2``, ``mlp.c_fc``, ``mlp.c_proj``) with ``nn.Linear`` weights [out, in]."""

    def __init__(self, dim: int, n_heads: int, ffn: int, *, causal: bool = True, pre_ln: bool = True,
                 activation: str = "gelu_tanh", eps: float = 1e-5, dtype=torch.bfloat16, init_std=0.02):
        super().__init__()
        assert dim % n_heads == 0 and activation in ("gelu_tanh", "gelu_erf", "relu")
        self.dim, self.n_heads, self.ffn = dim, n_heads, ffn
        self.causal, self.pre_ln, self.activation = causal, pre_ln, activation
        self.ln_1 = nn.LayerNorm(dim, eps=eps, dtype=dtype)
        self.attn = nn.Module()
        self.attn.c_attn = nn.Linear(dim, 3 * dim, dtype=dtype)
        self.attn.c_proj = nn.Linear(dim, dim, dtype=dtype)
        self.ln_2 = nn.LayerNorm(dim, eps=eps, dtype=dtype)
        self.mlp = nn.Module()
        self.mlp.c_fc = nn.Linear(dim, ffn, dtype=dtype)
        self.mlp.c_proj = nn.Linear(ffn, dim, dtype=dtype)
        for lin in (self.attn.c_attn, self.attn.c_proj, self.mlp.c_fc, self.mlp.c_proj):
            nn.init.normal_(lin.weight, std=init_std)
            nn.init.zeros_(lin.bias)

    attn_scale = None      # the factor on the attention scores; None: 1 / sqrt(head size)
    n_kv_heads = None      # fewer key / value heads than query heads (multi-query: 1); None: as many

    # torch statement of the layer
    def _attention(self, h):
        Bn, S, Cc = h.shape
        H, D = self.n_heads, Cc // self.n_heads
        Hkv = self.n_kv_heads or H
        q, k, v = self._project_qkv(h).split([H * D, Hkv * D, Hkv * D], dim=-1)
        q = q.reshape(Bn, S, H, D).transpose(1, 2)
        k, v = (t.reshape(Bn, S, Hkv, D).transpose(1, 2).repeat_interleave(H // Hkv, dim=1) for t in (k, v))
        o = F.scaled_dot_product_attention(q, k, v, is_causal=self.causal, scale=self.attn_scale)
        return self.attn.c_proj(o.transpose(1, 2).reshape(Bn, S, Cc))

    def forward(self, x):
        if self.pre_ln:
            x = x + self._attention(self.ln_1(x))
            return x + self.mlp.c_proj(_torch_act(self.mlp.c_fc(self.ln_2(x)), self.activation))
        x = self.ln_1(x + self._attention(x))
        return self.ln_2(x + self.mlp.c_proj(_torch_act(self.mlp.c_fc(x), self.activation)))

    # the q|k|v projection: one fused layer here; subclasses around a user's model may hold three
    def _qkv_layers(self):
        return (self.attn.c_attn,)

    def _project_qkv(self, h):
        return torch.cat([lin(h) for lin in self._qkv_layers()], dim=-1)

    def _lower_qkv(self, b, h2d):
        """Emits the projection; returns the [tokens, 3 d] buffer the attention kernels read."""
        layers = self._qkv_layers()
        if len(layers) == 1:
            return lower_linear(b, "qkv", layers[0], h2d)[0]
        return lower_stacked_linears(b, "qkv", layers, h2d)

    def _qkv_backward(self, b, h2d, dqkv, *, dx_epilogue=N.EPI_NONE, dx_aux=None, dx_out=None):
        """Emits input and weight gradients of the projection; returns the gradient of its input."""
        layers = self._qkv_layers()
        if len(layers) == 1:
            return linear_backward(b, "c_attn", layers[0], h2d, dqkv, dx_epilogue=dx_epilogue, dx_aux=dx_aux,
                                   dx_out=dx_out)
        # one product of the whole gradient with the transposed weights side by side
        dx = dx_out if dx_out is not None else b.grad("c_attn.dx", tuple(h2d.shape))
        b.i(P.op_gemm(dqkv, b.weight_t_cat(*(lin.weight for lin in layers)), dx, epilogue=dx_epilogue,
                      aux_in=dx_aux))
        lo = 0
        for name, lin in zip("qkv", layers):
            linear_backward(b, name, lin, h2d, dqkv[:, lo:lo + lin.out_features], need_dx=False)
            lo += lin.out_features
        return dx

    def lower(self, b, x):
        if x.dim() != 3:
            raise RuntimeError(f"TransformerLayer expects [batch, seq, dim], got {tuple(x.shape)}")
        Bn, S, Cc = x.shape
        if Cc != self.dim:
            raise RuntimeError(f"TransformerLayer of width {self.dim} got width {Cc}")
        return self._lower_pre_ln(b, x) if self.pre_ln else self._lower_post_ln(b, x)

    def _lower_pre_ln(self, b, x):
        Bn, S, Cc = x.shape
        T, H = Bn * S, self.n_heads
        x2d = x.view(T, Cc)
        act, dact = _ACT_EPI[self.activation], _ACT_DEPI[self.activation]
        ln1, mean1, rstd1 = lower_layernorm(b, "ln1", self.ln_1, x2d)
        qkv = self._lower_qkv(b, ln1)
        att, attention_backward = lower_attention(b, qkv, Bn, S, H, self.causal, n_kv_heads=self.n_kv_heads, scale=self.attn_scale)
        x2, _ = lower_linear(b, "x2", self.attn.c_proj, att, epilogue=N.EPI_BIAS_RESIDUAL, aux_in=x2d)
        ln2, mean2, rstd2 = lower_layernorm(b, "ln2", self.ln_2, x2)
        # (the derivative of a ReLU is read off its output; a GELU's needs the value before it)
        h, h_pre = lower_linear(b, "h", self.mlp.c_fc, ln2, epilogue=act,
                                save_pre=b.training and self.activation != "relu")
        if self.activation == "relu":
            h_pre = h
        y, _ = lower_linear(b, "y", self.mlp.c_proj, h, epilogue=N.EPI_BIAS_RESIDUAL, aux_in=x2)

        def bwd(dy, need_dx, dx_out):
            dy2d = dy.view(T, Cc)
            # feed-forward: dI through c_proj carries gelu'(h_pre) in its epilogue
            d_hpre = linear_backward(b, "c_proj", self.mlp.c_proj, h, dy2d, dx_epilogue=dact, dx_aux=h_pre)
            d_ln2 = linear_backward(b, "c_fc", self.mlp.c_fc, ln2, d_hpre)
            d_x2 = layernorm_backward(b, "ln2", self.ln_2, x2, mean2, rstd2, d_ln2, dres=dy2d)
            # attention
            d_att = linear_backward(b, "attn_proj", self.attn.c_proj, att, d_x2)
            dqkv = attention_backward(d_att)
            d_ln1 = self._qkv_backward(b, ln1, dqkv)
            dx = layernorm_backward(b, "ln1", self.ln_1, x2d, mean1, rstd1, d_ln1, dres=d_x2,
                                    dx_out=dx_out.view(T, Cc) if dx_out is not None else None)
            return dx.view(Bn, S, Cc)

        b.on_backward(bwd)
        return y.view(Bn, S, Cc)

    def _lower_post_ln(self, b, x):
        Bn, S, Cc = x.shape
        T, H = Bn * S, self.n_heads
        x2d = x.view(T, Cc)
        act, dact = _ACT_EPI[self.activation], _ACT_DEPI[self.activation]
        qkv = self._lower_qkv(b, x2d)
        att, attention_backward = lower_attention(b, qkv, Bn, S, H, self.causal, n_kv_heads=self.n_kv_heads, scale=self.attn_scale)
        a, _ = lower_linear(b, "a", self.attn.c_proj, att, epilogue=N.EPI_BIAS_RESIDUAL, aux_in=x2d)
        x1, mean1, rstd1 = lower_layernorm(b, "ln1", self.ln_1, a)
        h, h_pre = lower_linear(b, "h", self.mlp.c_fc, x1, epilogue=act,
                                save_pre=b.training and self.activation != "relu")
        if self.activation == "relu":
            h_pre = h
        f, _ = lower_linear(b, "f", self.mlp.c_proj, h, epilogue=N.EPI_BIAS_RESIDUAL, aux_in=x1)
        y, mean2, rstd2 = lower_layernorm(b, "ln2", self.ln_2, f)

        def bwd(dy, need_dx, dx_out):
            # a sum of two gradients in front of a LayerNorm is formed by the residual epilogue
            # (without a bias) of the input-gradient GEMM that produces one of them
            d_f = layernorm_backward(b, "ln2", self.ln_2, f, mean2, rstd2, dy.view(T, Cc))
            d_hpre = linear_backward(b, "c_proj", self.mlp.c_proj, h, d_f, dx_epilogue=dact, dx_aux=h_pre)
            d_x1 = linear_backward(b, "c_fc", self.mlp.c_fc, x1, d_hpre, dx_epilogue=N.EPI_BIAS_RESIDUAL,
                                   dx_aux=d_f)
            d_a = layernorm_backward(b, "ln1", self.ln_1, a, mean1, rstd1, d_x1)
            d_att = linear_backward(b, "attn_proj", self.attn.c_proj, att, d_a)
            dqkv = attention_backward(d_att)
            dx = self._qkv_backward(b, x2d, dqkv, dx_epilogue=N.EPI_BIAS_RESIDUAL, dx_aux=d_a,
                                    dx_out=dx_out.view(T, Cc) if dx_out is not None else None)
            return dx.view(Bn, S, Cc)

        b.on_backward(bwd)
        return y.view(Bn, S, Cc)


def rope_tables(seq: int, head_dim: int, theta: float, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos, sin [seq, head_dim / 2] in fp32: the angle of position p and frequency index i is
    p * theta^(-2 i / head_dim)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32, device=device) / head_dim))
    ang = torch.arange(seq, dtype=torch.float32, device=device)[:, None] * inv_freq[None, :]
    return torch.cos(ang).contiguous(), torch.sin(ang).contiguous()


def _apply_rope(x, cos, sin):
    """Rotate-half rotary embedding on [batch, heads, seq, head_dim] (torch statement of the block)."""
    half = x.shape[-1] // 2
    a, b = x[..., :half].float(), x[..., half:].float()
    return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1).to(x.dtype)


def lower_rmsnorm(b: "P.Builder", name: str, norm: nn.Module, x2d: torch.Tensor):
    T, Cc = x2d.shape
    y = b.act(name, (T, Cc))
    rstd = b.act(name + ".rstd", (T,), torch.float32)
    b.f(P.op_ln_fwd(x2d, b.weight(norm.weight), None, y, None, rstd, norm.eps))
    return y, rstd


def rmsnorm_backward(b: "P.Builder", name: str, norm: nn.Module, x2d, rstd, dy2d, dres=None, dx_out=None):
    """I: dx = RMSNorm'(dy) + dres; W: dgamma."""
    T, Cc = x2d.shape
    dx = dx_out if dx_out is not None else b.grad(name + ".dx", (T, Cc))
    b.i(P.op_ln_bwd_input(dy2d, x2d, b.weight(norm.weight), None, rstd, dres, dx))
    ws = b.workspace("rms_bwd:" + str(id(norm)), (2 * ((T + 127) // 128) * Cc,), torch.float32)
    b.w_reduce(P.op_ln_bwd_weight(dy2d, x2d, None, rstd, b.grad_target(norm.weight), None, ws))
    return dx


class RMSNormBlock(NativeBlock):
    """A stand-alone ``nn.RMSNorm`` over the last dimension (the final norm of a Llama-style model)."""

    def __init__(self, norm: nn.Module):
        super().__init__()
        self.norm = norm

    def forward(self, x):
        return self.norm(x)

    def lower(self, b, x):
        x2d = _as2d(x)
        y, rstd = lower_rmsnorm(b, "y", self.norm, x2d)

        def bwd(dy, need_dx, dx_out):
            dx = rmsnorm_backward(b, "rms", self.norm, x2d, rstd, _as2d(dy),
                                  dx_out=_as2d(dx_out) if dx_out is not None else None)
            return dx.view(x.shape)

        b.on_backward(bwd)
        return y.view(x.shape)


class LlamaLayer(NativeBlock):
    """One Llama-style decoder layer: RMSNorm, causal self-attention with rotary position embedding
    on a fused q|k|v projection, RMSNorm, SwiGLU feed-forward; no biases.  Parameter names follow the
    Hugging Face layer (``input_layernorm``, ``self_attn.o_proj``, ``post_attention_layernorm``,
    ``mlp.gate_proj / up_proj / down_proj``) except for the fused ``self_attn.qkv_proj``, whose rows are
    the query heads, then the key heads, then the value heads.  ``n_kv_heads`` < ``n_heads`` makes it
    grouped-query attention (``num_key_value_heads`` of the Hugging Face configuration): every
    ``n_heads / n_kv_heads`` consecutive query heads share one key / value head."""

    def __init__(self, dim: int, n_heads: int, ffn: int, *, eps: float = 1e-5, rope_theta: float = 1e4,
                 dtype=torch.bfloat16, init_std=0.02, n_kv_heads: Optional[int] = None):
        super().__init__()
        assert dim % n_heads == 0 and (dim // n_heads) in (64, 128), "head dimension 64 or 128"
        self.dim, self.n_heads, self.ffn = dim, n_heads, ffn
        self.n_kv_heads = n_heads if n_kv_heads is None else n_kv_heads
        assert 0 < self.n_kv_heads <= n_heads and n_heads % self.n_kv_heads == 0, "n_kv_heads must divide n_heads"
        self.eps, self.rope_theta = eps, rope_theta
        self.input_layernorm = nn.RMSNorm(dim, eps=eps, dtype=dtype)
        self.self_attn = nn.Module()
        self.self_attn.qkv_proj = nn.Linear(dim, (n_heads + 2 * self.n_kv_heads) * (dim // n_heads), bias=False,
                                            dtype=dtype)
        self.self_attn.o_proj = nn.Linear(dim, dim, bias=False, dtype=dtype)
        self.post_attention_layernorm = nn.RMSNorm(dim, eps=eps, dtype=dtype)
        self.mlp = nn.Module()
        self.mlp.gate_proj = nn.Linear(dim, ffn, bias=False, dtype=dtype)
        self.mlp.up_proj = nn.Linear(dim, ffn, bias=False, dtype=dtype)
        self.mlp.down_proj = nn.Linear(ffn, dim, bias=False, dtype=dtype)
        for lin in (self.self_attn.qkv_proj, self.self_attn.o_proj, self.mlp.gate_proj, self.mlp.up_proj,
                    self.mlp.down_proj):
            nn.init.normal_(lin.weight, std=init_std)

    # torch statement of the layer
    # the size of a head when it is not dim / n_heads (the output projection then maps n_heads * head_dim
    # back to dim), and RMS norms over each head's values of the queries / keys in front of the rotary
    # embedding (Qwen3): attributes a wrapper around a user's layers may set
    head_dim = None

    def _head_dim(self) -> int:
        return self.head_dim or self.dim // self.n_heads

    def _head_norms(self):
        """(q_norm, k_norm): submodules when set (a class attribute would hide a registered submodule)."""
        return getattr(self, "q_norm", None), getattr(self, "k_norm", None)

    def forward(self, x):
        Bn, S, Cc = x.shape
        H, Hkv, D = self.n_heads, self.n_kv_heads, self._head_dim()
        cos, sin = self._rope(S, D, x.device)
        h = self.input_layernorm(x)
        q, k, v = self._project_qkv(h).split([H * D, Hkv * D, Hkv * D], dim=-1)
        q = q.reshape(Bn, S, H, D)
        k, v = (t.reshape(Bn, S, Hkv, D) for t in (k, v))
        q_norm, k_norm = self._head_norms()
        if q_norm is not None:
            q = q_norm(q)
        if k_norm is not None:
            k = k_norm(k)
        q, k, v = (t.transpose(1, 2) for t in (q, k, v))
        q, k = _apply_rope(q, cos, sin), _apply_rope(k, cos, sin)
        if Hkv != H:  # query heads g * (H / Hkv) .. share key / value head g
            k, v = (t.repeat_interleave(H // Hkv, dim=1) for t in (k, v))
        o = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        x = x + self.self_attn.o_proj(o.transpose(1, 2).reshape(Bn, S, H * D))
        return x + self._feed_forward(self.post_attention_layernorm(x))

    def _feed_forward(self, h):
        return self.mlp.down_proj(F.silu(self.mlp.gate_proj(h)) * self.mlp.up_proj(h))

    def _project_qkv(self, h):
        return self.self_attn.qkv_proj(h)

    def _rope(self, seq, head_dim, device):
        """(cos, sin) [seq, head_dim / 2] in fp32 and a key that names their content."""
        return rope_tables(seq, head_dim, self.rope_theta, device)

    def _rope_key(self):
        return str(self.rope_theta)

    def _lower_qkv(self, b, n1):
        """Emits the q|k|v projection of the normalised input; returns the [tokens, (H + 2 Hkv) D] buffer."""
        return lower_linear(b, "qkv", self.self_attn.qkv_proj, n1)[0]

    def _qkv_backward(self, b, n1, dqkv):
        """Emits input and weight gradients of the q|k|v projection; returns the gradient of ``n1``."""
        return linear_backward(b, "qkv", self.self_attn.qkv_proj, n1, dqkv)

    def lower(self, b, x):
        if x.dim() != 3 or x.shape[-1] != self.dim:
            raise RuntimeError(f"{type(self).__name__} of width {self.dim} expects [batch, seq, dim], got "
                               f"{tuple(x.shape)}")
        Bn, S, Cc = x.shape
        T, H, Hkv = Bn * S, self.n_heads, self.n_kv_heads
        D = self._head_dim()
        W = (H + 2 * Hkv) * D  # width of the fused projection
        x2d = x.view(T, Cc)
        cos = b.sp.shared(f"rope_cos:{S}:{D}:{self._rope_key()}", (S, D // 2), torch.float32)
        sin = b.sp.shared(f"rope_sin:{S}:{D}:{self._rope_key()}", (S, D // 2), torch.float32)
        c, s_ = self._rope(S, D, x.device)
        cos.copy_(c)
        sin.copy_(s_)
        n1, rstd1 = lower_rmsnorm(b, "n1", self.input_layernorm, x2d)
        qkv = self._lower_qkv(b, n1)
        # per-head norms: the heads of the queries (keys) leave the fused buffer as rows of their own, are
        # normalised, and go back to where the rotary embedding and the attention read them
        es = qkv.element_size()
        head_norms = []
        q_norm, k_norm = self._head_norms()
        for name, norm, first, count in (("q", q_norm, 0, H), ("k", k_norm, H, Hkv)):
            if norm is None:
                continue
            part = qkv[:, first * D:(first + count) * D]
            pre = b.act(name + "_heads", (T * count, D))
            b.f(P.op_copy_rows(part, pre, T, count * D * es, W * es, count * D * es))
            normed, rstd = lower_rmsnorm(b, name + "_normed", norm, pre)
            b.f(P.op_copy_rows(normed, part, T, count * D * es, count * D * es, W * es))
            head_norms.append((name, norm, first, count, pre, rstd))
        b.f(P.op_rope(qkv, cos, sin, S, H + Hkv, D))
        att, attention_backward = lower_attention(b, qkv, Bn, S, H, True, n_kv_heads=Hkv)
        x2, _ = lower_linear(b, "x2", self.self_attn.o_proj, att, epilogue=N.EPI_BIAS_RESIDUAL, aux_in=x2d)
        y, ffn_backward = self._lower_feed_forward(b, x2)

        def bwd(dy, need_dx, dx_out):
            d_x2 = ffn_backward(dy.view(T, Cc))
            d_att = linear_backward(b, "o", self.self_attn.o_proj, att, d_x2)
            dqkv = attention_backward(d_att)
            # gradients w.r.t. the rotated q and k go back through the transposed rotation
            b.i(P.op_rope(dqkv, cos, sin, S, H + Hkv, D, inverse=True))
            for name, norm, first, count, pre, rstd in head_norms:
                part = dqkv[:, first * D:(first + count) * D]
                d_normed = b.grad(name + "_heads.dy", (T * count, D))
                b.i(P.op_copy_rows(part, d_normed, T, count * D * es, W * es, count * D * es))
                d_pre = rmsnorm_backward(b, name + "_heads", norm, pre, rstd, d_normed)
                b.i(P.op_copy_rows(d_pre, part, T, count * D * es, count * D * es, W * es))
            d_n1 = self._qkv_backward(b, n1, dqkv)
            dx = rmsnorm_backward(b, "n1", self.input_layernorm, x2d, rstd1, d_n1, dres=d_x2,
                                  dx_out=dx_out.view(T, Cc) if dx_out is not None else None)
            return dx.view(Bn, S, Cc)

        b.on_backward(bwd)
        return y.view(Bn, S, Cc)

    def _lower_feed_forward(self, b, x2):
        """Emits y = x2 + FFN(RMSNorm(x2)); returns (y, emitter of the backward: dy -> d_x2)."""
        T = x2.shape[0]
        n2, rstd2 = lower_rmsnorm(b, "n2", self.post_attention_layernorm, x2)
        mlp = self.mlp
        if (x2.dtype == torch.bfloat16 and self.ffn % 8 == 0 and
                all(lin.bias is None for lin in (mlp.gate_proj, mlp.up_proj, mlp.down_proj))):
            return self._lower_feed_forward_fused(b, x2, n2, rstd2)
        g, _ = lower_linear(b, "g", self.mlp.gate_proj, n2)
        u, _ = lower_linear(b, "u", self.mlp.up_proj, n2)
        h = b.act("h", (T, self.ffn))
        b.f(P.op_swiglu_fwd(g, u, h))
        y, _ = lower_linear(b, "y", self.mlp.down_proj, h, epilogue=N.EPI_BIAS_RESIDUAL, aux_in=x2)

        def backward(dy2d):
            d_h = linear_backward(b, "down", self.mlp.down_proj, h, dy2d)
            dg = b.grad("dg", (T, self.ffn))
            du = b.grad("du", (T, self.ffn))
            b.i(P.op_swiglu_bwd(g, u, d_h, dg, du))
            # the two branches that read n2 add up in the residual epilogue of the second GEMM
            d_n2a = linear_backward(b, "gate", self.mlp.gate_proj, n2, dg)
            d_n2 = linear_backward(b, "up", self.mlp.up_proj, n2, du, dx_epilogue=N.EPI_BIAS_RESIDUAL,
                                   dx_aux=d_n2a)
            return rmsnorm_backward(b, "n2", self.post_attention_layernorm, x2, rstd2, d_n2, dres=dy2d)

        return y, backward


    def _lower_feed_forward_fused(self, b, x2, n2, rstd2):
        """The bf16 feed-forward with SwiGLU inside the GEMMs around it: the gate and up products come
        out of one kernel together with h = silu(g) * u; the input-gradient GEMM of the down projection
        writes dg and du instead of dh; and the two input-gradient GEMMs of gate and up are one
        product of [dg | du] with the two transposed weights side by side.  g, u, h, dg, du carry the
        bits of the separate kernels; the gradient of the normalised input is one fp32 sum over both
        branches (rounded once) instead of a rounded branch added in the epilogue of the other."""
        T, ffn, mlp = x2.shape[0], self.ffn, self.mlp
        gu = b.act("gu", (T, 2 * ffn))
        h = b.act("h", (T, ffn))
        b.f(P.op_gemm_swiglu(n2, b.weight(mlp.gate_proj.weight), b.weight(mlp.up_proj.weight), gu, h))
        y, _ = lower_linear(b, "y", mlp.down_proj, h, epilogue=N.EPI_BIAS_RESIDUAL, aux_in=x2)

        def backward(dy2d):
            dgu = b.grad("dgu", (T, 2 * ffn))
            b.i(P.op_gemm_dswiglu(dy2d, b.weight_t(mlp.down_proj.weight), gu, dgu))
            d_n2 = b.grad("gate_up.dx", (T, x2.shape[1]))
            b.i(P.op_gemm(dgu, b.weight_t_cat(mlp.gate_proj.weight, mlp.up_proj.weight), d_n2))
            linear_backward(b, "down", mlp.down_proj, h, dy2d, need_dx=False)
            linear_backward(b, "gate", mlp.gate_proj, n2, dgu[:, :ffn], need_dx=False)
            linear_backward(b, "up", mlp.up_proj, n2, dgu[:, ffn:], need_dx=False)
            return rmsnorm_backward(b, "n2", self.post_attention_layernorm, x2, rstd2, d_n2, dres=dy2d)

        return y, backward


class _Expert(nn.Module):
    """SwiGLU expert with Mixtral's parameter names: w2(silu(w1 x) * w3 x)."""

    def __init__(self, dim, ffn, dtype, init_std):
        super().__init__()
        self.w1 = nn.Linear(dim, ffn, bias=False, dtype=dtype)
        self.w2 = nn.Linear(ffn, dim, bias=False, dtype=dtype)
        self.w3 = nn.Linear(dim, ffn, bias=False, dtype=dtype)
        for lin in (self.w1, self.w2, self.w3):
            nn.init.normal_(lin.weight, std=init_std)

    def forward(self, x):
        return self.w2(F.silu(self.w1(x)) * self.w3(x))


class _ExpertModules:
    """The expert weights of a layer that keeps one module per expert (``w1`` gate, ``w3`` up, ``w2``
    down, each an ``nn.Linear``): per projection, the [out, in] weights, their transposed copies and the
    places their gradients go, one tensor per expert."""

    _ATTR = {"gate": "w1", "up": "w3", "down": "w2"}

    def __init__(self, experts):
        self.experts = list(experts)

    def __len__(self):
        return len(self.experts)

    def _params(self, which):
        return [getattr(ex, self._ATTR[which]).weight for ex in self.experts]

    def weights(self, b, which):
        return [b.weight(p) for p in self._params(which)], None

    def transposed(self, b, which):
        return [b.weight_t(p) for p in self._params(which)], None

    def transposed_gate_up(self, b):
        """Per expert [in, 2 f]: the transposed gate and up weights side by side, so that the input gradient
        of both projections is one product with [dg | du]."""
        return [b.weight_t_cat(g, u) for g, u in zip(self._params("gate"), self._params("up"))], None

    def grad_epilogue(self, b, which):
        epis = {b.weight_grad_epilogue(p) for p in self._params(which)}
        assert len(epis) == 1
        return epis.pop()

    def grad_accumulators(self, b, which):
        return [b.grad_acc(p) for p in self._params(which)], None

    def grad_targets(self, b, which):
        return [b.grad_target(p) for p in self._params(which)], None

    def apply(self, e, x):
        """Torch statement of expert ``e``."""
        return self.experts[e](x)


class _ExpertTensors:
    """The expert weights of a layer that keeps them stacked: ``gate_up`` [E, 2 f, d] (gate rows first)
    and ``down`` [E, d, f] (the Hugging Face Mixtral layout).  Same interface as ``_ExpertModules``; the
    second value of a pair is the leading dimension where a tensor is a column range of a wider one."""

    def __init__(self, gate_up: nn.Parameter, down: nn.Parameter):
        assert gate_up.dim() == 3 and down.dim() == 3 and gate_up.shape[0] == down.shape[0]
        assert gate_up.shape[1] == 2 * down.shape[2] and gate_up.shape[2] == down.shape[1]
        self.gate_up, self.down = gate_up, down
        self.ffn = down.shape[2]

    def __len__(self):
        return self.gate_up.shape[0]

    def _slices(self, stacked, which):
        f = self.ffn
        if which == "down":
            return [stacked[e] for e in range(len(self))]
        return [stacked[e, :f] if which == "gate" else stacked[e, f:] for e in range(len(self))]

    def _param(self, which):
        return self.down if which == "down" else self.gate_up

    def weights(self, b, which):
        return self._slices(b.weight(self._param(which)), which), None

    def transposed(self, b, which):
        t = b.sp.arena.weight_t_stack(self._param(which))      # [E, in, out]
        if which == "down":
            return [t[e] for e in range(len(self))], None
        f = self.ffn
        return [t[e][:, :f] if which == "gate" else t[e][:, f:] for e in range(len(self))], 2 * f

    def transposed_gate_up(self, b):
        t = b.sp.arena.weight_t_stack(self.gate_up)             # [E, in, 2 f]: gate columns first
        return [t[e] for e in range(len(self))], None

    def grad_epilogue(self, b, which):
        return b.weight_grad_epilogue(self._param(which))

    def grad_accumulators(self, b, which):
        return self._slices(b.grad_acc(self._param(which)), which), None

    def grad_targets(self, b, which):
        return self._slices(b.grad_target(self._param(which)), which), None

    def apply(self, e, x):
        f = self.ffn
        gu = F.linear(x, self.gate_up[e])
        return F.linear(F.silu(gu[..., :f]) * gu[..., f:], self.down[e])


class _MoEFeedForward:
    """The sparse feed-forward half of a Mixtral-style layer (mixed into a Llama-style layer class):
    a softmax router picks two of ``n_experts`` SwiGLU experts per token, weights renormalised over the
    pair.  Needs ``self.n_experts``, ``self.ffn``, ``self._experts`` (an expert-weight bank),
    ``self._router`` (an ``nn.Linear``-shaped layer) and ``self.forced_routing``."""

    TOPK = 2
    _pp_batch_weight_grads = True      # see PipelineStageBase.prefers_batched_weight_grads

    def _padded_experts(self) -> int:
        return (self.n_experts + 7) // 8 * 8

    def _pp_padded_rows(self):
        return [(self._router.weight, self._padded_experts())] if self.n_experts % 8 else []

    def _feed_forward(self, h):
        shape = h.shape
        h = h.reshape(-1, shape[-1])
        probs = torch.softmax(self._router(h).float(), dim=-1)
        if self.forced_routing:
            idx = self.forced_routing.pop(0).to(h.device)
        else:
            idx = torch.sort(probs, dim=-1, descending=True, stable=True).indices[:, :2]
        top = probs.gather(-1, idx)
        gate = top / top.sum(-1, keepdim=True)
        y = torch.zeros(h.shape, dtype=torch.float32, device=h.device)
        for e in range(self.n_experts):
            tok, slot = torch.where(idx == e)
            if tok.numel():
                y = y.index_add(0, tok, gate[tok, slot, None] * self._experts.apply(e, h[tok]).float())
        return y.to(h.dtype).reshape(shape)

    def _pointer_list(self, b, name, tensors):
        t = b.sp.shared(f"moe_ptrs:{id(self)}:{name}", (len(tensors),), torch.int64)
        t.copy_(torch.tensor([x.data_ptr() for x in tensors], dtype=torch.int64))
        return t

    def _lower_feed_forward(self, b, x2):
        T, Cc = x2.shape
        E, K, ffn = self.n_experts, self.TOPK, self.ffn
        # the router GEMMs run with the expert count as a leading dimension and as a reduction length:
        # the router weight is stored with zero rows up to a multiple of 8, and so are the logits
        Ep = self._padded_experts()
        R = T * K
        bank, router = self._experts, self._router
        n2, rstd2 = lower_rmsnorm(b, "n2", self.post_attention_layernorm, x2)
        logits = b.act("router_logits", (T, Ep))
        lower_linear(b, "router", router, n2, out=logits)
        idx = b.act("topk_idx", (T, K), torch.int32)
        gate = b.act("gate", (T, K), torch.float32)
        b.f(P.op_moe_router(logits, idx, gate, E))
        seg = b.act("seg_start", (E + 1,), torch.int32)
        row_src = b.act("row_src", (R,), torch.int32)
        pos = b.act("pos", (R,), torch.int32)
        b.f(P.op_moe_permute(idx.view(-1), E, seg, row_src, pos))
        xp = b.act("xp", (R, Cc))
        b.f(P.op_moe_gather(n2, row_src, K, xp))

        def pointers(name, pair):
            tensors, ld = pair
            return self._pointer_list(b, name, tensors), ld

        w1, ld1 = pointers("w1", bank.weights(b, "gate"))
        w3, ld3 = pointers("w3", bank.weights(b, "up"))
        w2, ld2 = pointers("w2", bank.weights(b, "down"))
        h = b.act("h", (R, ffn))
        yp = b.act("yp", (R, Cc))
        # SwiGLU inside the expert GEMMs (gate and up products side by side, as those kernels write and read
        # them) when both weights of a tile share a leading dimension; else GEMMs and element-wise kernels
        fused = ld1 == ld3
        if fused:
            gu = b.act("gu", (R, 2 * ffn))
            g, u = gu[:, :ffn], gu[:, ffn:]
            b.f(P.op_gemm_seg_swiglu(xp, w1, w3, seg, gu, h, ld=ld1))
        else:
            g = b.act("g", (R, ffn))
            u = b.act("u", (R, ffn))
            b.f(P.op_gemm_seg(N.SEG_ROWS, xp, w1, seg, Cm=g, ld=ld1))
            b.f(P.op_gemm_seg(N.SEG_ROWS, xp, w3, seg, Cm=u, ld=ld3))
            b.f(P.op_swiglu_fwd(g, u, h))
        b.f(P.op_gemm_seg(N.SEG_ROWS, h, w2, seg, Cm=yp, ld=ld2))
        y = b.act("y", (T, Cc))
        b.f(P.op_moe_combine(yp, pos, K, y, gate=gate.view(-1), resid=x2))

        def backward(dy2d):
            # expert rows receive the output gradient of their token times the routing weight
            d_yp = b.grad("d_yp", (R, Cc))
            b.i(P.op_moe_gather(dy2d, row_src, K, d_yp, scale=gate.view(-1)))
            dlogits = b.grad("dlogits", (T, Ep))
            b.i(P.op_moe_gate_bwd(dy2d, yp, pos, idx, gate, E, dlogits))
            w2t, ld2t = pointers("w2t", bank.transposed(b, "down"))
            if fused:
                dgu = b.grad("dgu", (R, 2 * ffn))
                dg, du = dgu[:, :ffn], dgu[:, ffn:]
                b.i(P.op_gemm_seg_dswiglu(d_yp, w2t, seg, gu, dgu, ld=ld2t))
            else:
                d_h = b.grad("d_h", (R, ffn))
                b.i(P.op_gemm_seg(N.SEG_ROWS, d_yp, w2t, seg, Cm=d_h, ld=ld2t))
                dg = b.grad("dg", (R, ffn))
                du = b.grad("du", (R, ffn))
                b.i(P.op_swiglu_bwd(g, u, d_h, dg, du))
            d_xp = b.grad("d_xp", (R, Cc))
            if fused:
                # dg W1 + du W3 as one product of [dg | du] with the two transposed weights side by side
                w13t, ld13t = pointers("w13t", bank.transposed_gate_up(b))
                b.i(P.op_gemm_seg(N.SEG_ROWS, dgu, w13t, seg, Cm=d_xp, ld=ld13t))
            else:
                w1t, ld1t = pointers("w1t", bank.transposed(b, "gate"))
                w3t, ld3t = pointers("w3t", bank.transposed(b, "up"))
                b.i(P.op_gemm_seg(N.SEG_ROWS, dg, w1t, seg, Cm=d_xp, ld=ld1t))
                b.i(P.op_gemm_seg(N.SEG_ROWS, du, w3t, seg, Cm=d_xp, ld=ld3t, epilogue=N.EPI_BIAS_RESIDUAL,
                                  aux_in=d_xp))
            # token gradient: its two expert rows, plus the router branch in the GEMM epilogue
            d_n2a = b.grad("d_n2a", (T, Cc))
            b.i(P.op_moe_combine(d_xp, pos, K, d_n2a))
            d_n2 = linear_backward(b, "router", router, n2, dlogits, dx_epilogue=N.EPI_BIAS_RESIDUAL,
                                   dx_aux=d_n2a)
            # expert weight gradients: one segmented GEMM per projection, reduced over each expert's rows
            for which, name, dy_rows, x_rows in (("gate", "w1", dg, xp), ("up", "w3", du, xp), ("down", "w2", d_yp, h)):
                epi = bank.grad_epilogue(b, which)
                if epi is not None:
                    ptrs, ld = pointers("acc_" + name, bank.grad_accumulators(b, which))
                    b.w(P.op_gemm_seg(N.SEG_K, dy_rows, ptrs, seg, other=x_rows, ld=ld, epilogue=epi,
                                      beta=1, c_f32=True), tag="beta")
                else:
                    ptrs, ld = pointers("stage_" + name, bank.grad_targets(b, which))
                    b.w(P.op_gemm_seg(N.SEG_K, dy_rows, ptrs, seg, other=x_rows, ld=ld))
            return rmsnorm_backward(b, "n2", self.post_attention_layernorm, x2, rstd2, d_n2, dres=dy2d)

        return y, backward


class MoELayer(_MoEFeedForward, LlamaLayer):
    """A Mixtral-style decoder layer: the attention half of ``LlamaLayer`` and, in place of the dense
    feed-forward, a sparse mixture of ``n_experts`` SwiGLU experts of which a softmax router picks
    two per token (weights renormalised over the pair).  Parameters: ``block_sparse_moe.gate`` and
    ``block_sparse_moe.experts.<e>.w1 / w2 / w3``.  The launch-list form takes 2 .. 64 experts (a count
    that is not a multiple of 8 runs with the router weight and the logits padded to one).

    ``forced_routing`` (a list of int64 [tokens, 2] tensors, one per forward call, consumed in
    order) overrides the expert selection of the torch statement; a comparison against a lower
    precision run uses it so that tokens whose second and third logits nearly tie do not count as
    errors of the arithmetic."""

    def __init__(self, dim: int, n_heads: int, ffn: int, n_experts: int = 8, *, eps: float = 1e-5,
                 rope_theta: float = 1e6, dtype=torch.bfloat16, init_std=0.02, n_kv_heads: Optional[int] = None):
        LlamaLayer.__init__(self, dim, n_heads, ffn, eps=eps, rope_theta=rope_theta, dtype=dtype,
                            init_std=init_std, n_kv_heads=n_kv_heads)
        del self.mlp
        assert 2 <= n_experts <= 64
        self.n_experts = n_experts
        self.block_sparse_moe = nn.Module()
        self.block_sparse_moe.gate = nn.Linear(dim, n_experts, bias=False, dtype=dtype)
        nn.init.normal_(self.block_sparse_moe.gate.weight, std=init_std)
        self.block_sparse_moe.experts = nn.ModuleList([_Expert(dim, ffn, dtype, init_std) for _ in range(n_experts)])
        self.forced_routing = None

    @property
    def _router(self):
        return self.block_sparse_moe.gate

    @property
    def _experts(self):
        return _ExpertModules(self.block_sparse_moe.experts)


class LMHead(NativeBlock):
    """Final LayerNorm and the (untied) vocabulary projection.  The weight is stored with its
    vocabulary dimension padded to a multiple of 128 (zero rows) so that logits rows are 256-byte
    aligned; the block's output is the [.., vocab] view of the padded logits buffer."""

    VOCAB_ALIGN = 128

    def __init__(self, dim: int, vocab: int, *, final_ln=True, eps: float = 1e-5,
                 dtype=torch.bfloat16, init_std=0.02):
        """``final_ln``: True (LayerNorm), "rms" (RMSNorm) or False (no final normalisation)."""
        super().__init__()
        self.dim, self.vocab = dim, vocab
        if final_ln == "rms":
            self.ln_f = nn.RMSNorm(dim, eps=eps, dtype=dtype)
        else:
            self.ln_f = nn.LayerNorm(dim, eps=eps, dtype=dtype) if final_ln else None
        self.lm_head = nn.Linear(dim, vocab, bias=False, dtype=dtype)
        nn.init.normal_(self.lm_head.weight, std=init_std)

    @property
    def padded_vocab(self):
        return (self.vocab + self.VOCAB_ALIGN - 1) // self.VOCAB_ALIGN * self.VOCAB_ALIGN

    def _pp_padded_rows(self):
        rows = [(self.lm_head.weight, self.padded_vocab)]
        if self.lm_head.bias is not None:
            rows.append((self.lm_head.bias, self.padded_vocab))   # zeros beyond the vocabulary, like the weight
        return rows

    def forward(self, x):
        if self.ln_f is not None:
            x = self.ln_f(x)
        return self.lm_head(x)

    def lower(self, b, x):
        Bn, S, Cc = x.shape
        T, V, Vp = Bn * S, self.vocab, self.padded_vocab
        x2d = x.view(T, Cc)
        rms = _is_rms(self.ln_f)
        if rms:
            h, rstd = lower_rmsnorm(b, "ln_f", self.ln_f, x2d)
        elif self.ln_f is not None:
            h, mean, rstd = lower_layernorm(b, "ln_f", self.ln_f, x2d)
        else:
            h = x2d
        logits = b.act("logits", (T, Vp))
        lower_linear(b, "logits", self.lm_head, h, out=logits)
        out = logits.view(Bn, S, Vp)[..., :V]
        out._pp_padded = logits

        def bwd(dy, need_dx, dx_out):
            # dy is the padded [T, Vp] gradient buffer of the logits
            d_h = linear_backward(b, "lm_head", self.lm_head, h, dy.view(T, Vp), need_dx=need_dx,
                                  dx_out=(dx_out.view(T, Cc) if (dx_out is not None and self.ln_f is None)
                                          else None))
            if not need_dx:
                return None
            if self.ln_f is None:
                return d_h.view(Bn, S, Cc)
            dx_view = dx_out.view(T, Cc) if dx_out is not None else None
            if rms:
                dx = rmsnorm_backward(b, "ln_f", self.ln_f, x2d, rstd, d_h, dx_out=dx_view)
            else:
                dx = layernorm_backward(b, "ln_f", self.ln_f, x2d, mean, rstd, d_h, dx_out=dx_view)
            return dx.view(Bn, S, Cc)

        b.on_backward(bwd)
        return out


# ---- the same blocks around layers that a user's model already owns ---------------------------------
# A model written with plain torch layers (``nn.Embedding``, ``nn.LayerNorm``, ``nn.Linear``,
# ``F.scaled_dot_product_attention``, residual adds) is lowered by recognising these groupings in its
# graph and wrapping the user's own layer objects: no parameter is copied or renamed.
class InOutLinear(nn.Module):
    """A user's affine layer that stores its weight as [in, out] (``y = x W + b``; Hugging Face's
    ``Conv1D`` is one), presented with the attributes of ``nn.Linear``.  The layer object, its
    parameters and their names stay the user's; ``weight_in_out`` tells the lowering helpers which
    GEMM operand the stored matrix is."""

    weight_in_out = True

    def __init__(self, layer: nn.Module):
        super().__init__()
        self.layer = layer
        self.in_features, self.out_features = layer.weight.shape

    @property
    def weight(self):
        return self.layer.weight

    @property
    def bias(self):
        return self.layer.bias

    def forward(self, x):
        return self.layer(x)


def in_out_linear_like(m: nn.Module) -> bool:
    """Whether ``m`` is a leaf layer with a 2-d ``weight`` [in, out] and an optional 1-d ``bias`` whose
    forward is ``x W + b`` over the last dimension — decided by running it on a few random rows."""
    if isinstance(m, nn.Linear) or next(m.children(), None) is not None or next(m.buffers(), None) is not None:
        return False
    params = dict(m.named_parameters(recurse=False))
    w = params.get("weight")
    bias = params.get("bias", getattr(m, "bias", None))
    if w is None or w.dim() != 2 or set(params) - {"weight", "bias"} or (bias is not None and bias.dim() != 1):
        return False
    cached = getattr(m, "_pp_in_out_linear", None)
    if cached is not None:
        return cached
    try:
        with torch.no_grad():
            x = torch.randn(3, 2, w.shape[0], generator=torch.Generator().manual_seed(0)).to(w.device, w.dtype)
            got = m(x).float()
            want = x.float() @ w.float() + (bias.float() if bias is not None else 0.0)
            ok = got.shape == want.shape and bool((got - want).abs().max() <= 2e-2 * want.abs().max() + 1e-6)
    except Exception:
        ok = False
    try:
        m._pp_in_out_linear = ok
    except Exception:
        pass
    return ok


class RMSNormLike(nn.Module):
    """A user's root-mean-square norm layer of another library (one 1-d ``weight``, an epsilon attribute;
    Hugging Face's ``LlamaRMSNorm`` is one), presented with the attributes of ``nn.RMSNorm``."""

    def __init__(self, layer: nn.Module, eps: float):
        super().__init__()
        self.layer = layer
        self.eps = eps
        self.normalized_shape = tuple(layer.weight.shape)

    @property
    def weight(self):
        return self.layer.weight

    def forward(self, x):
        return self.layer(x)


def rms_norm_like(m: nn.Module) -> Optional[float]:
    """The epsilon of a leaf layer that computes ``weight * x / sqrt(mean(x^2) + eps)`` over the last
    dimension with its single 1-d parameter ``weight`` (decided by running it on a few random rows), else
    None.  ``nn.RMSNorm`` itself is not meant."""
    if isinstance(m, nn.RMSNorm) or next(m.children(), None) is not None or next(m.buffers(), None) is not None:
        return None
    params = dict(m.named_parameters(recurse=False))
    w = params.get("weight")
    if w is None or set(params) != {"weight"} or w.dim() != 1:
        return None
    cached = getattr(m, "_pp_rms_norm_like", 0)
    if cached != 0:
        return cached
    found = None
    for attr in ("eps", "variance_epsilon", "epsilon"):
        eps = getattr(m, attr, None)
        if not isinstance(eps, float):
            continue
        try:
            with torch.no_grad():
                x = torch.randn(3, 2, w.shape[0], generator=torch.Generator().manual_seed(0)).to(w.device, w.dtype)
                got = m(x).float()
                xf = x.float()
                want = w.float() * xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
                if got.shape == want.shape and bool((got - want).abs().max() <= 2e-2 * want.abs().max() + 1e-6):
                    found = eps
        except Exception:
            found = None
        break
    try:
        m._pp_rms_norm_like = found
    except Exception:
        pass
    return found


class LayerNormView(nn.LayerNorm):
    """An ``nn.LayerNorm`` around the parameters of a user's own layer-norm layer (the same parameter
    objects; a layer without a bias gives ``bias = None``)."""

    def __init__(self, weight: nn.Parameter, bias: Optional[nn.Parameter], eps: float):
        nn.Module.__init__(self)
        self.normalized_shape, self.eps, self.elementwise_affine = (weight.shape[0],), eps, True
        self.weight = weight
        if bias is None:
            self.register_parameter("bias", None)
        else:
            self.bias = bias


def layer_norm_like(m: nn.Module) -> Optional[LayerNormView]:
    """An ``nn.LayerNorm`` view of a leaf layer that is not one but computes one over the last dimension
    with its 1-d ``weight`` and optional 1-d ``bias`` (decided by running a float32 copy on rows of small
    variance, which also tells its epsilon: the attribute ``eps`` / ``variance_epsilon`` / ``epsilon`` if
    there is one, else 1e-5, 1e-6 or 1e-12), else None."""
    import copy
    if isinstance(m, (nn.LayerNorm, nn.RMSNorm)) or next(m.children(), None) is not None \
            or next(m.buffers(), None) is not None:
        return None
    params = dict(m.named_parameters(recurse=False))
    w, bias = params.get("weight"), params.get("bias")
    if w is None or not set(params) <= {"weight", "bias"} or w.dim() != 1 or (bias is not None and bias.shape != w.shape):
        return None
    cached = m.__dict__.get("_pp_layer_norm_like", 0)      # (kept out of the layer's registered submodules)
    if cached != 0:
        return cached
    found = None
    named = [getattr(m, a) for a in ("eps", "variance_epsilon", "epsilon") if isinstance(getattr(m, a, None), float)]
    try:
        probe = copy.deepcopy(m).float().cpu()
        pw, pb = probe.weight, getattr(probe, "bias", None)
        with torch.no_grad():
            g = torch.Generator().manual_seed(0)
            x = torch.randn(3, 2, w.shape[0], generator=g) * 1e-3 + torch.randn(3, 2, 1, generator=g)
            got = probe(x)
            for eps in named or (1e-5, 1e-6, 1e-12):
                want = F.layer_norm(x, (w.shape[0],), pw, pb, eps)
                if got.shape == want.shape and bool((got - want).abs().max() <= 1e-4 * want.abs().max() + 1e-7):
                    found = LayerNormView(w, bias, eps)
                    break
    except Exception:
        found = None
    m.__dict__["_pp_layer_norm_like"] = found
    return found


def _is_rms(norm) -> bool:
    return isinstance(norm, (nn.RMSNorm, RMSNormLike))


def activation_like(m: nn.Module) -> Optional[str]:
    """"relu", "gelu_tanh", "gelu_erf", "silu" or "identity" for a parameter-free leaf module that computes that
    function elementwise (decided on sample values: activation classes of model libraries qualify),
    else None."""
    if next(m.children(), None) is not None or next(m.parameters(), None) is not None \
            or next(m.buffers(), None) is not None:
        return None
    if isinstance(m, nn.Dropout):
        return "identity" if (m.p == 0.0 or not m.training) else None
    cached = getattr(m, "_pp_activation_like", 0)
    if cached != 0:
        return cached
    found = None
    try:
        with torch.no_grad():
            x = torch.linspace(-6.0, 6.0, 193).view(1, 1, -1)
            y = m(x)
            if torch.is_tensor(y) and y.shape == x.shape:
                for name in ("relu", "gelu_tanh", "gelu_erf", "silu", "identity"):
                    if (y - _torch_act(x, name if name != "identity" else None)).abs().max() <= 1e-5:
                        found = name
                        break
    except Exception:
        found = None
    try:
        m._pp_activation_like = found
    except Exception:
        pass
    return found


class WrappedTokenEmbedding(TokenEmbedding):
    def __init__(self, wte: nn.Embedding, wpe: Optional[nn.Embedding], position_offset: int = 0):
        NativeBlock.__init__(self)
        self.wte = wte
        self.wpe = wpe
        self.position_offset = position_offset


class WrappedEncoderEmbedding(EncoderEmbedding):
    def __init__(self, word: nn.Embedding, position: nn.Embedding, token_type: nn.Embedding, norm: nn.LayerNorm,
                 padding_positions: Optional[int] = None):
        NativeBlock.__init__(self)
        self.word_embeddings, self.position_embeddings, self.token_type_embeddings = word, position, token_type
        self.LayerNorm = norm
        self.padding_positions = padding_positions


class WrappedParallelLayer(NativeBlock):
    """A decoder layer whose attention and feed-forward read the same residual stream side by side
    (Falcon): ``x + o(attn(rope(qkv(ln_a(x))))) + fc2(act(fc1(ln_m(x))))`` around a user's layers.  ``qkv``
    is one fused projection, query heads first, then the key heads, then the value heads (fewer of them
    than query heads for multi-query / grouped-query attention); ``ln_m`` may be ``ln_a`` itself;
    ``cos`` / ``sin`` are the model's own rotary tables [positions, head_dim / 2]."""

    def __init__(self, ln_a: nn.LayerNorm, ln_m: nn.LayerNorm, qkv: nn.Linear, o_proj: nn.Linear, fc1: nn.Linear,
                 fc2: nn.Linear, n_heads: int, activation: str, cos: torch.Tensor, sin: torch.Tensor):
        super().__init__()
        assert activation in _ACT_DEPI and cos.shape == sin.shape
        self.dim, self.n_heads, self.activation = o_proj.out_features, n_heads, activation
        D = 2 * cos.shape[1]
        assert o_proj.in_features == n_heads * D
        self.head_dim = D
        self.n_kv_heads = (qkv.out_features // D - n_heads) // 2
        assert self.n_kv_heads > 0 and (n_heads + 2 * self.n_kv_heads) * D == qkv.out_features \
            and n_heads % self.n_kv_heads == 0
        self.ln_a, self.qkv, self.o_proj, self.fc1, self.fc2 = ln_a, qkv, o_proj, fc1, fc2
        if ln_m is not ln_a:
            self.ln_m = ln_m
        self._cos, self._sin = cos.detach().float().cpu().contiguous(), sin.detach().float().cpu().contiguous()
        import hashlib
        self._table_key = hashlib.sha1(self._cos.numpy().tobytes() + self._sin.numpy().tobytes()).hexdigest()[:16]

    def _ln_m(self):
        return getattr(self, "ln_m", None) or self.ln_a

    def _tables(self, seq, device):
        if seq > self._cos.shape[0]:
            raise RuntimeError(f"the model's rotary table covers {self._cos.shape[0]} positions, asked for {seq}")
        return self._cos[:seq].to(device), self._sin[:seq].to(device)

    # torch statement of the layer
    def forward(self, x):
        Bn, S, Cc = x.shape
        H, Hkv, D = self.n_heads, self.n_kv_heads, self.head_dim
        cos, sin = self._tables(S, x.device)
        q, k, v = self.qkv(self.ln_a(x)).split([H * D, Hkv * D, Hkv * D], dim=-1)
        q = q.reshape(Bn, S, H, D).transpose(1, 2)
        k, v = (t.reshape(Bn, S, Hkv, D).transpose(1, 2) for t in (k, v))
        q, k = _apply_rope(q, cos, sin), _apply_rope(k, cos, sin)
        if Hkv != H:
            k, v = (t.repeat_interleave(H // Hkv, dim=1) for t in (k, v))
        o = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        a = self.o_proj(o.transpose(1, 2).reshape(Bn, S, H * D))
        return x + a + self.fc2(_torch_act(self.fc1(self._ln_m()(x)), self.activation))

    def lower(self, b, x):
        if x.dim() != 3 or x.shape[-1] != self.dim:
            raise RuntimeError(f"{type(self).__name__} of width {self.dim} expects [batch, seq, dim], got "
                               f"{tuple(x.shape)}")
        Bn, S, Cc = x.shape
        T, H, Hkv, D = Bn * S, self.n_heads, self.n_kv_heads, self.head_dim
        x2d = x.view(T, Cc)
        ln_a, ln_m = self.ln_a, self._ln_m()
        shared = ln_m is ln_a
        act, dact = _ACT_EPI[self.activation], _ACT_DEPI[self.activation]
        cos = b.sp.shared(f"rope_cos:{S}:{D}:{self._table_key}", (S, D // 2), torch.float32)
        sin = b.sp.shared(f"rope_sin:{S}:{D}:{self._table_key}", (S, D // 2), torch.float32)
        c, s_ = self._tables(S, x.device)
        cos.copy_(c)
        sin.copy_(s_)
        na, mean_a, rstd_a = lower_layernorm(b, "na", ln_a, x2d)
        nm, mean_m, rstd_m = (na, mean_a, rstd_a) if shared else lower_layernorm(b, "nm", ln_m, x2d)
        qkv, _ = lower_linear(b, "qkv", self.qkv, na)
        b.f(P.op_rope(qkv, cos, sin, S, H + Hkv, D))
        att, attention_backward = lower_attention(b, qkv, Bn, S, H, True, n_kv_heads=Hkv)
        a, _ = lower_linear(b, "a", self.o_proj, att, epilogue=N.EPI_BIAS_RESIDUAL, aux_in=x2d)      # x + attention
        relu = self.activation == "relu"
        h, h_pre = lower_linear(b, "h", self.fc1, nm, epilogue=act, save_pre=b.training and not relu)
        if relu:
            h_pre = h
        y, _ = lower_linear(b, "y", self.fc2, h, epilogue=N.EPI_BIAS_RESIDUAL, aux_in=a)

        def bwd(dy, need_dx, dx_out):
            dy2d = dy.view(T, Cc)
            d_hpre = linear_backward(b, "fc2", self.fc2, h, dy2d, dx_epilogue=dact, dx_aux=h_pre)
            d_nm = linear_backward(b, "fc1", self.fc1, nm, d_hpre)
            d_att = linear_backward(b, "o", self.o_proj, att, dy2d)
            dqkv = attention_backward(d_att)
            b.i(P.op_rope(dqkv, cos, sin, S, H + Hkv, D, inverse=True))
            out = dx_out.view(T, Cc) if dx_out is not None else None
            if shared:
                # the two gradients of the one norm's output are added by the residual epilogue of the
                # second input-gradient GEMM
                d_n = linear_backward(b, "qkv", self.qkv, na, dqkv, dx_epilogue=N.EPI_BIAS_RESIDUAL, dx_aux=d_nm)
                dx = layernorm_backward(b, "na", ln_a, x2d, mean_a, rstd_a, d_n, dres=dy2d, dx_out=out)
            else:
                d_na = linear_backward(b, "qkv", self.qkv, na, dqkv)
                dx1 = layernorm_backward(b, "nm", ln_m, x2d, mean_m, rstd_m, d_nm, dres=dy2d)
                dx = layernorm_backward(b, "na", ln_a, x2d, mean_a, rstd_a, d_na, dres=dx1, dx_out=out)
            return dx.view(Bn, S, Cc)

        b.on_backward(bwd)
        return y.view(Bn, S, Cc)


class LinearView(nn.Linear):
    """An ``nn.Linear`` around parameters that a module keeps without a layer of their own (the packed
    q|k|v projection of ``nn.MultiheadAttention``): the same parameter objects, so names, gradients and
    optimizer state stay with the owner."""

    def __init__(self, weight: nn.Parameter, bias: Optional[nn.Parameter]):
        nn.Module.__init__(self)
        self.out_features, self.in_features = weight.shape
        self.weight = weight
        if bias is None:
            self.register_parameter("bias", None)
        else:
            self.bias = bias


def torch_encoder_layer_block(layer: nn.TransformerEncoderLayer, causal: bool = False) -> "WrappedTransformerLayer":
    """``nn.TransformerEncoderLayer`` (called with its input alone: no mask) as a transformer block around
    the layer's own parameters.  Raises ValueError with what keeps it from that."""
    att = layer.self_attn
    if not getattr(att, "batch_first", False):
        raise ValueError("nn.TransformerEncoderLayer with batch_first=False (sequence-major activations)")
    if not att._qkv_same_embed_dim or att.in_proj_weight is None or att.bias_k is not None or att.add_zero_attn:
        raise ValueError("nn.MultiheadAttention with separate key / value widths, bias_k / bias_v or add_zero_attn")
    drops = [layer.dropout, layer.dropout1, layer.dropout2]
    if (layer.training and any(d.p > 0 for d in drops)) or (att.dropout > 0 and layer.training):
        raise ValueError("dropout with p > 0 in training mode")
    act = layer.activation
    name = {F.relu: "relu", torch.relu: "relu"}.get(act)
    if name is None and act is F.gelu:
        name = "gelu_erf"
    if name is None and isinstance(act, nn.Module):
        name = activation_like(act)
    if name not in ("relu", "gelu_erf", "gelu_tanh"):
        raise ValueError(f"feed-forward activation {act!r} (ReLU, erf-GELU and tanh-GELU are built)")
    if any(not isinstance(n, nn.LayerNorm) or not n.elementwise_affine or n.bias is None for n in (layer.norm1, layer.norm2)):
        raise ValueError("norm layers other than affine LayerNorms with a bias")
    qkv = LinearView(att.in_proj_weight, att.in_proj_bias)
    return WrappedTransformerLayer(layer.norm1, qkv, att.out_proj, layer.norm2, layer.linear1, layer.linear2,
                                   att.num_heads, causal, name, pre_ln=bool(layer.norm_first))


class WrappedTransformerLayer(TransformerLayer):
    """``TransformerLayer`` around a user's layers.  ``c_attn`` is the fused q|k|v projection or the
    three separate ones; ``pre_ln=False`` is the encoder form, where ``ln_1`` / ``ln_2`` follow the two
    residual additions."""

    def __init__(self, ln_1: nn.LayerNorm, c_attn, c_proj: nn.Linear, ln_2: nn.LayerNorm,
                 c_fc: nn.Linear, mlp_proj: nn.Linear, n_heads: int, causal: bool, activation: str,
                 pre_ln: bool = True, attn_scale: Optional[float] = None, n_kv_heads: Optional[int] = None):
        NativeBlock.__init__(self)
        self.attn_scale = attn_scale
        self.n_kv_heads = n_kv_heads
        self.dim, self.n_heads, self.ffn = c_proj.out_features, n_heads, c_fc.out_features
        self.causal, self.pre_ln, self.activation = causal, pre_ln, activation
        self.ln_1, self.ln_2 = ln_1, ln_2
        self.attn = nn.Module()
        self.attn.c_proj = c_proj
        if isinstance(c_attn, (tuple, list)):
            self.attn.q, self.attn.k, self.attn.v = c_attn
            self._qkv = tuple(c_attn)
        else:
            self.attn.c_attn = c_attn
            self._qkv = (c_attn,)
        self.mlp = nn.Module()
        self.mlp.c_fc, self.mlp.c_proj = c_fc, mlp_proj

    def _qkv_layers(self):
        return self._qkv


class WrappedLlamaLayer(LlamaLayer):
    """``LlamaLayer`` around the layers of a user's model.  ``qkv`` is the fused q|k|v projection or the
    three separate ones (the Hugging Face Llama layout), ``gate_up`` the fused gate|up projection or
    the two separate ones.  Separate projections run as one forward GEMM over the arena's row-stacked
    copy of their weights; the gradient of their common input is one product with the transposed
    weights side by side; each weight gradient reads its column range of the output gradient."""

    def __init__(self, input_layernorm, qkv, o_proj, post_attention_layernorm, gate_up, down_proj,
                 n_heads: int, cos: torch.Tensor, sin: torch.Tensor, q_norm=None, k_norm=None):
        """``cos`` / ``sin``: the model's own rotary tables, [positions, head_dim / 2] (whatever base,
        scaling or rounding the model applies is in them); ``q_norm`` / ``k_norm``: RMS norms over each
        head's values of the queries / keys."""
        NativeBlock.__init__(self)
        self._init_attention(input_layernorm, qkv, o_proj, n_heads, cos, sin, q_norm, k_norm)
        self.post_attention_layernorm = post_attention_layernorm
        self._gate_up = tuple(gate_up) if isinstance(gate_up, (tuple, list)) else (gate_up,)
        self.ffn = down_proj.in_features
        assert sum(lin.out_features for lin in self._gate_up) == 2 * self.ffn
        self.mlp = nn.Module()
        if len(self._gate_up) == 2:
            self.mlp.gate_proj, self.mlp.up_proj = self._gate_up
        else:
            self.mlp.gate_up_proj = self._gate_up[0]
        self.mlp.down_proj = down_proj

    def _init_attention(self, input_layernorm, qkv, o_proj, n_heads, cos, sin, q_norm=None, k_norm=None):
        self._qkv = tuple(qkv) if isinstance(qkv, (tuple, list)) else (qkv,)
        self.dim, self.n_heads = o_proj.out_features, n_heads
        assert o_proj.in_features % n_heads == 0
        D = o_proj.in_features // n_heads
        self.head_dim = D if D * n_heads != self.dim else None
        if q_norm is not None:
            self.q_norm = q_norm
        if k_norm is not None:
            self.k_norm = k_norm
        assert cos.shape == sin.shape and cos.shape[1] == D // 2
        width = sum(lin.out_features for lin in self._qkv)
        self.n_kv_heads = (width // D - n_heads) // 2
        assert self.n_kv_heads > 0 and (n_heads + 2 * self.n_kv_heads) * D == width
        self.eps, self.rope_theta = input_layernorm.eps, None
        self._cos, self._sin = cos.detach().float().cpu().contiguous(), sin.detach().float().cpu().contiguous()
        import hashlib
        self._table_key = hashlib.sha1(self._cos.numpy().tobytes() + self._sin.numpy().tobytes()).hexdigest()[:16]
        self.input_layernorm = input_layernorm
        self.self_attn = nn.Module()
        if len(self._qkv) == 3:
            self.self_attn.q_proj, self.self_attn.k_proj, self.self_attn.v_proj = self._qkv
        else:
            self.self_attn.qkv_proj = self._qkv[0]
        self.self_attn.o_proj = o_proj

    def _rope(self, seq, head_dim, device):
        if seq > self._cos.shape[0] or head_dim != 2 * self._cos.shape[1]:
            raise RuntimeError(f"the model's rotary table covers {self._cos.shape[0]} positions of head size "
                               f"{2 * self._cos.shape[1]}, asked for {seq} of {head_dim}")
        return self._cos[:seq].to(device), self._sin[:seq].to(device)

    def _rope_key(self):
        return self._table_key

    def _project_qkv(self, h):
        return torch.cat([lin(h) for lin in self._qkv], dim=-1)

    def _lower_qkv(self, b, n1):
        if len(self._qkv) == 1:
            return lower_linear(b, "qkv", self._qkv[0], n1)[0]
        return lower_stacked_linears(b, "qkv", self._qkv, n1)

    def _qkv_backward(self, b, n1, dqkv):
        if len(self._qkv) == 1:
            return linear_backward(b, "qkv", self._qkv[0], n1, dqkv)
        d_n1 = b.grad("qkv.dx", (n1.shape[0], n1.shape[1]))
        b.i(P.op_gemm(dqkv, b.weight_t_cat(*(lin.weight for lin in self._qkv)), d_n1))
        lo = 0
        for name, lin in zip("qkv", self._qkv):
            linear_backward(b, name, lin, n1, dqkv[:, lo:lo + lin.out_features], need_dx=False)
            lo += lin.out_features
        return d_n1

    def _feed_forward(self, h):
        if len(self._gate_up) == 2:
            return super()._feed_forward(h)
        gate, up = self._gate_up[0](h).chunk(2, dim=-1)
        return self.mlp.down_proj(F.silu(gate) * up)

    def _lower_feed_forward(self, b, x2):
        if len(self._gate_up) == 2:
            return super()._lower_feed_forward(b, x2)
        # one [2 f, d] weight whose first f rows are the gate: both halves of the product come out of the
        # SwiGLU GEMM as they do for two weights, and the backward treats the pair as the one layer it is
        T, ffn, packed, down = x2.shape[0], self.ffn, self._gate_up[0], self.mlp.down_proj
        if x2.dtype != torch.bfloat16 or ffn % 8 or packed.bias is not None:
            raise RuntimeError("a fused gate|up projection lowers in bf16, without a bias, with a width that is a "
                               "multiple of 8")
        n2, rstd2 = lower_rmsnorm(b, "n2", self.post_attention_layernorm, x2)
        w = b.weight(packed.weight)
        gu = b.act("gu", (T, 2 * ffn))
        h = b.act("h", (T, ffn))
        b.f(P.op_gemm_swiglu(n2, w[:ffn], w[ffn:], gu, h))
        y, _ = lower_linear(b, "y", down, h, epilogue=N.EPI_BIAS_RESIDUAL, aux_in=x2)

        def backward(dy2d):
            dgu = b.grad("dgu", (T, 2 * ffn))
            b.i(P.op_gemm_dswiglu(dy2d, b.weight_t(down.weight), gu, dgu))
            d_n2 = linear_backward(b, "gate_up", packed, n2, dgu)
            linear_backward(b, "down", down, h, dy2d, need_dx=False)
            return rmsnorm_backward(b, "n2", self.post_attention_layernorm, x2, rstd2, d_n2, dres=dy2d)

        return y, backward


class RouterLayer(nn.Module):
    """An ``nn.Linear``-shaped view of a router module that holds its [experts, d] weight itself and
    does more than the projection in its forward (Hugging Face's ``MixtralTopKRouter``)."""

    bias = None

    def __init__(self, layer: nn.Module):
        super().__init__()
        self.layer = layer
        self.out_features, self.in_features = layer.weight.shape

    @property
    def weight(self):
        return self.layer.weight

    def forward(self, x):
        return F.linear(x, self.layer.weight)


class WrappedMoELayer(_MoEFeedForward, WrappedLlamaLayer):
    """A Mixtral-style layer around a user's model that keeps its experts stacked in two 3-d parameters
    (``gate_up`` [E, 2 f, d], ``down`` [E, d, f]) and its router weight in a module of its own: the
    attention half of ``WrappedLlamaLayer`` and the sparse feed-forward of ``MoELayer``, reading the
    expert matrices in place."""

    def __init__(self, input_layernorm, qkv, o_proj, post_attention_layernorm, router: nn.Module,
                 experts: nn.Module, gate_up: nn.Parameter, down: nn.Parameter, n_heads: int,
                 cos: torch.Tensor, sin: torch.Tensor):
        NativeBlock.__init__(self)
        self._init_attention(input_layernorm, qkv, o_proj, n_heads, cos, sin)
        self.post_attention_layernorm = post_attention_layernorm
        self.n_experts, self.ffn = gate_up.shape[0], down.shape[2]
        assert 2 <= self.n_experts <= 64
        self.mlp = nn.Module()
        self.mlp.router = RouterLayer(router)
        self.mlp.experts = experts      # the module that owns the two stacked parameters
        self._bank = _ExpertTensors(gate_up, down)
        self.forced_routing = None

    @property
    def _router(self):
        return self.mlp.router

    @property
    def _experts(self):
        return self._bank


class WrappedLMHead(LMHead):
    def __init__(self, ln_f: Optional[nn.Module], lm_head: nn.Linear):
        NativeBlock.__init__(self)
        self.dim, self.vocab = lm_head.in_features, lm_head.out_features
        self.ln_f = ln_f
        self.lm_head = lm_head


class StageSequence(nn.Module):
    """A stage module that applies its children in order.  Children keep the names they had in the
    un-split model (``add_block("transformer.h.3", layer)`` registers nested containers), so a
    stage's ``state_dict`` keys are a subset of the original model's."""

    def __init__(self):
        super().__init__()
        self._order: List[str] = []

    def add_block(self, fqn: str, module: nn.Module):
        parts = fqn.split(".")
        parent = self
        for p in parts[:-1]:
            if not hasattr(parent, p):
                parent.add_module(p, nn.Module())
            parent = getattr(parent, p)
        parent.add_module(parts[-1], module)
        self._order.append(fqn)

    def blocks(self) -> List[nn.Module]:
        return [self.get_submodule(f) for f in self._order]

    def forward(self, x):
        for blk in self.blocks():
            x = blk(x)
        return x
