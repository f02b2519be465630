"""Decides whether a stage module can run as HIP launch lists and, if so, as which blocks.

A stage lowers when it is a chain: its forward applies one lowerable piece after another to a
single tensor.  Lowerable pieces are the blocks of ``stage_modules`` and the standard torch layers
``nn.Linear`` (optionally followed by ReLU / GELU), ``nn.LayerNorm`` and ``nn.RMSNorm``.  A stage that is
not such a chain still lowers when its graph is a stack of transformer layers written with plain
layers (second half of this file): the GPT-2, BERT and Llama families, traced with ``torch.fx`` or
exported with ``torch.export``.  Anything else returns None and the stage runs through torch autograd
like the reference does.
"""
from __future__ import annotations

import operator
from typing import List, Optional, Tuple

import torch
import torch.fx as fx
import torch.nn as nn
import torch.nn.functional as F

from .stage_modules import (InOutLinear, LayerNormBlock, LinearAct, LinearView, NativeBlock, RMSNormBlock, RMSNormLike,
                            StageSequence, torch_encoder_layer_block, WrappedEncoderEmbedding, WrappedLlamaLayer, WrappedLMHead, WrappedMoELayer, WrappedParallelLayer,
                            WrappedTokenEmbedding,
                            WrappedTransformerLayer, activation_like, in_out_linear_like, layer_norm_like, rms_norm_like)

_LEAF_TYPES = (NativeBlock, nn.Linear, nn.LayerNorm, nn.RMSNorm, nn.ReLU, nn.GELU, nn.Identity, nn.Dropout,
               nn.Embedding)


class _ChainTracer(fx.Tracer):
    def is_leaf_module(self, m, qualname):
        return isinstance(m, _LEAF_TYPES + (nn.TransformerEncoderLayer,)) or in_out_linear_like(m) \
            or activation_like(m) is not None or layer_norm_like(m) is not None \
            or rms_norm_like(m) is not None or super().is_leaf_module(m, qualname)


def _as_linear(m: nn.Module) -> Optional[nn.Module]:
    """``m`` itself when it is an ``nn.Linear``, an ``nn.Linear``-shaped view of it when it is an affine
    layer with an [in, out] weight, else None."""
    if isinstance(m, nn.Linear):
        return m
    if in_out_linear_like(m):
        return InOutLinear(m)
    return None


def _layer_of(root: nn.Module, target: str) -> nn.Module:
    """The submodule ``target`` of ``root``, seen as the torch.nn layer it amounts to where it is a layer of
    another library (an affine layer with an [in, out] weight, an RMS norm, a layer norm)."""
    m = root.get_submodule(target)
    return _as_linear(m) or _as_rms_norm(m) or layer_norm_like(m) or m


def _as_rms_norm(m: nn.Module) -> Optional[nn.Module]:
    """``m`` itself when it is a usable ``nn.RMSNorm``, an ``nn.RMSNorm``-shaped view of it when it is a
    root-mean-square norm layer of another library, else None."""
    if isinstance(m, nn.RMSNorm):
        return m if (len(m.normalized_shape) == 1 and m.weight is not None and m.eps is not None) else None
    eps = rms_norm_like(m)
    return RMSNormLike(m, eps) if eps is not None else None


def _activation_of(node: fx.Node, root: nn.Module) -> Optional[str]:
    """Name of the activation a node applies, "identity" for a no-op, or None if it is neither."""
    if node.op == "call_function":
        if node.target in (torch.relu, F.relu, torch.nn.functional.relu):
            return "relu"
        if node.target is _ATEN.relu.default:
            return "relu"
        if node.target in (F.silu, _ATEN.silu.default):
            return "silu"
        if node.target in (F.gelu, _ATEN.gelu.default):
            approx = node.kwargs.get("approximate", "none")
            return "gelu_tanh" if approx == "tanh" else "gelu_erf"
    if node.op == "call_method" and node.target == "relu":
        return "relu"
    if node.op == "call_module":
        m = root.get_submodule(node.target)
        if isinstance(m, nn.ReLU):
            return "relu"
        if isinstance(m, nn.SiLU):
            return "silu"
        if isinstance(m, nn.GELU):
            return "gelu_tanh" if m.approximate == "tanh" else "gelu_erf"
        if isinstance(m, nn.Identity):
            return "identity"
        if isinstance(m, nn.Dropout) and (m.p == 0.0 or not m.training):
            return "identity"
        return activation_like(m)
    if node.op == "call_function" and node.target in _ATEN_DROPOUT:
        p_drop, train = node.args[1], node.args[2] if len(node.args) > 2 else True
        return "identity" if (p_drop == 0.0 or not train) else None
    return None


_ATEN = torch.ops.aten
_ATEN_DROPOUT = (_ATEN.dropout.default,)
# ATen-level nodes of an exported stage that only change how a tensor is viewed; the walk over the
# residual structure steps over them, and the numerical check of the recognised blocks covers them
_ATEN_VIEWS = (_ATEN.view.default, _ATEN.reshape.default, _ATEN._unsafe_view.default, _ATEN.slice.Tensor,
               _ATEN.contiguous.default, _ATEN.clone.default, _ATEN.alias.default, _ATEN.detach.default)


class NotLowerable(Exception):
    """Why a stage module cannot run as launch lists (the message names the construct)."""


def _chain_nodes(gm_graph: fx.Graph) -> Optional[List[fx.Node]]:
    """The compute nodes of a graph that is a pure chain (one placeholder, every node consuming
    exactly the previous node's value, the last one returned), else None."""
    placeholders = [n for n in gm_graph.nodes if n.op == "placeholder"]
    if len(placeholders) != 1:
        raise NotLowerable(f"the stage takes {len(placeholders)} inputs; a launch-list stage takes one tensor")
    prev = placeholders[0]
    chain = []
    for n in gm_graph.nodes:
        if n.op == "placeholder":
            continue
        if n.op == "output":
            out = n.args[0]
            if isinstance(out, (tuple, list)):
                if len(out) != 1:
                    return None
                out = out[0]
            return chain if out is prev else None
        tensor_args = [a for a in n.args if isinstance(a, fx.Node)]
        tensor_args += [a for a in n.kwargs.values() if isinstance(a, fx.Node)]
        if tensor_args != [prev] or len(prev.users) != 1:
            raise NotLowerable(f"node '{n.format_node()}' does not continue a chain of single-input layers "
                               "(branches, residual adds and multi-input ops need one of the blocks of "
                               "pippy_amd.stage_modules around them)")
        chain.append(n)
        prev = n
    return None


def blocks_from_graph(root: nn.Module, graph: fx.Graph) -> Optional[List[NativeBlock]]:
    nodes = _chain_nodes(graph)
    if nodes is None:
        raise NotLowerable("the stage does not return the value of its last layer")
    blocks: List[NativeBlock] = []
    i = 0
    while i < len(nodes):
        n = nodes[i]
        act = _activation_of(n, root)
        if act == "identity":
            i += 1
            continue
        if n.op != "call_module":
            raise NotLowerable(f"'{n.format_node()}' is not a module call or a supported activation")
        m = _layer_of(root, n.target)
        if isinstance(m, NativeBlock):
            blocks.append(m)
        elif isinstance(m, nn.TransformerEncoderLayer):
            blocks.append(_torch_layer(m, n, root))
        elif isinstance(m, (nn.Linear, InOutLinear)):
            nxt = _activation_of(nodes[i + 1], root) if i + 1 < len(nodes) else None
            if nxt == "silu":
                raise NotLowerable("a linear layer followed by SiLU outside a gated feed-forward")
            if nxt not in (None, "identity"):
                blocks.append(LinearAct(m, nxt))
                i += 1
            else:
                blocks.append(LinearAct(m, None))
        elif isinstance(m, nn.LayerNorm):
            if len(m.normalized_shape) != 1 or not m.elementwise_affine:
                raise NotLowerable(f"LayerNorm '{n.target}' normalises over {len(m.normalized_shape)} dimensions "
                                   "or has no affine parameters")
            blocks.append(LayerNormBlock(m))
        elif isinstance(m, nn.RMSNorm):
            if len(m.normalized_shape) != 1 or m.weight is None or m.eps is None:
                raise NotLowerable(f"RMSNorm '{n.target}' needs one normalised dimension, a weight and an eps")
            blocks.append(RMSNormBlock(m))
        elif isinstance(m, RMSNormLike):
            blocks.append(RMSNormBlock(m))
        else:
            # a user container (e.g. a block that wraps a linear and an activation): lower it as
            # a chain of its own and splice the result in
            blocks.extend(_lower(m))
        i += 1
    if not blocks:
        raise NotLowerable("the stage holds no layer")
    # a last projection onto a width that is no multiple of 8 (a vocabulary of 50257): the head block keeps
    # its weight rows and its output padded to one, which the GEMM and the loss kernel need
    last = blocks[-1]
    if type(last) is LinearAct and last.activation is None and isinstance(last.lin, nn.Linear) \
            and last.lin.weight.dtype == torch.bfloat16 and last.lin.out_features % 8:
        norm = None
        if len(blocks) > 1 and type(blocks[-2]) in (LayerNormBlock, RMSNormBlock):
            norm = blocks[-2].ln if type(blocks[-2]) is LayerNormBlock else blocks[-2].norm
        blocks = blocks[:-2 if norm is not None else -1] + [WrappedLMHead(norm, last.lin)]
    return blocks


def _torch_layer(m: nn.TransformerEncoderLayer, n: fx.Node, root: Optional[nn.Module] = None) -> NativeBlock:
    """torch's own encoder layer, called with its input alone or with a constant causal mask (a registered
    buffer: additive, or boolean with True for what is masked) and / or ``is_causal=True``."""
    given = dict(zip(("src", "src_mask", "src_key_padding_mask", "is_causal"), n.args))
    given.update(n.kwargs)
    causal = False
    if given.get("src_key_padding_mask") is not None:
        raise NotLowerable(f"'{n.format_node()}': an nn.TransformerEncoderLayer called with a padding mask")
    if given.get("src_mask") is not None:
        value = _constant_of(root, given["src_mask"]) if root is not None else None
        if value is not None and value.dtype == torch.bool:
            value = ~value
        if value is None or not _is_causal_mask(value):
            raise NotLowerable(f"'{n.format_node()}': an nn.TransformerEncoderLayer called with a mask that is not a "
                               "constant causal mask")
        causal = True
    elif given.get("is_causal"):
        raise NotLowerable(f"'{n.format_node()}': is_causal without the mask it describes")
    head = m.self_attn.embed_dim // m.self_attn.num_heads
    if head not in (64, 128):
        raise NotLowerable(f"nn.TransformerEncoderLayer '{n.target}' with head size {head} (64 and 128 are built)")
    try:
        block = torch_encoder_layer_block(m, causal)
        # like every recognised stage, the block is compared with what it stands for (fp32, on the host)
        import copy
        probe = copy.deepcopy(m).float().cpu().eval()
        x = torch.randn(2, 16, m.self_attn.embed_dim, generator=torch.Generator().manual_seed(0))
        mask = nn.Transformer.generate_square_subsequent_mask(16) if causal else None
        with torch.no_grad():
            want, got = probe(x, src_mask=mask), torch_encoder_layer_block(probe, causal)(x)
        err = (got - want).abs().max().item() / max(want.abs().max().item(), 1e-30)
    except ValueError as e:
        raise NotLowerable(f"nn.TransformerEncoderLayer '{n.target}': {e}") from None
    except Exception as e:
        raise NotLowerable(f"nn.TransformerEncoderLayer '{n.target}' could not be compared with its block "
                           f"({type(e).__name__}: {e})") from None
    if err > 1e-4:
        raise NotLowerable(f"nn.TransformerEncoderLayer '{n.target}': the block differs from the layer's own "
                           f"forward (relative error {err:.2e})")
    return block


def _lower(submod: nn.Module) -> List[NativeBlock]:
    if isinstance(submod, NativeBlock):
        return [submod]
    if isinstance(submod, StageSequence):
        out: List[NativeBlock] = []
        for child in submod.blocks():
            out.extend(_lower(child))
        if not out:
            raise NotLowerable("the stage holds no layer")
        return out
    if isinstance(submod, fx.GraphModule):
        try:
            return blocks_from_graph(submod, submod.graph)
        except NotLowerable as chain_reason:
            try:
                return blocks_from_residual_graph(submod)
            except NotLowerable as residual_reason:
                raise NotLowerable(f"as a stack of transformer layers: {residual_reason}; as a plain chain of layers: "
                                   f"{chain_reason}") from None
    if isinstance(submod, (nn.Linear, nn.LayerNorm, nn.RMSNorm)):
        # a stage that is one standard layer: the same rules as for that layer inside a chain
        holder = nn.Module()
        holder.layer = submod
        g = fx.Graph()
        g.output(g.call_module("layer", (g.placeholder("x"),)))
        return blocks_from_graph(holder, g)
    try:
        graph = _ChainTracer().trace(submod)
    except Exception as e:
        raise NotLowerable(f"torch.fx cannot trace {type(submod).__name__}: {type(e).__name__}: {e}") from e
    try:
        return blocks_from_graph(submod, graph)
    except NotLowerable as chain_reason:
        # not a chain of layers: maybe a transformer written with plain torch layers
        try:
            return blocks_from_residual_graph(submod)
        except NotLowerable as residual_reason:
            raise NotLowerable(f"as a stack of transformer layers: {residual_reason}; as a plain chain of layers: "
                                   f"{chain_reason}") from None


# ---- transformers written with plain torch layers ---------------------------------------------------
# Recognised, in this order along the stage:
#  * an optional embedding front: a token table, optionally plus a position table read at k .. k+S-1
#    (GPT-2; OPT reads from row 2 on), or word + position + token-type-0 tables, under a LayerNorm (BERT) or
#    not (a pre-LayerNorm encoder), the positions 0 .. S-1 or counted over the tokens that are not padding
#    (RoBERTa);
#  * any number of layers: a whole ``nn.TransformerEncoderLayer`` (batch first, no mask), or a residual
#    pair, attention then feed-forward, of one of these forms
#      pre-LayerNorm    x = x + proj(attn(qkv(ln(x))))                 x = x + fc2(act(fc1(ln(x))))
#      post-LayerNorm   x = ln(x + proj(attn(qkv(x))))                 x = ln(x + fc2(act(fc1(x))))
#      rotary, gated    x = x + o(attn(rope(q(n(x)), k(n(x))), v(n(x)))) x = x + down(silu(gate(n(x))) * up(n(x)))
#      side by side     x = x + o(attn(rope(qkv(ln(x))))) + fc2(act(fc1(ln'(x))))   (ln' = ln or a second LayerNorm)
#      rotary, experts  the same attention; x = x + (two of E gated experts per token, weights in stacked
#                       tensors, chosen by a softmax router)
#    where qkv is one fused projection or three separate ones; the affine layers are ``nn.Linear``, layers
#    with an [in, out] weight, or ``linear`` applied as a function to parameters; act is tanh-GELU,
#    erf-GELU or ReLU, as a function, a torch.nn module or a library's own activation class; n is an RMS
#    norm, and queries and keys may have an RMS norm over each head's values in front of the rotary
#    embedding; attn is ``scaled_dot_product_attention`` or softmax(q k^T c + mask) v spelled out, with
#    ``is_causal``, no mask, or a constant mask that is causal or masks nothing, and any constant factor
#    c on the scores (also applied to queries or keys beforehand); the rotary tables are constants of the
#    (exported) stage, and their width is the head size;
#  * an optional tail: norms and projections with activations, then a final norm and / or the vocabulary
#    projection.
# The walk only looks at which layers feed which residual add; how the model reshapes between them is
# not parsed but checked: the torch statement of the recognised blocks must reproduce the stage's own
# forward on a random input (fp32, on the host), otherwise the stage stays with torch autograd.
_SDPA = (F.scaled_dot_product_attention, _ATEN.scaled_dot_product_attention.default)
_ADD_FNS = (operator.add, operator.iadd, torch.add, _ATEN.add.Tensor, _ATEN.add_.Tensor)
_LINEAR_FNS = (_ATEN.linear.default,)      # an affine map written as a function of parameters
_ACT_FNS = (F.gelu, F.relu, torch.relu, F.silu, _ATEN.gelu.default, _ATEN.relu.default, _ATEN.silu.default)


def _is_add(n: fx.Node) -> bool:
    return (n.op == "call_function" and n.target in _ADD_FNS) or (n.op == "call_method" and n.target in ("add", "add_"))


def _branch_layers(y: fx.Node, stream: fx.Node, order: dict, state: bool = False) -> List[fx.Node]:
    """The layer and function nodes that ``y`` is computed from, back to ``stream`` (in graph order);
    with ``state`` also the ``get_attr`` nodes (parameters the model's own forward reads), top-k and
    softmax nodes."""
    seen, stack, found = set(), [y], []
    while stack:
        n = stack.pop()
        if n in seen or n is stream:
            continue
        seen.add(n)
        if n.op == "placeholder":
            continue
        if n.op == "call_module" or (n.op == "call_function" and n.target in _SDPA + _ACT_FNS + _LINEAR_FNS) \
                or _is_add(n):
            found.append(n)
        elif state and (n.op == "get_attr" or (n.op == "call_function" and
                                               n.target in (_ATEN.topk.default,) + _SOFTMAX)):
            found.append(n)
        stack.extend(a for a in n.all_input_nodes)
    return sorted(found, key=order.get)


def _constant_of(root: nn.Module, node, depth: int = 0) -> Optional[torch.Tensor]:
    """The tensor behind a ``get_attr`` node that reads a buffer or constant of ``root``, or what a few
    ATen operators make of such tensors (a mask cut out of a registered lower-triangular buffer and
    compared with zero: persistent buffers are not folded when a model is exported), else None."""
    if not isinstance(node, fx.Node):
        return None
    if node.op == "get_attr":
        obj = root
        try:
            for part in str(node.target).split("."):
                obj = getattr(obj, part)
        except AttributeError:
            return None
        return obj if torch.is_tensor(obj) and not isinstance(obj, nn.Parameter) else None
    if node.op != "call_function" or not isinstance(node.target, torch._ops.OpOverload) or depth > 16:
        return None
    op = node.target
    if op.namespace != "aten" or op._schema.is_mutable or torch.Tag.nondeterministic_seeded in op.tags:
        return None
    inputs = {}
    for a in node.all_input_nodes:
        value = _constant_of(root, a, depth + 1)
        if value is None or value.numel() > (1 << 26):
            return None
        inputs[a] = value
    if not inputs:
        return None
    try:
        with torch.no_grad():
            out = op(*fx.node.map_arg(node.args, lambda a: inputs[a]), **fx.node.map_arg(node.kwargs, lambda a: inputs[a]))
    except Exception:
        return None
    return out if torch.is_tensor(out) else None


def _parameter_of(root: nn.Module, node) -> Optional[nn.Parameter]:
    """The parameter behind a ``get_attr`` node of ``root``, else None."""
    if not isinstance(node, fx.Node) or node.op != "get_attr":
        return None
    obj = root
    try:
        for part in str(node.target).split("."):
            obj = getattr(obj, part)
    except AttributeError:
        return None
    return obj if isinstance(obj, nn.Parameter) else None


def _is_causal_mask(mask: torch.Tensor) -> bool:
    """A boolean (keep) or additive (0 / a huge negative number) mask, broadcast over batch and heads, that
    lets query i see exactly the keys 0..i."""
    if mask.dim() < 2 or mask.shape[-1] != mask.shape[-2]:
        return False
    S = mask.shape[-1]
    planes = mask.reshape(-1, S, S)
    if not bool((planes == planes[0]).all()):
        return False
    m = planes[0]
    keep = torch.ones(S, S, dtype=torch.bool, device=m.device).tril()
    if m.dtype == torch.bool:
        return bool((m == keep).all())
    if not m.dtype.is_floating_point:
        return False
    # -inf, the lowest value of some dtype (possibly of a narrower one than the tensor has now), -1e9,
    # -10000: addends under which exp() is zero in any precision
    masked = m <= -1e4
    return bool((masked == ~keep).all()) and bool((m[keep] == 0).all())


def _is_full_mask(mask: torch.Tensor) -> bool:
    """A boolean mask that keeps everything or an additive one that is zero everywhere."""
    return bool(mask.all()) if mask.dtype == torch.bool else bool((mask == 0).all())


_SOFTMAX = (_ATEN._softmax.default, _ATEN.softmax.int)
_MATMULS = (_ATEN.matmul.default, _ATEN.bmm.default, _ATEN.baddbmm.default)
_PASS_THROUGH = _ATEN_VIEWS + (_ATEN.transpose.int, _ATEN.permute.default, _ATEN.expand.default,
                               _ATEN._to_copy.default, _ATEN.to.dtype, _ATEN.to.dtype_layout,
                               _ATEN.unsqueeze.default, _ATEN.squeeze.dim, _ATEN.dropout.default)


def _scalar_of(root: nn.Module, arg) -> Optional[float]:
    """A Python number, or the value of a one-element constant tensor of the stage."""
    if isinstance(arg, (int, float)) and not isinstance(arg, bool):
        return float(arg)
    value = _constant_of(root, arg)
    if value is not None and value.numel() == 1 and (value.is_floating_point() or not value.dtype == torch.bool):
        return float(value)
    return None


def _constant_factors_back(root: nn.Module, node):
    """Walks from ``node`` towards its producer over views, casts and products / quotients with constants.
    Returns (the first node that is none of those, the accumulated factor)."""
    factor = 1.0
    while isinstance(node, fx.Node) and node.op == "call_function":
        if node.target in _PASS_THROUGH:
            node = node.args[0]
        elif node.target in (_ATEN.mul.Tensor, _ATEN.mul.Scalar, _ATEN.div.Tensor, _ATEN.div.Scalar) \
                and _scalar_of(root, node.args[1]) is not None:
            c = _scalar_of(root, node.args[1])
            factor = factor * c if "mul" in str(node.target) else factor / c
            node = node.args[0]
        else:
            break
    return node, factor


def _mask_is_causal(root: nn.Module, mask, causal: bool, inverted: bool = False) -> bool:
    """Folds a constant mask into ``causal``; raises for a mask that is neither causal nor empty."""
    value = _constant_of(root, mask)
    if value is not None and inverted and value.dtype == torch.bool:
        value = ~value
    if value is not None and _is_full_mask(value):
        return causal         # a mask that masks nothing (an encoder without padding)
    if value is None or not _is_causal_mask(value):
        raise NotLowerable("attention with a mask tensor other than a constant causal mask")
    return True               # (a model may apply its causal mask twice, as a selection and as an addend)


_WHOLE_ATTENTION = object()      # stands for the attention inside a call of nn.MultiheadAttention


def _check_whole_attention(att: nn.MultiheadAttention, n: fx.Node) -> None:
    """Raises unless the call ``n`` of ``att`` is plain self-attention over batch-first activations whose
    averaged weights nobody reads."""
    given = dict(zip(("query", "key", "value", "key_padding_mask", "need_weights", "attn_mask",
                      "average_attn_weights", "is_causal"), n.args))
    given.update(n.kwargs)
    if not (given.get("query") is given.get("key") is given.get("value")):
        raise NotLowerable(f"'{n.format_node()}': nn.MultiheadAttention on different query / key / value tensors")
    if given.get("key_padding_mask") is not None or given.get("attn_mask") is not None or given.get("is_causal"):
        raise NotLowerable(f"'{n.format_node()}': nn.MultiheadAttention with a mask that is not a constant of the stage")
    if not att.batch_first or not att._qkv_same_embed_dim or att.in_proj_weight is None or att.bias_k is not None \
            or att.add_zero_attn or (att.dropout > 0 and att.training):
        raise NotLowerable(f"nn.MultiheadAttention '{n.target}': sequence-major, separate key / value widths, "
                           "bias_k / bias_v, add_zero_attn or dropout")
    for user in n.users:
        first = user.op == "call_function" and user.target is operator.getitem and user.args[1] == 0
        if not first and user.users:
            raise NotLowerable(f"'{n.format_node()}': the attention weights of nn.MultiheadAttention are read")


def _attention_form(root: nn.Module, node: fx.Node):
    """(causal, (scale, factor)) of an attention, read off its scaled_dot_product_attention node or — for
    a model that spells attention out as softmax(q k^T * c + mask) v — off its softmax node.  ``scale`` is
    the explicit factor on the scores (None: the default 1 / sqrt(head size)), ``factor`` what the model
    multiplied queries and keys with beforehand.  Raises unless it is plain softmax attention, causal or
    full; whatever this reading misses shows when the recognised blocks are compared with the stage."""
    if node.op == "call_module":          # a whole nn.MultiheadAttention, checked by _check_whole_attention
        return False, (None, 1.0)
    if node.target in _SOFTMAX:
        causal, factor = False, 1.0
        x = node.args[0]
        while isinstance(x, fx.Node) and x.op == "call_function" and x.target not in _MATMULS:
            before, c = _constant_factors_back(root, x)
            if before is not x:
                x, factor = before, factor * c
            elif x.target is _ATEN.add.Tensor:
                causal = _mask_is_causal(root, x.args[1], causal)
                x = x.args[0]
            elif x.target is _ATEN.where.self:            # where(keep, scores, fill)
                causal = _mask_is_causal(root, x.args[0], causal)
                x = x.args[1]
            elif x.target in (_ATEN.masked_fill.Scalar, _ATEN.masked_fill.Tensor):   # fill where the mask is set
                causal = _mask_is_causal(root, x.args[1], causal, inverted=True)
                x = x.args[0]
            else:
                raise NotLowerable(f"'{x.format_node()}' between the score product and the softmax")
        if not (isinstance(x, fx.Node) and x.op == "call_function" and x.target in _MATMULS):
            raise NotLowerable("a softmax that does not follow a product of queries and keys")
        operands = x.args[:2]
        if x.target is _ATEN.baddbmm.default:      # mask + q k^T in one operator
            if x.kwargs.get("beta", 1) != 1 or x.kwargs.get("alpha", 1) != 1:
                raise NotLowerable(f"'{x.format_node()}' with factors of its own")
            causal = _mask_is_causal(root, x.args[0], causal)
            operands = x.args[1:3]
        for operand in operands:
            factor *= _constant_factors_back(root, operand)[1]
        return causal, (1.0, factor)
    names = ("query", "key", "value", "attn_mask", "dropout_p", "is_causal", "scale", "enable_gqa")
    given = dict(zip(names, node.args))
    given.update(node.kwargs)
    if given.get("dropout_p", 0.0) not in (0, 0.0) or given.get("enable_gqa"):
        raise NotLowerable("scaled_dot_product_attention with dropout or grouped queries")
    scale = given.get("scale")
    factor = 1.0
    if node.target in (_ATEN.scaled_dot_product_attention.default,):
        factor = _constant_factors_back(root, given["query"])[1] * _constant_factors_back(root, given["key"])[1]
    causal = bool(given.get("is_causal", False))
    if given.get("attn_mask") is not None:
        causal = _mask_is_causal(root, given["attn_mask"], causal)
    return causal, (None if scale is None else float(scale), factor)


def _score_factor(form, D: int) -> Optional[float]:
    """The factor on the scores for head size ``D``; None when it is the default 1 / sqrt(D)."""
    scale, factor = form
    total = (D ** -0.5 if scale is None else scale) * factor
    return None if abs(total - D ** -0.5) <= 1e-6 * D ** -0.5 else total


def _classify_expert_branch(root: nn.Module, norm, state: List[fx.Node]):
    """("mlp_moe", norm, router module, experts module, gate_up, down) for a feed-forward branch that reads
    a router weight [E, d] and two stacked expert parameters, gate|up [E, 2 f, d] and down [E, d, f], and
    picks two experts per token.  How the model routes and combines is not parsed: the block's own
    statement (softmax over all experts, top-2, renormalised) is compared with the stage numerically."""
    params, owners = [], {}
    for n in state:
        if n.op != "get_attr":
            continue
        path = str(n.target).split(".")
        try:
            owner = root.get_submodule(".".join(path[:-1]))
            value = getattr(owner, path[-1])
        except AttributeError:
            continue
        if isinstance(value, nn.Parameter) and id(value) not in owners:
            owners[id(value)] = owner
            params.append(value)
    top = [n for n in state if n.op == "call_function"]
    if len(top) != 1 or top[0].args[1] != 2:
        raise NotLowerable("a mixture-of-experts feed-forward that does not pick two experts per token")
    routers = [p for p in params if p.dim() == 2]
    stacked = [p for p in params if p.dim() == 3]
    if len(params) != 3 or len(routers) != 1 or len(stacked) != 2:
        raise NotLowerable("a mixture-of-experts feed-forward whose parameters are not a router weight and two "
                           "stacked expert tensors")
    router = routers[0]
    E, d = router.shape
    gate_up = next((p for p in stacked if p.shape[0] == E and p.shape[2] == d and p.shape[1] % 2 == 0), None)
    down = next((p for p in stacked if p is not gate_up), None)
    if gate_up is None or down is None or tuple(down.shape) != (E, d, gate_up.shape[1] // 2) or not 2 <= E <= 64:
        raise NotLowerable("stacked expert tensors that are not gate|up [E, 2 f, d] and down [E, d, f]")
    return ("mlp_moe", norm, owners[id(router)], owners[id(gate_up)], gate_up, down)


def _classify_branch(root: nn.Module, layers: List[fx.Node]):
    """What a residual branch is, from the layers between the stream and the addition:
    ("attn", ln, qkv, proj, causal) / ("mlp", ln, fc1, fc2, activation) for the GPT-2 and BERT families
    (ln is None when the branch does not start with a LayerNorm; qkv is one fused layer or three),
    ("attn_rope", norm, qkv, o) / ("mlp_gated", norm, gate_up, down) for the Llama family (qkv: the
    fused projection or the three separate ones; gate_up: the fused projection or the two separate ones)."""
    mods, inner_adds, state, soft = [], [], [], []
    for n in layers:
        if n.op == "get_attr" or (n.op == "call_function" and n.target is _ATEN.topk.default):
            state.append(n)
            continue
        if n.op == "call_function" and n.target in _SOFTMAX:
            soft.append(n)
            continue
        if _activation_of(n, root) == "identity":
            continue
        if n.op == "call_module" and isinstance(root.get_submodule(n.target), nn.MultiheadAttention):
            # torch's attention layer as one call: its packed projection, the attention, its output projection
            att = root.get_submodule(n.target)
            _check_whole_attention(att, n)
            mods += [(n, LinearView(att.in_proj_weight, att.in_proj_bias)), (n, _WHOLE_ATTENTION), (n, att.out_proj)]
        elif n.op == "call_module":
            mods.append((n, _layer_of(root, n.target)))
        elif n.op == "call_function" and n.target in _LINEAR_FNS:
            # (nn.MultiheadAttention applies its packed q|k|v parameters and its output projection this way)
            weight = _parameter_of(root, n.args[1])
            bias = _parameter_of(root, n.args[2]) if len(n.args) > 2 and n.args[2] is not None else None
            if weight is None or weight.dim() != 2 or (len(n.args) > 2 and n.args[2] is not None and bias is None):
                raise NotLowerable(f"'{n.format_node()}': a linear function of something other than parameters")
            mods.append((n, LinearView(weight, bias)))
        elif _is_add(n):
            if any(_constant_of(root, a) is not None for a in n.args[:2]):
                continue             # a constant added on (the mask of an attention that is spelled out)
            inner_adds.append(n)     # rotary embeddings add two products; nothing else may
        else:
            mods.append((n, None))

    def kind(n, m):
        if m is _WHOLE_ATTENTION:
            return "sdpa"
        if m is None:
            return "sdpa" if n.target in _SDPA + _SOFTMAX else "act"
        if isinstance(m, (nn.Linear, InOutLinear)):
            return "Linear"
        if isinstance(m, (nn.RMSNorm, RMSNormLike)):
            return "RMSNorm"
        if isinstance(m, nn.LayerNorm):
            return "LayerNorm"
        return "act" if _activation_of(n, root) is not None else type(m).__name__

    kinds = [kind(n, m) for n, m in mods]
    # (a router applied as a function of its weight is among the parameters the expert branch reads)
    modules = [(n, m) for n, m in mods if not isinstance(m, LinearView)]
    if [kind(n, m) for n, m in modules] == ["RMSNorm", "act"] and _activation_of(modules[1][0], root) == "silu":
        return _classify_expert_branch(root, modules[0][1], state)
    if len(soft) == 1 and kinds and set(kinds[1:]) == {"Linear"} and kinds[-1] == "Linear":
        # attention spelled out (softmax(q k^T) v between the projections): the softmax stands for the call
        mods.insert(len(mods) - 1, (soft[0], None))
        kinds.insert(len(kinds) - 1, "sdpa")
    head_norms = {}
    if kinds[:1] == ["RMSNorm"] and "sdpa" in kinds and kinds.count("RMSNorm") > 1:
        # RMS norms inside the branch: over the values of each head of the queries / keys, each fed (through
        # views) by the projection it belongs to
        for n, m in [x for x in mods[1:] if kind(*x) == "RMSNorm"]:
            src = _constant_factors_back(root, n.all_input_nodes[0])[0] if n.all_input_nodes else None
            if not (isinstance(src, fx.Node) and src.op == "call_module" and m.weight.shape[0] in (64, 128)):
                raise NotLowerable(f"a norm inside an attention branch that does not follow a projection "
                                   f"('{n.format_node()}')")
            head_norms[src] = m
            mods.remove((n, m))
        kinds = [kind(n, m) for n, m in mods]
    if kinds == ["RMSNorm", "Linear", "Linear", "Linear", "sdpa", "Linear"]:
        (_, norm), (qn, q), (kn, k), (vn, v), (sd, _), (_, o) = mods
        if not all(isinstance(lin, nn.Linear) for lin in (q, k, v, o)):
            raise NotLowerable("rotary attention whose projections keep [in, out] weights")
        if k.out_features != v.out_features or q.out_features != o.in_features or q.out_features % k.out_features:
            raise NotLowerable("query / key / value projections of unexpected widths")
        if set(head_norms) - {qn, kn}:
            raise NotLowerable("a per-head norm on something other than queries and keys")
        causal, form = _attention_form(root, sd)
        if not causal:
            raise NotLowerable("rotary attention that is not causal")
        return ("attn_rope", norm, (q, k, v), o, form, (head_norms.get(qn), head_norms.get(kn)))
    if head_norms:
        raise NotLowerable("per-head norms in an attention branch without separate query / key / value projections")
    norms = 2 if kinds[:2] == ["LayerNorm", "LayerNorm"] else 1
    if kinds[:norms] == ["LayerNorm"] * norms and kinds[norms:] == ["Linear", "sdpa", "Linear", "Linear", "act", "Linear"] \
            and inner_adds:
        # attention and feed-forward side by side on one stream (their sum is one of the inner additions,
        # the rotary embedding makes the others), behind one LayerNorm or one each
        (qn, qkv), (sd, _), (_, o), (fn, fc1), (an, _), (_, fc2) = mods[norms:]
        feeds = {node: m for node, m in mods[:norms]}
        ln_a = feeds.get(_constant_factors_back(root, qn.all_input_nodes[0])[0])
        ln_m = feeds.get(_constant_factors_back(root, fn.all_input_nodes[0])[0])
        act = _activation_of(an, root)
        if ln_a is None or ln_m is None or not all(isinstance(lin, nn.Linear) for lin in (qkv, o, fc1, fc2)) \
                or act not in ("gelu_tanh", "gelu_erf", "relu") or fc2.in_features != fc1.out_features:
            raise NotLowerable("attention and feed-forward side by side, but not as ln -> q|k|v -> attention -> o "
                               "next to ln -> fc1 -> GELU / ReLU -> fc2")
        causal, form = _attention_form(root, sd)
        if not causal:
            raise NotLowerable("rotary attention that is not causal")
        return ("parallel", ln_a, ln_m, qkv, o, fc1, fc2, act, form)
    if kinds == ["RMSNorm", "Linear", "sdpa", "Linear"] and inner_adds:
        (_, norm), (_, qkv), (sd, _), (_, o) = mods       # one fused q|k|v projection under a rotary embedding
        if not all(isinstance(lin, nn.Linear) for lin in (qkv, o)) or o.in_features != o.out_features \
                or qkv.out_features <= o.in_features or (qkv.out_features - o.in_features) % 2:
            raise NotLowerable("a fused projection in front of rotary attention that is not q|k|v")
        causal, form = _attention_form(root, sd)
        if not causal:
            raise NotLowerable("rotary attention that is not causal")
        return ("attn_rope", norm, qkv, o, form, (None, None))
    if kinds == ["RMSNorm", "Linear", "act", "Linear", "Linear"] or kinds == ["RMSNorm", "Linear", "Linear", "act", "Linear"]:
        norm, down = mods[0][1], mods[-1][1]
        an = next(n for n, m in mods if kind(n, m) == "act")
        if _activation_of(an, root) != "silu":
            raise NotLowerable(f"gated feed-forward with the activation '{an.format_node()}' (SiLU is built)")
        lins = {n: m for n, m in mods[1:-1] if kind(n, m) == "Linear"}
        gate_node = an.all_input_nodes[0] if an.all_input_nodes else None
        if gate_node not in lins or inner_adds:
            raise NotLowerable("a feed-forward that is not down(silu(gate(x)) * up(x))")
        gate = lins.pop(gate_node)
        up = next(iter(lins.values()))
        if any(lin.bias is not None or not isinstance(lin, nn.Linear) for lin in (gate, up, down)) or \
                gate.out_features != up.out_features or down.in_features != gate.out_features:
            raise NotLowerable("gated feed-forward projections with biases, [in, out] weights or unexpected widths")
        return ("mlp_gated", norm, (gate, up), down)
    if kinds == ["RMSNorm", "Linear", "act", "Linear"] and not inner_adds and \
            _activation_of(mods[2][0], root) == "silu":
        (_, norm), (_, packed), _, (_, down) = mods         # gate | up in one projection
        if not all(isinstance(lin, nn.Linear) and lin.bias is None for lin in (packed, down)) or \
                packed.out_features != 2 * down.in_features:
            raise NotLowerable("a SiLU feed-forward that is not down(silu(gate) * up) over a fused gate|up projection")
        return ("mlp_gated", norm, packed, down)
    if inner_adds:
        raise NotLowerable(f"an addition inside a residual branch ('{inner_adds[0].format_node()}')")
    ln = None
    if kinds and kinds[0] == "LayerNorm":      # pre-LayerNorm; without it the norm follows the addition
        ln, mods, kinds = mods[0][1], mods[1:], kinds[1:]
    if kinds == ["Linear", "sdpa", "Linear"]:
        (_, qkv), (sd, _), (_, proj) = mods
        d = qkv.in_features
        if proj.in_features != d or not d < qkv.out_features <= 3 * d or (qkv.out_features - d) % 2:
            raise NotLowerable("the projection in front of the attention is not a fused q|k|v projection (width 3 d, "
                               "or d + 2 k for fewer key / value heads)")
        return ("attn", ln, qkv, proj) + _attention_form(root, sd)
    if kinds == ["Linear", "Linear", "Linear", "sdpa", "Linear"]:
        (_, q), (_, k), (_, v), (sd, _), (_, proj) = mods
        if not all(isinstance(lin, nn.Linear) and lin.in_features == lin.out_features == proj.in_features
                   for lin in (q, k, v)):
            raise NotLowerable("separate query / key / value projections that are not d -> d nn.Linear layers")
        return ("attn", ln, (q, k, v), proj) + _attention_form(root, sd)
    if kinds == ["Linear", "act", "Linear"]:
        (_, fc1), (an, am), (_, fc2) = mods
        act = _activation_of(an, root)
        if act not in ("gelu_tanh", "gelu_erf", "relu"):
            raise NotLowerable(f"feed-forward activation '{an.format_node()}' (tanh-GELU, erf-GELU and ReLU are built)")
        if fc2.in_features != fc1.out_features or fc2.out_features != fc1.in_features:
            raise NotLowerable("feed-forward projections do not map d -> f -> d")
        return ("mlp", ln, fc1, fc2, act)
    raise NotLowerable(f"a residual branch made of {kinds}")


def _skip_identities(root: nn.Module, stream: fx.Node) -> fx.Node:
    """Steps over what does nothing behind ``stream``: a dropout with p = 0 or in eval mode, a re-view of
    the rows ([batch, seq, d] as [batch * seq, d] and back; the blocks work on rows either way, and the
    comparison with the stage checks the final shape)."""
    def passes(user: fx.Node) -> bool:
        if _activation_of(user, root) == "identity":
            return True
        return user.op == "call_function" and user.target in (_ATEN.view.default, _ATEN.reshape.default,
                                                              _ATEN._unsafe_view.default, _ATEN.alias.default)
    while len(stream.users) == 1 and passes(next(iter(stream.users))):
        stream = next(iter(stream.users))
    return stream


def _only_layer_user(root: nn.Module, node: fx.Node) -> Tuple[Optional[fx.Node], Optional[nn.Module]]:
    """(user, its module) when ``node`` feeds exactly one layer call, else (None, None)."""
    users = list(node.users)
    if len(users) == 1 and users[0].op == "call_module":
        return users[0], _layer_of(root, users[0].target)
    return None, None


def _embedding_front(root: nn.Module, nodes: List[fx.Node], order: dict, stream: fx.Node):
    """The embedding block at the head of a stage, if it has one: a lone token table, token + position
    tables (GPT-2), or word + position (+ token type 0) tables under a LayerNorm (the BERT family).
    Returns (blocks, the node that carries the residual stream from there on)."""
    emb = [n for n in nodes if n.op == "call_module" and isinstance(root.get_submodule(n.target), nn.Embedding)]
    if not emb:
        return [], stream
    ids = emb[0].all_input_nodes[0] if len(emb[0].all_input_nodes) == 1 else None
    while ids is not None and ids is not stream and ids.op == "call_function" and ids.target in _ATEN_VIEWS:
        ids = ids.args[0]   # an exported model may re-view its indices first ([-1, seq])
    if len(emb) > 3 or ids is not stream:
        raise NotLowerable("embedding tables other than a token table, a position table and a token-type table")
    wte = root.get_submodule(emb[0].target)
    if len(emb) == 1:
        return [WrappedTokenEmbedding(wte, None)], _skip_identities(root, emb[0])
    # the sum of all the look-ups: an addition fed by exactly these tables (and additions of them)
    joins = [n for n in nodes if _is_add(n) and set(_branch_layers(n, stream, order)) - {n} >= set(emb) and
             all(_is_add(x) or x in emb for x in _branch_layers(n, stream, order))]
    if not joins:
        raise NotLowerable("the embedding look-ups are not simply added")
    norm_node, norm = _only_layer_user(root, joins[0])
    if len(emb) == 2:
        position = root.get_submodule(emb[1].target)
        if isinstance(norm, nn.LayerNorm):      # an encoder front without token types
            return [WrappedEncoderEmbedding(wte, position, None, norm)], _skip_identities(root, norm_node)
        # positions 0 .. S-1 may read the table from a later row on (a constant index of k .. k+S-1)
        index = _constant_of(root, emb[1].all_input_nodes[0]) if len(emb[1].all_input_nodes) == 1 else None
        offset = 0
        if index is not None and index.dtype == torch.int64 and index.numel():
            rows = index.reshape(-1, index.shape[-1])
            offset = int(rows[0, 0])
            if offset < 0 or not bool((rows == torch.arange(rows.shape[1]) + offset).all()):
                raise NotLowerable("a position table that is not read at consecutive positions")
        return [WrappedTokenEmbedding(wte, position, offset)], _skip_identities(root, joins[0])
    # three tables: which is which shows in their constant index tensors (all zero: token type 0; 0 .. S-1: positions)
    # an index computed from the ids: positions counted over the tokens that are not padding, for a table
    # with a padding row; else taken for token type 0 (RoBERTa gathers it from a buffer of zeros at those
    # positions) — the comparison with the stage decides whether that reading holds
    roles, pad = {}, None
    for e in emb[1:]:
        index = _constant_of(root, e.all_input_nodes[0]) if len(e.all_input_nodes) == 1 else None
        if index is not None and index.dtype == torch.int64:
            if bool((index == 0).all()):
                roles["type"] = e
            elif bool((index.reshape(-1, index.shape[-1]) == torch.arange(index.shape[-1])).all()):
                roles["position"] = e
        elif index is None and len(e.all_input_nodes) == 1:
            table = root.get_submodule(e.target)
            if table.padding_idx is not None and "position" not in roles:
                roles["position"], pad = e, int(table.padding_idx)
            elif table.padding_idx is None and "type" not in roles:
                roles["type"] = e
    if len(roles) != 2:
        raise NotLowerable("three embedding tables that are not word + position + token type 0")
    if not isinstance(norm, nn.LayerNorm):      # (a pre-LayerNorm encoder normalises inside its layers)
        norm, norm_node = None, joins[0]
    block = WrappedEncoderEmbedding(wte, root.get_submodule(roles["position"].target),
                                    root.get_submodule(roles["type"].target), norm, padding_positions=pad)
    return [block], _skip_identities(root, norm_node)


def _layer_block(attention, attention_norm, feed_forward, feed_forward_norm, n_heads: int, rope) -> NativeBlock:
    """One transformer layer from its two classified branches (and, for post-LayerNorm layers, the
    LayerNorms that follow their additions)."""
    if (attention[0], feed_forward[0]) not in (("attn", "mlp"), ("attn_rope", "mlp_gated"), ("attn_rope", "mlp_moe")):
        raise NotLowerable(f"a '{attention[0]}' branch followed by a '{feed_forward[0]}' branch")
    d = attention[3].in_features
    if attention[0] == "attn_rope" and rope is not None:
        n_heads = max(1, d // (2 * rope[0].shape[1]))     # the table's width is the head size
    if d % n_heads or d // n_heads not in (64, 128):
        raise NotLowerable(f"head dimension {d}/{n_heads} (64 and 128 are built)")
    if feed_forward[0] == "mlp":
        _, ln1, qkv, proj, causal, form = attention
        _, ln2, fc1, fc2, act = feed_forward
        scale = _score_factor(form, d // n_heads)
        kv_heads = None
        if not isinstance(qkv, tuple) and qkv.out_features != 3 * d:      # multi-query / grouped-query q|k|v
            D = d // n_heads
            kv_heads = (qkv.out_features - d) // (2 * D)
            if kv_heads < 1 or kv_heads * 2 * D != qkv.out_features - d or n_heads % kv_heads:
                raise NotLowerable(f"a fused projection of width {qkv.out_features} that is not {n_heads} query heads "
                                   f"plus whole key / value heads of size {D}")
        if (ln1 is None) != (ln2 is None) or (ln1 is None) != (attention_norm is not None) \
                or (ln2 is None) != (feed_forward_norm is not None):
            raise NotLowerable("a layer that is neither pre-LayerNorm nor post-LayerNorm throughout")
        if ln1 is None:
            return WrappedTransformerLayer(attention_norm, qkv, proj, feed_forward_norm, fc1, fc2, n_heads, causal,
                                           act, pre_ln=False, attn_scale=scale, n_kv_heads=kv_heads)
        return WrappedTransformerLayer(ln1, qkv, proj, ln2, fc1, fc2, n_heads, causal, act, attn_scale=scale,
                                       n_kv_heads=kv_heads)
    _, norm1, qkv, o, form, (q_norm, k_norm) = attention
    width = sum(lin.out_features for lin in qkv) if isinstance(qkv, tuple) else qkv.out_features
    D = d // n_heads
    if _score_factor(form, D) is not None:
        raise NotLowerable(f"rotary attention with the score factor {_score_factor(form, D):.6g} (1 / sqrt(head "
                           f"size) is built)")
    if width % D or (width // D - n_heads) % 2 or width // D <= n_heads:
        raise NotLowerable("query / key / value projections that are not whole heads")
    if rope is None:
        raise NotLowerable("rotary attention, but the stage holds no constant cos / sin table of the positions "
                           "(exported models do)")
    if feed_forward[0] == "mlp_moe":
        _, norm2, router, experts, gate_up, down = feed_forward
        if q_norm is not None or k_norm is not None:
            raise NotLowerable("per-head norms in a mixture-of-experts layer")
        return WrappedMoELayer(norm1, qkv, o, norm2, router, experts, gate_up, down, n_heads, *rope)
    _, norm2, gate_up, down = feed_forward
    return WrappedLlamaLayer(norm1, qkv, o, norm2, gate_up, down, n_heads, *rope, q_norm=q_norm, k_norm=k_norm)


def _tail_blocks(root: nn.Module, stream: fx.Node, result: fx.Node, after_layers: bool) -> List[NativeBlock]:
    """What follows the last residual addition must be a chain: projections with activations, a final
    norm, the vocabulary projection."""
    tail, cur = [], stream
    while cur is not result:
        users = list(cur.users)
        if len(users) != 1:
            raise NotLowerable(f"'{cur.format_node()}' feeds {len(users)} nodes after the last residual addition")
        cur = users[0]
        if cur.op == "output":
            break
        tail.append(cur)
    mods = []
    for n in tail:
        act = _activation_of(n, root)
        if act == "identity" or (n.op == "call_function" and n.target in _ATEN_VIEWS):
            continue
        if act in ("relu", "gelu_tanh", "gelu_erf") and mods and isinstance(mods[-1], (nn.Linear, InOutLinear)):
            mods[-1] = LinearAct(mods[-1], act)     # a projection with its activation
            continue
        if n.op != "call_module":
            raise NotLowerable(f"'{n.format_node()}' after the last residual addition")
        mods.append(_layer_of(root, n.target))
    blocks: List[NativeBlock] = []
    head: List[NativeBlock] = []
    norm_types, linear_types = (nn.LayerNorm, nn.RMSNorm, RMSNormLike), (nn.Linear, InOutLinear)
    # the chain ends in a norm and a projection (a language-model head; in front of it there may be the
    # last norm of a pre-LayerNorm encoder and the transform of a masked-language-model head), or in a
    # projection without a bias behind nothing but projections with activations
    if len(mods) >= 2 and isinstance(mods[-2], norm_types) and isinstance(mods[-1], nn.Linear):
        head, mods = [WrappedLMHead(mods[-2], mods[-1])], mods[:-2]
    elif mods and isinstance(mods[-1], nn.Linear) and mods[-1].bias is None and (after_layers or len(mods) > 1) \
            and all(isinstance(m, LinearAct) for m in mods[:-1]):
        head, mods = [WrappedLMHead(None, mods[-1])], mods[:-1]
    for m in mods:
        if isinstance(m, nn.LayerNorm):
            blocks.append(LayerNormBlock(m))
        elif isinstance(m, (nn.RMSNorm, RMSNormLike)):
            blocks.append(RMSNormBlock(m))
        elif isinstance(m, linear_types):
            blocks.append(LinearAct(m, None))
        elif isinstance(m, LinearAct):
            blocks.append(m)
        else:
            raise NotLowerable(f"a {type(m).__name__} after the last residual addition")
    return blocks + head


def _residual_blocks(root: nn.Module, graph: fx.Graph, n_heads: int, rope=None) -> List[NativeBlock]:
    """The blocks of a stage that is an embedding front, residual layers and a tail (each optional except
    that there must be a layer).  ``rope``: the (cos, sin) tables of rotary layers."""
    nodes = list(graph.nodes)
    order = {n: i for i, n in enumerate(nodes)}
    placeholders = [n for n in nodes if n.op == "placeholder"]
    if len(placeholders) != 1:
        raise NotLowerable(f"the stage takes {len(placeholders)} inputs; a launch-list stage takes one tensor")
    result = next(n for n in nodes if n.op == "output").args[0]
    if isinstance(result, (tuple, list)):
        if len(result) != 1:
            raise NotLowerable("the stage returns several values")
        result = result[0]
    blocks, stream = _embedding_front(root, nodes, order, placeholders[0])
    # residual pairs: the stream feeds one addition whose other operand is a branch computed from the stream
    attention = attention_norm = None
    while True:
        whole = next(iter(stream.users)) if len(stream.users) == 1 else None
        if whole is not None and whole.op == "call_module" and attention is None and \
                isinstance(root.get_submodule(whole.target), nn.TransformerEncoderLayer):
            blocks.append(_torch_layer(root.get_submodule(whole.target), whole, root))    # a layer of torch's own
            stream = _skip_identities(root, whole)
            continue
        adds = [u for u in stream.users if _is_add(u)]
        if len(adds) != 1:
            break
        add = adds[0]
        other = [a for a in add.all_input_nodes if a is not stream]
        if len(other) != 1:
            break
        kind = _classify_branch(root, _branch_layers(other[0], stream, order, state=True))
        # post-LayerNorm layers: the sum goes through a LayerNorm before anything else reads it
        post_norm, after = None, add
        if kind[0] in ("attn", "mlp") and kind[1] is None:
            after, post_norm = _only_layer_user(root, add)
            if not isinstance(post_norm, nn.LayerNorm):
                raise NotLowerable("a residual branch without a LayerNorm before it or after its addition")
        if kind[0] == "parallel":
            if attention is not None:
                raise NotLowerable("an attention branch without its feed-forward branch before a side-by-side layer")
            _, ln_a, ln_m, qkv, o, fc1, fc2, act, form = kind
            if rope is None:
                raise NotLowerable("rotary attention, but the stage holds no constant cos / sin table of the positions")
            D = 2 * rope[0].shape[1]
            if o.in_features % D or _score_factor(form, D) is not None:
                raise NotLowerable("a side-by-side layer whose heads do not match the rotary table, or with a score "
                                   "factor other than 1 / sqrt(head size)")
            heads = o.in_features // D
            if qkv.out_features % D or (qkv.out_features // D - heads) % 2 or qkv.out_features // D <= heads \
                    or heads % ((qkv.out_features // D - heads) // 2):
                raise NotLowerable("a fused projection that is not whole query, key and value heads")
            blocks.append(WrappedParallelLayer(ln_a, ln_m, qkv, o, fc1, fc2, heads, act, *rope))
            stream = _skip_identities(root, add)
            continue
        if kind[0] in ("attn", "attn_rope"):
            if attention is not None:
                raise NotLowerable("two attention branches in a row")
            attention, attention_norm = kind, post_norm
        else:
            if attention is None:
                raise NotLowerable("a feed-forward branch without an attention branch before it")
            blocks.append(_layer_block(attention, attention_norm, kind, post_norm, n_heads, rope))
            attention = None
        stream = _skip_identities(root, after)
    if attention is not None:
        raise NotLowerable("an attention branch without its feed-forward branch in the same stage")
    if not any(isinstance(b, (WrappedTransformerLayer, WrappedLlamaLayer, WrappedParallelLayer)) for b in blocks):
        raise NotLowerable("no attention / feed-forward residual pair found")
    return blocks + _tail_blocks(root, stream, result, after_layers=True)


def _example_input(blocks: List[NativeBlock], shape=None, seq: int = 16) -> torch.Tensor:
    """A random stage input; ``shape`` is given for exported stages, whose graphs hold the sizes of the
    example microbatch; ``seq``: the sequence length otherwise (a stage that holds a square mask runs at
    that mask's size only)."""
    g = torch.Generator().manual_seed(0)
    first = blocks[0]
    if isinstance(first, WrappedTokenEmbedding):
        seq = seq if first.wpe is None else min(seq, first.wpe.num_embeddings)
        return torch.randint(0, first.wte.num_embeddings, shape or (2, seq), generator=g)
    if isinstance(first, WrappedEncoderEmbedding):
        seq = min(seq, first.position_embeddings.num_embeddings)
        x = torch.randint(0, first.word_embeddings.num_embeddings, shape or (2, seq), generator=g)
        if first.padding_positions is not None:      # some padding, so that its handling is compared too
            x[0, :1] = first.padding_positions
            x[-1, x.shape[1] // 2:] = first.padding_positions
        return x
    d = next(b for b in blocks if isinstance(b, (WrappedTransformerLayer, WrappedLlamaLayer, WrappedParallelLayer))).dim
    return torch.randn(shape or (2, seq, d), generator=g)


def _rotary_tables(submod: nn.Module, d: int):
    """(heads, (cos, sin)) read off the constants of an exported stage: two [.., positions, head_dim]
    tensors whose halves repeat, whose squares add up to one and which are 1 and 0 at position 0.  The
    tables are taken as the model made them (its base, scaling and rounding).  None when there are none."""
    tables = []
    for _, t in submod.named_buffers():
        if not t.is_floating_point() or t.dim() < 2 or t.shape[-1] not in (64, 128) or d % t.shape[-1]:
            continue
        D, S = t.shape[-1], t.shape[-2]
        planes = t.detach().float().cpu().reshape(-1, S, D)
        if bool((planes == planes[0]).all()) and bool((planes[0][:, :D // 2] == planes[0][:, D // 2:]).all()):
            tables.append(planes[0][:, :D // 2])
    for c in tables:
        for s_ in tables:
            if c.shape == s_.shape and bool((c[0] == 1).all()) and bool((s_[0] == 0).all()) \
                    and bool(((c * c + s_ * s_) - 1).abs().max() <= 2e-2):
                return d // (2 * c.shape[1]), (c, s_)
    return None


def blocks_from_residual_graph(submod: nn.Module) -> List[NativeBlock]:
    """Blocks of a stage that is a stack of plain-torch transformer layers, verified numerically."""
    import copy
    shape = None
    if isinstance(submod, fx.GraphModule):
        inputs = [n for n in submod.graph.nodes if n.op == "placeholder"]
        if len(inputs) == 1 and hasattr(inputs[0].meta.get("val"), "shape"):
            shape = tuple(int(s) for s in inputs[0].meta["val"].shape)
    try:
        graph = _ChainTracer().trace(submod)
    except Exception as e:
        raise NotLowerable(f"torch.fx cannot trace {type(submod).__name__}: {type(e).__name__}: {e}") from e
    widths = {m.normalized_shape[0] for m in submod.modules()
              if isinstance(m, (nn.LayerNorm, nn.RMSNorm)) and len(m.normalized_shape) == 1}
    widths |= {m.weight.shape[0] for m in submod.modules() if rms_norm_like(m) is not None or layer_norm_like(m) is not None}
    if len(widths) > 1 and all(w in (64, 128) for w in widths - {max(widths)}):
        widths = {max(widths)}       # (norms over the values of one head, on queries and keys)
    if len(widths) != 1:
        raise NotLowerable("no single model width (the normalisation layers of the stage disagree)")
    d = widths.pop()
    candidates = [h for h in (d // 64, d // 128) if h >= 1 and d % h == 0]
    if not candidates:
        raise NotLowerable(f"model width {d} allows no head dimension of 64 or 128")
    rotary = _rotary_tables(submod, d)
    if rotary is not None:
        candidates = [rotary[0]]      # the table's width is the head size
    rope = rotary[1] if rotary is not None else None
    _residual_blocks(submod, graph, candidates[0], rope)   # raises unless the structure is recognised
    # the structure fits; which head count (if any) reproduces the stage is decided on an fp32 copy
    try:
        probe = copy.deepcopy(submod).float().cpu().eval()
    except Exception as e:
        raise NotLowerable(f"the stage module cannot be copied for verification: {e}") from e
    _widen_baked_casts(probe)
    # a mask kept as a buffer of fixed size (a traced model that hands it to its layers) fixes the length
    square = [t.shape[-1] for _, t in submod.named_buffers() if t.dim() >= 2 and t.shape[-1] == t.shape[-2] > 1
              and (t.dtype == torch.bool or t.is_floating_point())]
    seq = min(square) if square and shape is None else 16
    probe_graph = _ChainTracer().trace(probe)
    tolerance = 1e-4
    reasons = []
    for n_heads in candidates:
        trial = _residual_blocks(probe, probe_graph, n_heads, rope)
        x = _example_input(trial, shape, seq)
        try:
            with torch.no_grad():
                want = probe(x)
                got = x
                for blk in trial:
                    got = blk(got)
        except Exception as e:
            raise NotLowerable(f"the recognised blocks could not be compared with the stage's own forward "
                               f"({type(e).__name__}: {e})") from e
        if isinstance(want, (tuple, list)):
            want = want[0]
        err = (got - want).abs().max().item() / max(want.abs().max().item(), 1e-30) if got.shape == want.shape else 1.0
        if err <= tolerance:
            return _residual_blocks(submod, graph, n_heads, rope)
        reasons.append(f"with {n_heads} heads the recognised blocks differ from the stage's own forward "
                       f"(relative error {err:.2e})")
    raise NotLowerable("; ".join(reasons))


def _widen_baked_casts(probe: nn.Module) -> None:
    """A model exported in bf16 / fp16 holds the casts its forward made to "the input's dtype" as casts to
    that dtype.  On the fp32 copy that the recognised blocks are compared with they would round where
    nothing else does: they become casts to fp32."""
    if not isinstance(probe, fx.GraphModule):
        return
    low = (torch.bfloat16, torch.float16)
    changed = False
    for n in probe.graph.nodes:
        if n.op != "call_function":
            continue
        if n.target is _ATEN.to.dtype and len(n.args) > 1 and n.args[1] in low:
            n.args = (n.args[0], torch.float32) + tuple(n.args[2:])
            changed = True
        elif n.target in (_ATEN._to_copy.default, _ATEN.to.dtype_layout) and n.kwargs.get("dtype") in low:
            n.kwargs = {**n.kwargs, "dtype": torch.float32}
            changed = True
    if changed:
        probe.recompile()


def _check_kernel_requirements(submod: nn.Module, blocks: List[NativeBlock]) -> None:
    """What the kernels need beyond a recognised structure.  Launch lists compute in the parameter
    dtype: the MFMA kernels (GEMM epilogues beyond bias / ReLU, attention, norms, embeddings) are bf16,
    float32 stages can only be chains of ``nn.Linear`` with no activation or ReLU."""
    dtypes = {p.dtype for p in submod.parameters()}
    if len(dtypes) > 1:
        raise NotLowerable(f"parameters of several dtypes ({sorted(str(d) for d in dtypes)}); a launch-list stage "
                           "keeps one")
    if dtypes and dtypes != {torch.bfloat16} and dtypes != {torch.float32}:
        raise NotLowerable(f"parameters of dtype {dtypes.pop()} (bfloat16 and float32 are built)")
    for blk in blocks if dtypes == {torch.float32} else ():
        plain = isinstance(blk, LinearAct) and isinstance(blk.lin, nn.Linear) and blk.activation in (None, "relu")
        if not plain:
            raise NotLowerable(f"float32 parameters: {type(blk).__name__} runs as bfloat16 kernels only (convert the "
                               "model with .to(torch.bfloat16) to run it as launch lists)")
    if dtypes == {torch.bfloat16}:
        # the bf16 kernels move 16-byte groups: widths are multiples of 8, except where a block keeps a
        # weight's rows padded (a vocabulary projection, a router)
        padded = set()
        for blk in blocks:
            for m in blk.modules():
                padded |= {id(p) for p, _ in getattr(m, "_pp_padded_rows", lambda: [])()}
        for blk in blocks:
            for name, m in blk.named_modules():
                if isinstance(m, (nn.Linear, InOutLinear)):
                    widths = [("in", m.in_features)] + ([] if id(m.weight) in padded else [("out", m.out_features)])
                elif isinstance(m, (nn.LayerNorm, nn.Embedding)):
                    widths = [("", m.weight.shape[-1])] if getattr(m, "weight", None) is not None else []
                else:
                    continue
                for which, w in widths:
                    if w % 8:
                        raise NotLowerable(f"{type(m).__name__} '{name}' of {type(blk).__name__} has {which + ' ' if which else ''}"
                                           f"width {w}; the bfloat16 kernels take multiples of 8")


def lower_stage_module(submod: nn.Module, why: Optional[List[str]] = None, for_kernels: bool = False) -> Optional[List[NativeBlock]]:
    """Blocks of a lowerable stage module, or None when it has to run eagerly; the reason is then
    appended to ``why``.  ``for_kernels`` also requires what the kernels need of dtypes and (known) shapes;
    the stage runtime asks for it, recognising the structure of a model does not depend on it."""
    try:
        blocks = _lower(submod)
        if for_kernels:
            _check_kernel_requirements(submod, blocks)
        return blocks
    except NotLowerable as e:
        if why is not None:
            reason = str(e)
            # the most common cause, and one that the structural messages do not name: a dropout that does
            # something keeps its residual branch from being recognised
            live = [n for n, m in submod.named_modules()
                    if (isinstance(m, nn.modules.dropout._DropoutNd) and m.p > 0 and m.training)
                    or (isinstance(m, nn.MultiheadAttention) and m.dropout > 0 and m.training)]
            if live and "dropout" not in reason:
                shown = ", ".join(live[:3]) + (", ..." if len(live) > 3 else "")
                reason = (f"dropout with p > 0 in training mode ({shown}): the launch lists hold no dropout; "
                          f"set p = 0 or build the stage in eval mode.  The recogniser says: {reason}")
            why.append(reason)
        return None
