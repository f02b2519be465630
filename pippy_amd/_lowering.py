"""Decides whether a stage module can run as HIP launch lists and, if so, as which blocks.

A stage lowers when it is a chain: its forward applies one lowerable piece after another to a
single tensor.  Lowerable pieces are the blocks of ``stage_modules`` and the standard torch layers
``nn.Linear`` (optionally followed by ReLU / GELU), ``nn.LayerNorm`` and ``nn.RMSNorm``.  Anything else returns
None and the stage runs through torch autograd like the reference does.
"""
from __future__ import annotations

import operator
from typing import List, Optional

import torch
import torch.fx as fx
import torch.nn as nn
import torch.nn.functional as F

from .stage_modules import LayerNormBlock, LinearAct, NativeBlock, RMSNormBlock, StageSequence

_LEAF_TYPES = (NativeBlock, nn.Linear, nn.LayerNorm, nn.RMSNorm, nn.ReLU, nn.GELU, nn.Identity, nn.Dropout)


class _ChainTracer(fx.Tracer):
    def is_leaf_module(self, m, qualname):
        return isinstance(m, _LEAF_TYPES) or super().is_leaf_module(m, qualname)


def _activation_of(node: fx.Node, root: nn.Module) -> Optional[str]:
    """Name of the activation a node applies, "identity" for a no-op, or None if it is neither."""
    if node.op == "call_function":
        if node.target in (torch.relu, F.relu, torch.nn.functional.relu):
            return "relu"
        if node.target is F.gelu:
            approx = node.kwargs.get("approximate", "none")
            return "gelu_tanh" if approx == "tanh" else "gelu_erf"
    if node.op == "call_method" and node.target == "relu":
        return "relu"
    if node.op == "call_module":
        m = root.get_submodule(node.target)
        if isinstance(m, nn.ReLU):
            return "relu"
        if isinstance(m, nn.GELU):
            return "gelu_tanh" if m.approximate == "tanh" else "gelu_erf"
        if isinstance(m, nn.Identity):
            return "identity"
        if isinstance(m, nn.Dropout) and (m.p == 0.0 or not m.training):
            return "identity"
    return None


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
        m = root.get_submodule(n.target)
        if isinstance(m, NativeBlock):
            blocks.append(m)
        elif isinstance(m, nn.Linear):
            nxt = _activation_of(nodes[i + 1], root) if i + 1 < len(nodes) else None
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
        else:
            # a user container (e.g. a block that wraps a linear and an activation): lower it as
            # a chain of its own and splice the result in
            blocks.extend(_lower(m))
        i += 1
    if not blocks:
        raise NotLowerable("the stage holds no layer")
    return blocks


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
        return blocks_from_graph(submod, submod.graph)
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
    return blocks_from_graph(submod, graph)


def lower_stage_module(submod: nn.Module, why: Optional[List[str]] = None) -> Optional[List[NativeBlock]]:
    """Blocks of a lowerable stage module, or None when it has to run eagerly; the reason is then
    appended to ``why``."""
    try:
        return _lower(submod)
    except NotLowerable as e:
        if why is not None:
            why.append(str(e))
        return None
