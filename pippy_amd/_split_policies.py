"""Automatic split policies for ``pipeline(..., split_policy=...)`` (the two size-based ones of the
reference, ``pippy/ModelSplit.py:158-206``): cut the traced graph into stages by the number of parameter
and buffer elements that the nodes of a stage use."""
from __future__ import annotations

from typing import Callable, Dict, List, Tuple

import torch
import torch.fx as fx

from ._IR import _attr, pipe_split


def _state_of_nodes(gm: fx.GraphModule) -> List[Tuple[fx.Node, Dict[int, int], bool]]:
    """(node, {id(tensor): elements}, whole) for every node that reads parameters or buffers, in graph
    order: a layer call reads the parameters of its module (``whole``: always counted in full, reference
    ``ModelSplit.py:107-110``), any other node the tensors that ``get_attr`` nodes hand it."""
    found = []
    for node in gm.graph.nodes:
        state: Dict[int, int] = {}
        if node.op == "call_module":
            sub = gm.get_submodule(node.target)
            # parameters only, and in full on every call of the module, as the reference counts a layer
            # (``ModelSplit.py:45-52``: ``named_parameters``; buffers of a layer are not counted)
            for t in sub.parameters():
                state[id(t)] = t.numel()
            whole = True
        else:
            for a in node.all_input_nodes:
                if a.op != "get_attr":
                    continue
                try:
                    t = _attr(gm, a.target)
                except AttributeError:
                    continue
                if torch.is_tensor(t):      # a parameter or buffer that the model's own forward reads
                    state[id(t)] = t.numel()
            whole = False
        if state:
            found.append((node, state, whole))
    return found


def _cut_by_size(gm: fx.GraphModule, threshold: int, max_stages: int = -1) -> Tuple[fx.GraphModule, int]:
    """Greedy buckets: a node joins the current stage while the stage's state stays within ``threshold``
    elements; otherwise a new stage starts in front of it (after it, when the node alone exceeds the
    threshold and the stage is still empty).  State that a function node shares with the stage so far
    is counted once.  Returns the graph module with the markers inserted and the number of stages."""
    cuts: List[fx.Node] = []
    held: Dict[int, int] = {}
    for node, state, whole in _state_of_nodes(gm):
        fresh = state if whole else {k: v for k, v in state.items() if k not in held}
        size, new = sum(held.values()), sum(fresh.values())
        if size + new <= threshold:
            held.update(fresh)
        elif size == 0:
            cuts.append(node.next)
        else:
            cuts.append(node)
            held = dict(state)
    stages = 1
    for node in cuts:
        if stages == max_stages:
            break
        with gm.graph.inserting_before(node):
            gm.graph.call_function(pipe_split, (), {})
        stages += 1
    gm.recompile()
    return gm, stages


def split_on_size_threshold(threshold: int) -> Callable[[fx.GraphModule], fx.GraphModule]:
    """A policy that starts a new stage before a stage would hold more than ``threshold`` parameter and
    buffer elements (reference ``ModelSplit.py:158-167``)."""
    def policy(gm: fx.GraphModule) -> fx.GraphModule:
        return _cut_by_size(gm, threshold)[0]
    return policy


def split_into_equal_size(nstages: int = 1) -> Callable[[fx.GraphModule], fx.GraphModule]:
    """A policy that cuts the model into ``nstages`` stages of about equal state size
    (reference ``ModelSplit.py:180-206``)."""
    def policy(gm: fx.GraphModule) -> fx.GraphModule:
        total = sum(p.numel() for p in gm.parameters()) + sum(b.numel() for b in gm.buffers())
        gm, found = _cut_by_size(gm, total // nstages, nstages)
        if found != nstages:
            raise AssertionError(f"the model splits into {found} stages of at most {total // nstages} elements, "
                                 f"not {nstages}")
        return gm
    return policy


def split_by_graph(nstages: int):
    """The reference's third policy solves a mixed-integer program over the graph
    (``ModelSplit.py:220-260``, ``graphsplit.py``); it is not built here."""
    raise NotImplementedError("split_by_graph is not provided; use split_into_equal_size, "
                              "split_on_size_threshold or explicit split points")
