"""Pipeline front end: split a model into stage modules (mirrors the public part of
``pippy/_IR.py``: ``pipeline``, ``Pipe``, ``SplitPoint``, ``pipe_split``,
``annotate_split_points``, ``ArgsChunkSpec``, ``KwargsChunkSpec``).

The reference exports the model with ``torch.export`` and cuts the ATen graph at ``pipe_split``
markers (``_IR.py:679-1125``).  This front end runs once at set-up and does no device work, so it
is kept small: the model is traced with ``torch.fx`` at module granularity (a module that does not
contain a split point stays one node, so stage modules keep whole layers that the stage runtime
can lower to kernels), markers are placed from ``split_spec`` or from ``pipe_split()`` calls in the
model's ``forward``, and ``torch.fx.passes.split_module`` cuts the graph.  As in the reference,
stage ``i`` is ``pipe.split_gm.submod_i`` and its parameters keep their original qualified names.
"""
from __future__ import annotations

import copy
import logging
import operator
from dataclasses import dataclass
from enum import Enum
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch
import torch.fx as fx
import torch.nn as nn
from torch.fx.passes.split_module import split_module

from .microbatch import TensorChunkSpec, split_args_kwargs_into_chunks
from .stage_modules import NativeBlock

logger = logging.getLogger(__name__)


_active_tracer: Optional["fx.Tracer"] = None


# The marker as an operator, so that ``torch.export`` records it too (the reference registers
# ``pippy::_pipe_split`` for the same purpose, ``_IR.py:319-329``): no inputs, no outputs, no effect.
@torch.library.custom_op("pippy_amd::_pipe_split", mutates_args=())
def _pipe_split_op() -> None:
    return None


@_pipe_split_op.register_fake
def _pipe_split_fake() -> None:
    return None


fx.node._side_effectful_functions.add(torch.ops.pippy_amd._pipe_split.default)


def pipe_split():
    """Marks a stage boundary when called inside a model's ``forward``
    (reference ``_IR.py:319-342``).  While ``pipeline()`` traces the model symbolically it records a
    marker node at the current position of the graph; otherwise it calls the marker operator, which
    does nothing when the model simply runs and which ``torch.export`` keeps in the exported graph."""
    if _active_tracer is not None:
        _active_tracer.create_proxy("call_function", pipe_split, (), {})
        return None
    torch.ops.pippy_amd._pipe_split()
    return None


class SplitPoint(Enum):
    BEGINNING = 1
    END = 2


class PipeSplitWrapper:
    """Kept for source compatibility: ``PipeSplitWrapper.SplitPoint`` (reference ``_IR.py:1299-1303``)."""
    SplitPoint = SplitPoint


class _ModuleGranularityTracer(fx.Tracer):
    def __init__(self, split_names: Optional[List[str]]):
        super().__init__()
        self._split_names = split_names

    def trace(self, root, concrete_args=None):
        global _active_tracer
        saved, _active_tracer = _active_tracer, self
        try:
            return super().trace(root, concrete_args)
        finally:
            _active_tracer = saved

    def is_leaf_module(self, m: nn.Module, qualname: str) -> bool:
        if isinstance(m, NativeBlock):
            return True
        if next(m.children(), None) is None and not type(m).__module__.startswith("torch.nn"):
            # a library's or a user's own affine layer, norm or activation stays one call, as torch.nn's do
            from .stage_modules import activation_like, in_out_linear_like, layer_norm_like, rms_norm_like
            if in_out_linear_like(m) or activation_like(m) is not None or rms_norm_like(m) is not None \
                    or layer_norm_like(m) is not None:
                return True
        if self._split_names is None:
            return super().is_leaf_module(m, qualname)
        # descend only into modules that contain a split point
        is_ancestor = any(s.startswith(qualname + ".") for s in self._split_names)
        if is_ancestor:
            return False
        if qualname in self._split_names:
            return True
        return super().is_leaf_module(m, qualname)


def _insert_markers(gm_graph: fx.Graph, split_spec: Dict[str, SplitPoint]):
    for name, point in split_spec.items():
        hits = [n for n in gm_graph.nodes if n.op == "call_module" and n.target == name]
        if not hits:
            raise ValueError(f"Specified split point {name!r} is not a module called by the model")
        node = hits[0] if point == SplitPoint.BEGINNING else hits[-1]
        if point == SplitPoint.BEGINNING:
            with gm_graph.inserting_before(node):
                gm_graph.call_function(pipe_split, (), {})
        elif point == SplitPoint.END:
            with gm_graph.inserting_after(node):
                gm_graph.call_function(pipe_split, (), {})
        else:
            raise ValueError(f"Unknown split point type {point}")


def _attr(root: nn.Module, target: str):
    obj = root
    for part in target.split("."):
        obj = getattr(obj, part)
    return obj


# regions the model ran under torch.no_grad() / torch.autocast(...): exported as one higher-order node
# around a sub-graph each
_WRAPPED_REGIONS = tuple(op for op in (getattr(torch.ops.higher_order, name, None) for name in
                                       ("wrap_with_set_grad_enabled", "wrap_with_autocast")) if op is not None)


def _drop_noop_casts(gm: fx.GraphModule) -> None:
    """``x.to(dtype)`` of a tensor that already has that dtype returns ``x``; the exporter still records a
    node, which hides that the layers around it read the same tensor."""
    for n in list(gm.graph.nodes):
        if n.op == "call_function" and n.target is torch.ops.aten.to.dtype and len(n.args) == 2 and not n.kwargs:
            src = n.args[0]
            have = getattr(src.meta.get("val"), "dtype", None) if isinstance(src, fx.Node) else None
            if have is not None and have == n.args[1]:
                n.replace_all_uses_with(src)
                gm.graph.erase_node(n)


def _fold_constants(gm: fx.GraphModule, state: frozenset = frozenset()) -> None:
    """Evaluates, once, every part of an exported graph that depends on no model input and no part of the
    model's state (position indices, attention masks built from the example's sequence length, ...), and
    replaces it by non-persistent buffers of ``gm``.  Stages then receive only activations from their
    predecessor instead of also such tensors computed by the first stage, and a stage's graph shows a
    constant mask as what it is.  ``state``: the names of the model's persistent buffers; like parameters
    they may be loaded from a checkpoint after the pipeline is built, so what is computed from them stays
    in the graph (and they stay in their stage's state_dict)."""
    graph = gm.graph
    value: Dict[fx.Node, Any] = {}
    for n in graph.nodes:
        if n.op == "get_attr":
            try:
                obj = _attr(gm, n.target)
            except AttributeError:
                continue
            written = any(u.op == "call_function" and getattr(getattr(u.target, "_schema", None), "is_mutable", False)
                          and u.target is not torch.ops.aten.detach_.default for u in n.users)
            if torch.is_tensor(obj) and not isinstance(obj, nn.Parameter) and not written and n.target not in state:
                value[n] = obj
            elif isinstance(obj, fx.GraphModule):
                value[n] = obj     # the body of a higher-order operator (below)
        elif n.op == "call_function" and (n.target is operator.getitem or n.target in _WRAPPED_REGIONS):
            # with constant inputs such a region is a constant like any other
            if any(a not in value for a in n.all_input_nodes):
                continue
            try:
                with torch.no_grad():
                    value[n] = n.target(*fx.node.map_arg(n.args, lambda a: value[a]),
                                        **fx.node.map_arg(n.kwargs, lambda a: value[a]))
            except Exception:
                continue
        elif n.op == "call_function" and n.target is torch.ops.aten.detach_.default:
            if n.args[0] in value:      # (in place, but it changes nothing about a constant)
                value[n] = value[n.args[0]]
        elif n.op == "call_function" and isinstance(n.target, torch._ops.OpOverload):
            if n.target.namespace != "aten" or torch.Tag.nondeterministic_seeded in n.target.tags \
                    or n.target._schema.is_mutable or any(a not in value for a in n.all_input_nodes):
                continue
            try:
                with torch.no_grad():
                    value[n] = n.target(*fx.node.map_arg(n.args, lambda a: value[a]),
                                        **fx.node.map_arg(n.kwargs, lambda a: value[a]))
            except Exception:
                continue
    count = 0
    for c in [n for n in value if n.op == "call_function" and torch.is_tensor(value[n])]:
        outside = [u for u in c.users if u not in value]
        if not outside:
            continue
        name = f"_folded_constant_{count}_tensor"   # (a name that fx's _1, _2 suffixes of node names cannot collide with)
        count += 1
        gm.register_buffer(name, value[c].clone(), persistent=False)
        for u in outside:
            with graph.inserting_before(u):
                const = graph.get_attr(name)
            const.meta = {k: v for k, v in c.meta.items() if k == "val"}
            u.replace_input_with(c, const)
    for n in reversed(list(graph.nodes)):
        if n in value and not n.users:
            graph.erase_node(n)


# Layers of torch.nn that take one tensor and whose exported nodes can be put back as one call of the layer
_REROLLED_TYPES = (nn.Linear, nn.LayerNorm, nn.RMSNorm, nn.Embedding, nn.Dropout, nn.GELU, nn.ReLU, nn.SiLU,
                   nn.Identity)


def _reroll_leaf_layers(mod: nn.Module, gm: fx.GraphModule) -> None:
    """``torch.export`` dissolves every layer into ATen nodes.  This puts the standard leaf layers of
    the model back: the nodes that the exporter recorded as coming from one call of such a layer, when
    they read one tensor from outside and hand one tensor on, become a ``call_module`` node on the
    model's own layer object (installed in ``gm`` under its qualified name).  A stage cut from the graph
    then holds whole layers, which is what the stage runtime lowers to kernels; the result computed is
    unchanged.  Besides the torch.nn types this covers layers of other libraries that are recognisably
    an affine map with an [in, out] weight or an elementwise activation (checked on sample values, and
    their exported nodes are checked against the layer itself)."""
    from .stage_modules import activation_like, in_out_linear_like, layer_norm_like, rms_norm_like
    graph = gm.graph
    leaves = {}
    for name, m in mod.named_modules():
        if not name or next(m.children(), None) is not None:
            continue
        base = next((t for t in _REROLLED_TYPES if isinstance(m, t)), None)
        if base is not None:
            # a subclass with a forward of its own (a position table that shifts its indices, say) is
            # put back only if that forward is what the exported nodes compute
            leaves[name] = (m, type(m).forward is not base.forward, base)
        elif in_out_linear_like(m) or activation_like(m) is not None or rms_norm_like(m) is not None \
                or layer_norm_like(m) is not None:
            leaves[name] = (m, True, None)
    calls: Dict[Tuple[str, str], List[fx.Node]] = {}
    for n in graph.nodes:
        stack = n.meta.get("nn_module_stack") if n.op == "call_function" else None
        if not stack:
            continue
        key, entry = list(stack.items())[-1]
        if entry[0] in leaves:
            calls.setdefault((key, entry[0]), []).append(n)
    for (_key, fqn), nodes in calls.items():
        layer, verify, base = leaves[fqn]
        inside = set(nodes)
        external, own = [], []
        for n in nodes:
            for a in n.all_input_nodes:
                if a in inside:
                    continue
                if a.op == "get_attr" and str(a.target).startswith(fqn + "."):
                    own.append(a)
                elif a not in external:
                    external.append(a)
        results = [n for n in nodes if any(u not in inside for u in n.users)]
        if len(external) != 1 or len(results) != 1:
            continue
        src, res = external[0], results[0]
        if verify:
            fake = src.meta.get("val")

            def same_as(forward) -> bool:
                try:
                    shape = tuple(int(d) for d in fake.shape)
                    if fake.dtype.is_floating_point:
                        x = torch.randn(shape, dtype=fake.dtype)
                    else:       # indices into a table: the lower half of its rows
                        x = torch.randint(0, max(1, getattr(layer, "num_embeddings", 2) // 2), shape, dtype=fake.dtype)
                    env = {src: x}
                    env.update({a: _attr(gm, a.target) for a in own})
                    with torch.no_grad():
                        for n in nodes:
                            env[n] = n.target(*fx.node.map_arg(n.args, lambda a: env[a]),
                                              **fx.node.map_arg(n.kwargs, lambda a: env[a]))
                        want, got = env[res], forward(x)
                    return got.shape == want.shape and bool((got.float() - want.float()).abs().max()
                                                            <= 1e-5 + 2e-2 * want.float().abs().max()
                                                            * (want.dtype != torch.float32))
                except Exception:
                    return False

            if not same_as(layer):
                # the nodes may still be the base layer's arithmetic on these parameters (the rest of the
                # subclass's forward was folded into a constant or lies outside): then the base layer's
                # view of the same parameter objects goes into the graph
                if base is None or not same_as(lambda x: base.forward(layer, x)):
                    continue
                layer = copy.copy(layer)
                layer.__class__ = base
        gm.add_submodule(fqn, layer)
        with graph.inserting_after(nodes[-1]):
            call = graph.call_module(fqn, (src,))
        call.meta = dict(res.meta)
        res.replace_all_uses_with(call)
        for n in reversed(nodes):
            graph.erase_node(n)
    for n in reversed(list(graph.nodes)):
        if n.op == "get_attr" and not n.users:
            graph.erase_node(n)


def _export_and_mark(mod: nn.Module, mb_args: Tuple[Any, ...], mb_kwargs: Optional[Dict[str, Any]],
                     split_spec: Optional[Dict[str, SplitPoint]]) -> Tuple[fx.GraphModule, fx.Graph]:
    """The route of the reference (``_IR.py:1141-1145``): ``torch.export`` on the inputs of one
    microbatch, for models that symbolic tracing cannot follow (Python control flow on shapes, calls
    torch.fx has no proxy for).  Returns the exported module, whose parameters and buffers keep their
    qualified names, and its ATen-level graph with a ``pipe_split`` marker node at every stage
    boundary: where the model called ``pipe_split()``, and where ``split_spec`` names a submodule (the
    first / last node that the exporter recorded as coming from inside it)."""
    ep = torch.export.export(mod, tuple(mb_args), dict(mb_kwargs or {}), strict=False)
    gm = ep.module()
    graph = gm.graph
    for n in list(graph.nodes):
        if (n.op == "call_module" and str(n.target).startswith("_guards")) or \
                (n.op == "call_function" and n.target is torch.ops.aten._assert_tensor_metadata.default):
            graph.erase_node(n)   # guards of the example inputs' shapes and dtypes: stages re-check nothing
    _drop_noop_casts(gm)
    _fold_constants(gm, frozenset(k for k, _ in mod.named_buffers()) & frozenset(mod.state_dict().keys()))
    _reroll_leaf_layers(mod, gm)
    # what nothing reads (a pooling head whose result the model drops, say) would otherwise give the last
    # layer a second reader; split markers and in-place operators stay
    for n in reversed(list(graph.nodes)):
        if n.users or n.op not in ("call_function", "call_module", "get_attr"):
            continue
        if n.op == "call_function" and (n.target is torch.ops.pippy_amd._pipe_split.default or
                                        getattr(getattr(n.target, "_schema", None), "is_mutable", False)):
            continue
        graph.erase_node(n)
    for n in list(graph.nodes):
        if n.op == "call_function" and n.target is torch.ops.pippy_amd._pipe_split.default:
            n.target = pipe_split
    compute = [n for n in graph.nodes if n.op in ("call_function", "call_method", "call_module")]
    for name, point in (split_spec or {}).items():
        inside = [n for n in compute
                  if any(v[0] == name or v[0].startswith(name + ".")
                         for v in (n.meta.get("nn_module_stack") or {}).values())]
        if not inside:
            raise ValueError(f"Specified split point {name!r} is not a module called by the model")
        if point == SplitPoint.BEGINNING:
            with graph.inserting_before(inside[0]):
                graph.call_function(pipe_split, (), {})
        elif point == SplitPoint.END:
            with graph.inserting_after(inside[-1]):
                graph.call_function(pipe_split, (), {})
        else:
            raise ValueError(f"Unknown split point type {point}")
    # a model that returns one tensor exports as a one-element tuple plus an output spec: undo that
    out = next(n for n in graph.nodes if n.op == "output")
    spec = getattr(gm, "_out_spec", None)
    if spec is not None and spec.num_leaves == 1 and spec.num_nodes == 1 and isinstance(out.args[0], (tuple, list)):
        out.args = (out.args[0][0],)
    graph.lint()
    return gm, graph


@dataclass
class PipeInfo:
    """What the stage runtime needs from the front end (reference ``_IR.py:509-516``)."""
    graph: fx.Graph
    num_stages: int
    num_chunks: int
    has_loss_and_backward: bool
    args_chunk_spec: Optional[Tuple[Any, ...]] = None
    kwargs_chunk_spec: Optional[Dict[str, Any]] = None


class Pipe(nn.Module):
    """A model cut into stage modules ``split_gm.submod_0 .. submod_{n-1}``
    (reference ``_IR.py:494-1291``).  Calling a ``Pipe`` runs the stages one after another in this
    process, without microbatching (reference ``Pipe.forward``, ``_IR.py:620-651``)."""

    # set by the ArgsChunkSpec / KwargsChunkSpec context managers
    args_chunk_spec: Optional[Tuple[Any, ...]] = None
    kwargs_chunk_spec: Optional[Dict[str, Any]] = None

    PipeInfo = PipeInfo

    def __init__(self, split_gm: fx.GraphModule, num_stages: int, has_loss_and_backward: bool = False,
                 loss_spec=None):
        super().__init__()
        self.split_gm = split_gm
        self.num_stages = num_stages
        self.has_loss_and_backward = has_loss_and_backward
        self.loss_spec = loss_spec
        self.pipe_info: Optional[PipeInfo] = None

    def forward(self, *args, **kwargs):
        return self.split_gm(*args, **kwargs)

    def get_stage_module(self, stage_idx: int) -> nn.Module:
        if stage_idx < 0 or stage_idx >= self.num_stages:
            raise ValueError(f"Invalid stage index {stage_idx}!")
        return getattr(self.split_gm, f"submod_{stage_idx}")

    def info(self) -> PipeInfo:
        if self.pipe_info is None:
            raise RuntimeError("Pipe info is not available. Please use the `pipeline` method to create the `Pipe` object.")
        return self.pipe_info

    def build_stage(self, stage_index: int, device, group=None, **kw):
        """The runtime stage for ``stage_index`` (the spelling of the reference's examples,
        ``examples/llama/pippy_llama.py:36-39``); same as ``PipelineStage(pipe, stage_index, device, group)``."""
        from .stage import PipelineStage
        return PipelineStage(self, stage_index, device, group, **kw)

    def __str__(self):
        return self.split_gm.__str__()

    def __repr__(self):
        return self.split_gm.__repr__()

    @staticmethod
    def _from_traced(mod: nn.Module, graph: fx.Graph) -> "Pipe":
        # number the partitions by the markers and drop the markers
        part = 0
        part_of: Dict[fx.Node, int] = {}
        markers = []
        for n in graph.nodes:
            if n.op == "call_function" and n.target is pipe_split:
                part += 1
                markers.append(n)
                continue
            part_of[n] = part
        for m in markers:
            graph.erase_node(m)
        gm = fx.GraphModule(mod, graph)
        orig_target = {n.name: n.target for n in graph.nodes if n.op in ("call_module", "get_attr")}
        split = split_module(gm, mod, lambda n: part_of[n], keep_original_order=True)
        num_stages = part + 1
        # split_module flattens qualified names ("h.0" -> "h_0"); rebuild every stage module from the
        # original model with the original targets so that parameter names are unchanged
        # (the reference re-outlines for the same reason, ``_IR.py:765-769``)
        # parameters and buffers that the model's own forward reads (``self.scale``) stay behind in
        # the root as get_attr nodes feeding the stage call; they belong to the stage that uses them,
        # under their original name (the reference sinks them the same way, ``_IR.py:785-895``)
        sunk: Dict[str, Dict[int, str]] = {}
        for call in split.graph.nodes:
            if call.op != "call_module" or not str(call.target).startswith("submod_"):
                continue
            keep = []
            for i, a in enumerate(call.args):
                if isinstance(a, fx.Node) and a.op == "get_attr":
                    sunk.setdefault(call.target, {})[i] = orig_target.get(a.name, a.target)
                else:
                    keep.append(a)
            call.args = tuple(keep)
        for n in list(split.graph.nodes):
            if n.op == "get_attr" and not n.users:
                split.graph.erase_node(n)
        for name, sub in list(split.named_children()):
            if not name.startswith("submod_"):
                continue
            for n in sub.graph.nodes:
                if n.op in ("call_module", "get_attr") and n.name in orig_target:
                    n.target = orig_target[n.name]
            placeholders = [n for n in sub.graph.nodes if n.op == "placeholder"]
            for i, target in sunk.get(name, {}).items():
                ph = placeholders[i]
                with sub.graph.inserting_after(ph):
                    attr = sub.graph.create_node("get_attr", target)
                ph.replace_all_uses_with(attr)
                sub.graph.erase_node(ph)
            stage_mod = fx.GraphModule(mod, sub.graph, class_name=name)
            # constants folded out of an exported graph are not part of the model's state
            stage_mod._non_persistent_buffers_set.update(
                b for b, _ in stage_mod.named_buffers(recurse=False) if b.startswith("_folded_constant_"))
            setattr(split, name, stage_mod)
        split.recompile()
        found = [n for n, _ in split.named_children() if n.startswith("submod_")]
        if len(found) != num_stages:
            raise RuntimeError(f"expected {num_stages} stage modules after splitting, found {found} "
                               "(an empty stage: two split points with nothing between them)")
        # a parameter may live in one stage only (reference ``_IR.py:871-879``)
        owner: Dict[int, str] = {}
        for name, sub in split.named_children():
            if not name.startswith("submod_"):
                continue
            for pn, p in sub.named_parameters():
                if id(p) in owner and owner[id(p)] != name:
                    raise NotImplementedError(
                        f"Parameter {pn} is used in stages {owner[id(p)]} and {name}; parameters shared "
                        "between stages (e.g. tied embeddings) are not supported")
                owner[id(p)] = name
        return Pipe(split, num_stages)

    @staticmethod
    def from_tracing(mod: nn.Module, num_chunks: int, example_args: Tuple[Any, ...],
                     example_kwargs: Optional[Dict[str, Any]] = None,
                     split_policy: Optional[Callable[[fx.GraphModule], fx.GraphModule]] = None,
                     split_spec: Optional[Dict[str, SplitPoint]] = None) -> "Pipe":
        args_chunk_spec = Pipe.args_chunk_spec
        kwargs_chunk_spec = Pipe.kwargs_chunk_spec
        # validates the chunk specs against the example inputs (reference ``_IR.py:1172-1178``)
        split_args_kwargs_into_chunks(example_args, example_kwargs, num_chunks, args_chunk_spec,
                                      kwargs_chunk_spec)
        names = list(split_spec.keys()) if split_spec else None

        def exported(fx_error):
            """(root, graph) over torch.export on the first microbatch's inputs, as the reference traces
            (``_IR.py:1172-1185``); the stages are then ATen-level graphs."""
            args_split, kwargs_split = split_args_kwargs_into_chunks(example_args, example_kwargs, num_chunks,
                                                                     args_chunk_spec, kwargs_chunk_spec)
            try:
                return _export_and_mark(mod, args_split[0], kwargs_split[0], split_spec)
            except ValueError:
                raise
            except Exception as export_error:
                config = getattr(mod, "config", None)
                if "data pointer" in str(export_error) and getattr(config, "_experts_implementation", None) not in \
                        (None, "batched_mm"):
                    # a library's grouped expert product inspects tensor addresses, which torch.export cannot
                    # trace; its batched form computes the same and traces: export with that one selected
                    chosen = config._experts_implementation
                    config._experts_implementation = "batched_mm"
                    try:
                        traced = _export_and_mark(mod, args_split[0], kwargs_split[0], split_spec)
                        logger.warning("exported with config._experts_implementation = 'batched_mm' (the "
                                       f"'{chosen}' form inspects tensor addresses, which torch.export cannot trace)")
                        return traced
                    except Exception:
                        pass
                    finally:
                        config._experts_implementation = chosen
                if "Cache" in str(export_error) and getattr(config, "use_cache", False):
                    # the model returns a key / value cache object, which torch.export cannot flatten and a
                    # training or scoring pipeline has no use for: export without it
                    config.use_cache = False
                    try:
                        traced = _export_and_mark(mod, args_split[0], kwargs_split[0], split_spec)
                        logger.warning("exported with config.use_cache = False: the model's key / value cache object "
                                       "cannot be exported, and the pipeline's stages do not return one")
                        return traced
                    except Exception:
                        pass
                    finally:
                        config.use_cache = True
                hint = ""
                if "Cache" in str(export_error) and getattr(getattr(mod, "config", None), "use_cache", False):
                    hint = ("; the model returns a key / value cache object, which torch.export cannot flatten: "
                            "build it with config.use_cache = False")
                if "data pointer" in str(export_error) and hasattr(getattr(mod, "config", None), "_experts_implementation"):
                    hint = ("; the model's grouped expert product inspects tensor addresses, which torch.export "
                            "cannot trace: build it with config._experts_implementation = 'batched_mm'")
                raise RuntimeError(
                    f"pipeline(): neither torch.fx symbolic tracing ({type(fx_error).__name__}: {fx_error}) "
                    f"nor torch.export ({type(export_error).__name__}: {export_error}) can trace this model{hint}"
                ) from export_error

        def build(root, graph):
            if split_policy is not None:
                graph = split_policy(fx.GraphModule(root, graph)).graph
            return Pipe._from_traced(root, graph)

        def widest_boundary(pipe):
            return max([len([n for n in pipe.get_stage_module(i).graph.nodes if n.op == "placeholder"])
                        for i in range(1, pipe.num_stages)] or [0])

        try:
            graph = _ModuleGranularityTracer(names).trace(mod)
            if split_spec:
                _insert_markers(graph, split_spec)
        except Exception as fx_error:
            # symbolic tracing cannot follow this model
            logger.warning(f"torch.fx symbolic tracing failed ({type(fx_error).__name__}: {fx_error}); "
                           "falling back to torch.export on the inputs of one microbatch: the stages hold "
                           "that microbatch's shapes; standard layers are put back into the ATen-level graph, "
                           "and a stage whose structure is then recognised still runs as HIP launch lists")
            pipe = build(*exported(fx_error))
        else:
            pipe = build(mod, graph)
            if widest_boundary(pipe) > 1:
                # a symbolically traced forward keeps what it computes from shapes (a mask built from the
                # sequence length, say) as values that travel from stage to stage; exported on an example
                # they are constants of each stage.  The exported pipeline is taken when that leaves fewer
                # values on the boundaries; otherwise (real skip connections) the traced one stays.
                try:
                    other = build(*exported(None))
                except Exception:
                    other = None
                if other is not None and other.num_stages == pipe.num_stages and \
                        widest_boundary(other) < widest_boundary(pipe):
                    logger.warning("the symbolically traced stages would hand more than one tensor on (values "
                                   "computed from shapes); using torch.export on the inputs of one microbatch "
                                   "instead, where they are constants: the stages hold that microbatch's shapes")
                    pipe = other
        pipe.pipe_info = PipeInfo(graph=pipe.split_gm.graph, num_stages=pipe.num_stages,
                                  num_chunks=num_chunks, has_loss_and_backward=False,
                                  args_chunk_spec=args_chunk_spec, kwargs_chunk_spec=kwargs_chunk_spec)
        return pipe


def annotate_split_points(mod: nn.Module, spec: Dict[str, SplitPoint]):
    """Wraps the named submodules so that their ``forward`` calls ``pipe_split()`` before
    (BEGINNING) or after (END) itself (reference ``_IR.py:1306-1338``)."""
    for qualname, split_type in spec.items():
        try:
            target = mod.get_submodule(qualname)
        except AttributeError as e:
            raise AttributeError(f"Specified target {qualname} referenced nonexistent module") from e
        orig_forward = target.forward

        def make(orig_forward=orig_forward, split_type=split_type):
            def forward(*args, **kwargs):
                if split_type == SplitPoint.BEGINNING:
                    pipe_split()
                out = orig_forward(*args, **kwargs)
                if split_type == SplitPoint.END:
                    pipe_split()
                return out
            return forward

        target.forward = make()


def pipeline(module: nn.Module, num_chunks: Optional[int] = None, example_args: Optional[Tuple[Any, ...]] = None,
             example_kwargs: Optional[Dict[str, Any]] = None,
             split_spec: Optional[Dict[str, SplitPoint]] = None,
             split_policy: Optional[Callable[[fx.GraphModule], fx.GraphModule]] = None, *,
             mb_args: Optional[Tuple[Any, ...]] = None, mb_kwargs: Optional[Dict[str, Any]] = None) -> Pipe:
    """Splits ``module`` into pipeline stages (reference ``_IR.py:1341-1395``).

    ``split_spec`` maps submodule names to ``SplitPoint.BEGINNING`` / ``END``; alternatively the
    model's ``forward`` may call ``pipe_split()``, or ``split_policy`` may place the markers on the
    traced graph.  ``num_chunks`` and the example inputs describe one full batch; the chunk specs
    in force (``ArgsChunkSpec`` / ``KwargsChunkSpec``) are recorded for the schedules.

    The reference's examples are written against the later spelling of this call,
    ``pipeline(module, mb_args=..., mb_kwargs=...)`` with the inputs of ONE microbatch
    (``examples/huggingface/pippy_gpt2.py:50-65``); it is accepted too: the number of microbatches
    is then the schedule's ``n_microbatches``."""
    if split_spec is not None and split_policy is not None:
        raise ValueError("Cannot specify both `split_spec` and `split_policy`. Please use only one of them.")
    if mb_args is not None or mb_kwargs is not None:
        if num_chunks is not None or example_args is not None or example_kwargs is not None:
            raise ValueError("pass either (num_chunks, example_args, example_kwargs) or (mb_args, mb_kwargs)")
        num_chunks, example_args, example_kwargs = 1, tuple(mb_args or ()), mb_kwargs
    if num_chunks is None or example_args is None:
        raise TypeError("pipeline() needs num_chunks and example_args (or mb_args)")
    return Pipe.from_tracing(mod=module, num_chunks=num_chunks, example_args=example_args,
                             example_kwargs=example_kwargs, split_policy=split_policy,
                             split_spec=split_spec)


class ArgsChunkSpec:
    """Context manager that sets the chunk spec of positional args for ``pipeline()``
    (reference ``_IR.py:1399-1424``)."""

    def __init__(self, chunk_dims: Tuple[int, ...]):
        self.args_chunk_spec = tuple(TensorChunkSpec(d) for d in chunk_dims)

    def __enter__(self):
        self._saved = Pipe.args_chunk_spec
        Pipe.args_chunk_spec = self.args_chunk_spec
        return self.args_chunk_spec

    def __exit__(self, exc_type, exc_val, traceback):
        Pipe.args_chunk_spec = self._saved


class KwargsChunkSpec:
    """Context manager that sets the chunk spec of keyword args for ``pipeline()``
    (reference ``_IR.py:1427-1451``)."""

    def __init__(self, chunk_dims: Dict[str, int]):
        self.kwargs_chunk_spec = {k: TensorChunkSpec(d) for k, d in chunk_dims.items()}

    def __enter__(self):
        self._saved = Pipe.kwargs_chunk_spec
        Pipe.kwargs_chunk_spec = self.kwargs_chunk_spec
        return self.kwargs_chunk_spec

    def __exit__(self, exc_type, exc_val, traceback):
        Pipe.kwargs_chunk_spec = self._saved
