"""Pipeline stage runtime (mirrors ``pippy/_PipelineStage.py`` and ``pippy/ManualPipelineStage.py``).

Every stage of the pipeline is a *virtual* stage on one GPU.  The reference moves a microbatch's
activation from stage s to stage s+1 (and its gradient back) with ``dist.P2POp`` send/recv pairs
into per-microbatch receive buffers (``_PipelineStage.py:210-341``); here the producer's output
slot *is* the consumer's input, and the consumer's input-gradient pass writes straight into the
producer's output-gradient slot: the hand-off is a pointer, no bytes move.

Two execution modes per stage:

* native: the stage module lowers to HIP launch lists (``_program.py``); forward, input-gradient
  and weight-gradient passes are separate entry points and parameter gradients are accumulated in
  fp32: ``acc += float(g)`` with ``g`` the microbatch gradient in the parameter dtype, microbatches
  ascending (weight gradients by the epilogue of their GEMM, the small tensors by the accumulate
  kernel; ``fused_accumulate=True`` adds the unrounded fp32 sums instead, ``"staged"`` sends every
  gradient through the staging arena and the accumulate kernel, with the same bits as the default);
* eager: any other ``nn.Module`` runs through torch autograd on the GPU exactly as the reference
  does (``forward_one_chunk`` / ``stage_backward``), with the same caching rules.
"""
from __future__ import annotations

import logging
import os
from typing import Any, Dict, List, Optional, Tuple, Union

import torch
import torch.nn as nn

from . import _native as N
from . import _program as P
from ._backward import stage_backward
from ._lowering import lower_stage_module
from ._utils import flatten_args
from .losses import as_native_loss

logger = logging.getLogger(__name__)

# PIPPY_AMD_CHECK_INPUTS=1: token ids and loss targets are range-checked on the host before the kernels
# that index with them run (one device-to-host synchronisation per check; off by default)
_CHECK_INPUTS = os.environ.get("PIPPY_AMD_CHECK_INPUTS") == "1"


class VirtualGroup:
    """Stands in for the reference's process group: ``size`` virtual pipeline ranks that all live
    in this process.  ``stage_index % size`` is a stage's rank (wrap-around placement,
    ``_PipelineStage.py:129-136``)."""

    def __init__(self, size: int):
        if size < 1:
            raise ValueError("a virtual group needs at least one rank")
        self._size = size

    def size(self) -> int:
        return self._size


def _group_size(group) -> int:
    if group is None:
        return 1
    if isinstance(group, int):
        return group
    if isinstance(group, VirtualGroup):
        return group.size()
    try:  # a real torch.distributed group of this (single) process
        import torch.distributed as dist
        return dist.get_world_size(group)
    except Exception as e:  # pragma: no cover
        raise TypeError(f"unsupported group object {group!r}") from e


class PipelineStageBase:
    """State and per-microbatch entry points shared by ``PipelineStage`` and
    ``ManualPipelineStage`` (reference ``_PipelineStage.py:72-551``)."""

    def __init__(self, submodule: nn.Module, stage_index: int, num_stages: int,
                 device: Union[torch.device, str], num_microbatches: int, group=None, *,
                 fused_accumulate: Union[bool, str] = False, force_eager: bool = False):
        if stage_index >= num_stages:
            raise ValueError(f"Stage index {stage_index} is out of range of {num_stages}")
        self.submod = submodule
        self.stage_index = stage_index
        self.num_stages = num_stages
        self.device = torch.device(device)
        self.chunks = num_microbatches
        self.group = group
        self.group_size = _group_size(group)
        self.group_rank = stage_index % self.group_size
        if self.group_size > self.num_stages:
            raise RuntimeError(
                f"Pipeline group size {self.group_size} cannot be larger than number of stages {self.num_stages}")
        self.stage_index_to_group_rank = {i: i % self.group_size for i in range(num_stages)}

        # run-time state (reference names)
        self.fwd_cache: Dict[int, Tuple[Any, List[torch.Tensor]]] = {}
        self.fwd_chunk_id = 0
        self.bwd_chunk_id = 0
        self.bwd_weight_chunk_id = 0
        self.output_chunks: List[Any] = []
        self.grads_input: List[Optional[torch.Tensor]] = []
        self._has_backward = False
        self.log_prefix = f"[Stage {self.stage_index}]"

        # neighbours on the device; set by the schedule
        self._prev: Optional["PipelineStageBase"] = None
        self._next: Optional["PipelineStageBase"] = None
        self._fwd_done: Dict[int, bool] = {}
        self._bwd_done: Dict[int, bool] = {}
        self._input_grads: Dict[int, List[Optional[torch.Tensor]]] = {}  # eager hand-off
        self._bridge: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}  # generic loss on a native stage
        self._step_losses: Optional[torch.Tensor] = None

        self.fused_accumulate = fused_accumulate
        self.split_backward = False
        #: run the weight-gradient passes of a step as one batched pass (``flush_weight_grads``) instead of
        #: one per microbatch; set by the schedule, needs ``split_backward``
        self.batch_weight_grads = False
        why: List[str] = []
        if not force_eager and self.device.type != "cuda":
            force_eager = True
            why.append(f"its device is '{self.device}' and launch lists run on the GPU only")
        self._blocks = None if force_eager else lower_stage_module(submodule, why, for_kernels=True)
        # Whether a dropout does nothing is decided when the stage is lowered (p == 0, or eval mode).  The
        # layers that were taken as identity only because of the mode are remembered: a launch-list stage
        # whose module is switched to training mode afterwards would otherwise train without dropout.
        self._mode_bound_dropouts: List[nn.Module] = [] if self._blocks is None else [
            m for m in submodule.modules()
            if (isinstance(m, nn.modules.dropout._DropoutNd) and m.p > 0)
            or (isinstance(m, nn.MultiheadAttention) and m.dropout > 0)]
        self._program: Optional[P.StageProgram] = None
        #: why this stage runs through torch autograd instead of HIP launch lists (None: it is native)
        self.eager_reason: Optional[str] = None
        if self._blocks is None:
            self.eager_reason = why[0] if why else (
                "its inputs or outputs are not a single tensor chain between consecutive stages"
                if force_eager else "unknown")
            logger.warning(f"{self.log_prefix} runs eagerly through torch autograd, not as HIP launch lists: "
                           f"{self.eager_reason}")
            self.submod.to(self.device)
            self._move_ops_to_device()

    def _move_ops_to_device(self):
        """An exported graph holds the device of export time as a literal ``device=`` argument of the
        ops that create tensors; an eager stage runs that graph, so the literals are pointed at the
        stage's device (reference ``_PipelineStage.py:621-628``)."""
        if not isinstance(self.submod, torch.fx.GraphModule):
            return
        changed = False
        for node in self.submod.graph.nodes:
            if node.op == "call_function" and isinstance(node.kwargs.get("device"), torch.device) \
                    and node.kwargs["device"] != self.device:
                node.kwargs = {**node.kwargs, "device": self.device}
                changed = True
        if changed:
            self.submod.recompile()

    # -- reference properties -----------------------------------------------------------------
    @property
    def has_backward(self) -> bool:
        return self._has_backward

    @has_backward.setter
    def has_backward(self, has_backward: bool):
        self._has_backward = has_backward

    @property
    def is_first(self):
        return self.stage_index == 0

    @property
    def is_last(self):
        return self.stage_index == self.num_stages - 1

    @property
    def is_native(self) -> bool:
        return self._blocks is not None

    # The reference's schedules ask a stage for P2P op lists around every forward / backward.
    # With device-local hand-off there is nothing to post; the methods remain for API parity.
    def get_fwd_recv_ops(self):
        return []

    def get_bwd_recv_ops(self):
        return []

    def get_fwd_send_ops(self):
        return []

    def get_bwd_send_ops(self):
        return []

    def _configure_data_parallel_mode(self, last_backward: bool):
        """No data-parallel wrapper exists on one GPU (reference ``_PipelineStage.py:409-418``)."""

    def clear_runtime_states(self) -> None:
        """Resets per-step state (reference ``_PipelineStage.py:343-366``)."""
        if self._program is not None:
            self._program.arena.refresh_transposed()
        self.fwd_chunk_id = 0
        self.bwd_chunk_id = 0
        self.bwd_weight_chunk_id = 0
        self.fwd_cache.clear()
        self.output_chunks.clear()
        self._fwd_done.clear()
        self._bwd_done.clear()
        self._input_grads.clear()
        self._bridge.clear()
        self._step_losses = None  # per-step buffer of the native losses, allocated by the first of them

    # -- program management ---------------------------------------------------------------------
    def _stage_program(self) -> P.StageProgram:
        if self._program is None:
            self._program = P.StageProgram(self._blocks, self.submod, self.device,
                                           training=self.has_backward,
                                           split_backward=self.split_backward,
                                           fused_accumulate=self.fused_accumulate,
                                           is_first=self.is_first, is_last=self.is_last)
            self._publish_grad_views()
        elif self._program.training != self.has_backward or \
                self._program.split_backward != self.split_backward:
            # the schedule changed between steps (e.g. inference after training): re-lower
            self._program.training = self.has_backward
            self._program.split_backward = self.split_backward
            self._program.mbs.clear()
        return self._program

    def param_arena(self) -> "P.ParamArena":
        """The flat parameter / fp32-accumulator storage of a natively lowered stage (what the fused
        optimizers step on)."""
        if not self.is_native:
            raise RuntimeError(f"{self.log_prefix} is not lowered to launch lists and has no arena")
        return self._stage_program().arena

    def saved_activations(self, mb: int) -> Dict[str, torch.Tensor]:
        """The buffers a natively lowered stage keeps for microbatch ``mb`` between its forward and
        backward pass, by scoped name (for inspection, e.g. the expert selection of a
        mixture-of-experts layer: keys ending in ``topk_idx``)."""
        if not self.is_native:
            raise RuntimeError(f"{self.log_prefix} is not lowered to launch lists")
        return dict(self._stage_program().mbs[mb].acts)

    def _publish_grad_views(self):
        """fp32 parameters get their accumulator as ``.grad``; bf16 parameters expose it as
        ``.main_grad`` (torch does not allow an fp32 ``.grad`` on a bf16 parameter)."""
        arena = self._program.arena
        for _, p in arena.named:
            view = arena.grad_acc(p, padded=False)
            p.main_grad = view

    def zero_grad(self):
        """Forget accumulated parameter gradients: the next weight-gradient pass overwrites the
        fp32 accumulators instead of adding to them."""
        if self._program is not None:
            self._program.acc_initialized = False
            self._program.grads_handed_over = False
        for p in self.submod.parameters():
            p.grad = None

    def materialize_grads(self):
        """Sets ``param.grad`` from the fp32 accumulators (cast to the parameter dtype) so that a
        stock torch optimizer can step; fp32 parameters share memory with the accumulator."""
        if self._program is None:
            return
        for _, p in self._program.arena.named:
            p.grad = p.main_grad if p.dtype == torch.float32 else p.main_grad.to(p.dtype)
        # from here on a cleared ``.grad`` (``optimizer.zero_grad()``) means "start a new accumulation",
        # exactly as for fp32 parameters, whose ``.grad`` is the accumulator itself
        self._program.grads_handed_over = True

    def _input_for(self, mb: int, args, kwargs):
        """(x, dx_target, patch_input) of microbatch ``mb`` for a native stage."""
        if self.is_first:
            # the stage's graph has one input: it may arrive by position or by keyword
            # (``schedule.step(input_ids=ids)``, reference ``examples/huggingface/pippy_gpt2.py:73-77``)
            values = [a for a in list(args) + list(kwargs.values()) if a is not None]
            tensors = [a for a in values if isinstance(a, torch.Tensor)]
            if len(tensors) != 1 or len(values) != 1:
                raise RuntimeError(
                    f"{self.log_prefix} a native stage takes exactly one tensor input, got {len(args)} positional "
                    f"and {len(kwargs)} keyword values")
            x = tensors[0]
            if not x.is_cuda:
                raise RuntimeError(f"{self.log_prefix} input is on {x.device}; move it to {self.device}")
            return x, None, True
        prev = self._prev
        if prev is None:
            raise RuntimeError(
                f"{self.log_prefix} is not linked to stage {self.stage_index - 1}: pass every stage of "
                "the pipeline to the schedule (all stages are virtual stages of this process)")
        if not prev._fwd_done.get(mb):
            raise RuntimeError(f"{self.log_prefix} activation of microbatch {mb} has not been produced")
        if prev.is_native:
            pprog = prev._program.mbs[mb]
            x = pprog.output
            dx = getattr(pprog, "output_grad_buf", None) if self.has_backward else None
            if x.dim() and not x.is_contiguous():
                raise RuntimeError(f"{self.log_prefix} received a non-contiguous activation")
            return x, dx, False
        out = prev.output_chunks[mb]
        if not isinstance(out, torch.Tensor):
            raise RuntimeError(f"{self.log_prefix} native stages take a single tensor from the previous stage")
        x = out.detach().contiguous()
        dx = torch.zeros_like(x) if self.has_backward else None
        self._input_grads[mb] = [dx]
        return x, dx, False

    # -- forward ----------------------------------------------------------------------------------
    def forward_one_chunk(self, args: Tuple[Any, ...] = (), kwargs: Optional[Dict[str, Any]] = None):
        """Forward of the next microbatch (reference ``_PipelineStage.py:452-510``)."""
        mb = self.fwd_chunk_id
        try:
            if self.is_native:
                output, flat_inputs = self._forward_native(mb, args, kwargs or {})
            else:
                output, flat_inputs = self._forward_eager(mb, args, kwargs or {})
        except Exception as e:
            raise RuntimeError(f"{self.log_prefix} failed to run forward of microbatch {mb}: {e}") from e
        if type(output) is list:
            output = tuple(output)
        output_tuple = output if type(output) is tuple else (output,)
        self._check_live_shapes(flat_inputs, output_tuple)
        self.output_chunks.append(output)
        self.fwd_cache[mb] = (output_tuple, flat_inputs)
        self._fwd_done[mb] = True
        self.fwd_chunk_id += 1
        return output

    def _check_live_shapes(self, flat_inputs, output_tuple) -> None:
        """Hook for stages that were given example values (``ManualPipelineStage``)."""

    def _exported_input_shape(self):
        """The per-sample input shape a stage was exported on (None for a stage traced symbolically, which
        holds no shapes).  What an exported stage computes was fixed for that shape (a mask cut for that
        sequence length, a sliding window known to cover it, position indices): the launch lists run any
        batch size, samples being independent, but no other sequence length."""
        if "_exported_shape" not in self.__dict__:
            shape = None
            graph = getattr(self.submod, "graph", None)
            inputs = [n for n in graph.nodes if n.op == "placeholder"] if graph is not None else []
            if len(inputs) == 1 and hasattr(inputs[0].meta.get("val"), "shape") and \
                    any(b.startswith("_folded_constant_") for b, _ in self.submod.named_buffers(recurse=False)):
                shape = tuple(int(d) for d in inputs[0].meta["val"].shape[1:])
            self._exported_shape = shape
        return self._exported_shape

    def _forward_native(self, mb, args, kwargs):
        if self._mode_bound_dropouts and any(m.training for m in self._mode_bound_dropouts):
            raise RuntimeError(
                f"{self.log_prefix} was lowered to launch lists in eval mode, where its dropout layers (p > 0) do "
                "nothing, and its module is in training mode now: the launch lists hold no dropout.  Set the mode "
                "before the stage is built (a stage built in training mode with p > 0 runs through torch "
                "autograd), or set the dropout probabilities to 0")
        sp = self._stage_program()
        x, dx_target, patch = self._input_for(mb, args, kwargs)
        expected = self._exported_input_shape()
        if expected is not None and tuple(x.shape[1:]) != expected:
            raise RuntimeError(f"{self.log_prefix} was exported on inputs of shape [batch, {', '.join(map(str, expected))}] "
                               f"and holds constants made for it; got {tuple(x.shape)} (build the pipeline on an "
                               "example of the shape it will run on)")
        prog = sp.mbs.get(mb)
        if patch:
            xc = None
            if not x.is_contiguous() or (x.data_ptr() % 16):
                xc = torch.empty(x.shape, dtype=x.dtype, device=x.device)
                N.strided_copy_nd(xc, x)
                x = xc
            key = (tuple(x.shape), x.dtype)
            if prog is None or prog.in_key[:2] != key:
                slot = torch.empty(x.shape, dtype=x.dtype, device=self.device)
                prog = sp.build(mb, slot, None)
                prog.input_patches = [(lst, k, q) for lst in (prog.F, prog.I, prog.W)
                                      for (k, q) in lst.find_pointer(slot.data_ptr())]
            for lst, k, q in prog.input_patches:
                lst[k].p[q] = x.data_ptr()
            # a deferred weight-gradient pass on another stream still reads the copy after the
            # input-gradient pass has dropped the forward cache: the slot keeps it until its next forward
            prog.input_copy = xc
            if _CHECK_INPUTS and x.dtype == torch.int64:
                self._check_ids(x)
        else:
            key = (tuple(x.shape), x.dtype, x.data_ptr(), P._p(dx_target))
            if prog is None or prog.in_key != key:
                prog = sp.build(mb, x, dx_target)
        prog.F.run()
        return prog.output, [x]

    def _check_ids(self, ids):
        for blk in self._blocks:
            table = getattr(blk, "wte", None) or getattr(blk, "word_embeddings", None)
            if table is not None:
                vocab = table.weight.shape[0]
                if bool(((ids < 0) | (ids >= vocab)).any()):
                    raise RuntimeError(f"{self.log_prefix} token id outside [0, {vocab})")
                return

    def _received(self, value):
        if isinstance(value, torch.Tensor):
            value = value.detach()
            if self.has_backward and value.is_floating_point():
                value = value.requires_grad_(True)
        return value

    def _forward_eager(self, mb, args, kwargs):
        routes = getattr(self, "_arg_routes", None)
        if self.is_first:
            composite_args, composite_kwargs = args, kwargs
        elif routes is not None:
            # inputs as the pipe's graph wires them: any earlier stage, any of its outputs
            recv = []
            for src, out_idx in routes:
                producer = self._stages.get(src)
                if producer is None:
                    raise RuntimeError(
                        f"{self.log_prefix} takes an input from stage {src}: pass every stage of the "
                        "pipeline to the schedule")
                if not producer._fwd_done.get(mb):
                    raise RuntimeError(
                        f"{self.log_prefix} activation of microbatch {mb} from stage {src} has not been produced")
                out = producer.output_chunks[mb]
                recv.append(self._received(out[out_idx] if out_idx is not None else out))
            composite_args, composite_kwargs = tuple(recv), {}
        else:
            prev = self._prev
            if prev is None:
                raise RuntimeError(
                    f"{self.log_prefix} is not linked to stage {self.stage_index - 1}: pass every stage "
                    "of the pipeline to the schedule")
            if not prev._fwd_done.get(mb):
                raise RuntimeError(f"{self.log_prefix} activation of microbatch {mb} has not been produced")
            out = prev.output_chunks[mb]
            outs = out if isinstance(out, tuple) else (out,)
            composite_args, composite_kwargs = tuple(self._received(o) for o in outs), {}
        output = self.submod(*composite_args, **composite_kwargs)
        flat_inputs = flatten_args(composite_args) + flatten_args(composite_kwargs)
        return output, flat_inputs

    # -- loss ---------------------------------------------------------------------------------------
    def compute_loss(self, loss_fn, output, target, mb: int) -> torch.Tensor:
        """Runs ``loss_fn`` for microbatch ``mb`` of the last stage
        (reference ``PipelineSchedule.py:39-45``)."""
        if not self.is_native:
            return loss_fn(output, target)
        prog = self._program.mbs[mb]
        native = as_native_loss(loss_fn)
        logits = getattr(prog.output, "_pp_padded", None)
        if native is not None and (not getattr(native, "_requires_2d", False) or output.dim() == 2):
            V = output.shape[-1]
            if logits is None:
                logits = prog.output.reshape(-1, V)
            rows = logits.shape[0]
            if target.numel() != rows or target.dtype != torch.int64:
                raise RuntimeError(
                    f"cross entropy expects {rows} int64 targets, got {target.numel()} of {target.dtype}")
            if not target.is_contiguous():
                tc = torch.empty(target.shape, dtype=target.dtype, device=target.device)
                N.strided_copy_nd(tc, target)
                target = tc
            # the launch list is cached per microbatch slot by what shapes it (never by the identity of
            # the loss object, which a later object may reuse); the loss itself goes to a buffer that is
            # allocated afresh every step, so the tensors a caller keeps are not overwritten by later steps
            key = (native.ignore_index, V, self.has_backward)
            entry = prog.loss_ops.get(key)
            if entry is None:
                ws = torch.empty(rows + 2, dtype=torch.float32, device=self.device)
                dl = prog.output_grad_buf.view(logits.shape) if self.has_backward else None
                lst = P.OpList()
                lst.append(P.op_ce_loss(logits, target, ws[:1], dl, ws, V, native.ignore_index))
                lst.freeze()
                entry = (lst, ws)
                prog.loss_ops[key] = entry
            lst, _ = entry
            if self._step_losses is None or mb >= self._step_losses.numel():
                # (a pipe built from one microbatch's inputs does not know the schedule's microbatch
                # count; losses handed out earlier keep their old buffer)
                self._step_losses = torch.empty(max(self.chunks, 2 * (mb + 1), 8), dtype=torch.float32,
                                                device=self.device)
            if _CHECK_INPUTS:
                bad = ((target < 0) | (target >= V)) & (target != native.ignore_index)
                if bool(bad.any()):
                    raise RuntimeError(f"cross entropy target outside [0, {V}) in microbatch {mb}")
            loss = self._step_losses[mb:mb + 1]
            lst[0].p[1] = target.data_ptr()
            lst[0].p[2] = loss.data_ptr()
            lst.run()
            self._loss_targets = getattr(self, "_loss_targets", {})
            self._loss_targets[mb] = target  # keep alive until the kernel has run
            return loss.view(())
        # any other callable: autograd on a detached copy of the output
        leaf = output.detach().requires_grad_(self.has_backward)
        loss = loss_fn(leaf, target)
        self._bridge[mb] = (leaf, loss)
        return loss

    # -- backward -----------------------------------------------------------------------------------
    def backward_one_chunk(self, loss=None):
        """Full backward of the next microbatch (reference ``_PipelineStage.py:512-550``):
        input-gradient pass followed by the weight-gradient pass."""
        mb = self.bwd_chunk_id
        if self.is_native:
            self._backward_input_native(mb, loss)
            self.bwd_chunk_id += 1
            if self.batch_weight_grads and self.split_backward:
                return                      # the weight gradients of the step follow in one batched pass
            self._backward_weight_native(mb)
            self.bwd_weight_chunk_id += 1
        else:
            self._backward_eager(mb, loss)
            self.bwd_chunk_id += 1
            self.bwd_weight_chunk_id += 1

    def backward_input_one_chunk(self, loss=None):
        """Input-gradient pass only (dI): produces the gradient the previous stage waits for and
        keeps what the weight-gradient pass needs."""
        if not self.is_native:
            raise RuntimeError("split backward needs a native stage")
        if not self.split_backward:
            raise RuntimeError("enable split_backward (zero-bubble schedules do) before the first forward")
        mb = self.bwd_chunk_id
        self._backward_input_native(mb, loss)
        self.bwd_chunk_id += 1

    def backward_weight_one_chunk(self):
        """Weight-gradient pass (dW) of the oldest microbatch whose input-gradient pass has run."""
        if not self.is_native:
            raise RuntimeError("split backward needs a native stage")
        if self.batch_weight_grads:
            return                          # deferred to ``flush_weight_grads``
        mb = self.bwd_weight_chunk_id
        if mb >= self.bwd_chunk_id:
            raise RuntimeError(f"{self.log_prefix} weight-gradient pass of microbatch {mb} before its input-gradient pass")
        self._backward_weight_native(mb)
        self.bwd_weight_chunk_id += 1

    @property
    def prefers_batched_weight_grads(self) -> bool:
        """Whether one batched weight-gradient pass per step pays for this stage whatever the schedule:
        stages whose blocks say so (expert weights: their fp32 accumulators outweigh a microbatch's
        operands, so moving them once per step instead of once per microbatch is the larger part of the
        pass)."""
        return bool(self._blocks) and any(getattr(b, "_pp_batch_weight_grads", False) for b in self._blocks)

    def flush_weight_grads(self) -> int:
        """Runs the weight-gradient passes of all microbatches whose input-gradient pass has run and whose
        weight-gradient pass has not, as one batched pass (``_program.BatchedW``: every weight-gradient GEMM
        once over all of them, accumulation order and bits as microbatch by microbatch).  Returns how many
        microbatches it covered."""
        if not self.is_native:
            return 0
        lo, hi = self.bwd_weight_chunk_id, self.bwd_chunk_id
        if hi <= lo:
            return 0
        if hi - lo == 1:
            self._backward_weight_native(lo)
            self.bwd_weight_chunk_id = hi
            return 1
        sp = self._program
        self._start_accumulation_if_cleared(sp)
        sp.batched_w(tuple(range(lo, hi))).run(init=not sp.acc_initialized)
        self._after_weight_pass(sp)
        self.bwd_weight_chunk_id = hi
        return hi - lo

    def _backward_input_native(self, mb, loss):
        if mb not in self.fwd_cache:
            raise RuntimeError(f"{self.log_prefix} backward of microbatch {mb} before its forward")
        self.fwd_cache.pop(mb)
        prog = self._program.mbs[mb]
        if self.is_last:
            if mb in self._bridge:
                leaf, lss = self._bridge.pop(mb)
                lss.backward()
                prog.output_grad.copy_(leaf.grad)
            elif loss is None:
                raise RuntimeError(f"{self.log_prefix} last stage needs the loss of microbatch {mb}")
        else:
            nxt = self._next
            if nxt is None or not nxt._bwd_done.get(mb):
                raise RuntimeError(f"{self.log_prefix} gradient of microbatch {mb} has not been produced")
            if not nxt.is_native:
                g = nxt._input_grads[mb][0]
                prog.output_grad.copy_(g)
        prog.I.run()
        self._bwd_done[mb] = True
        self.grads_input = [prog.input_grad]

    @staticmethod
    def _start_accumulation_if_cleared(sp):
        fp32_params = sp.arena.dtype == torch.float32
        if (fp32_params or sp.grads_handed_over) and sp.acc_initialized and \
                any(p.grad is None for _, p in sp.arena.named):
            # the user cleared the gradients (optimizer.zero_grad()): start a new accumulation
            sp.acc_initialized = False
            sp.grads_handed_over = False

    @staticmethod
    def _after_weight_pass(sp):
        sp.acc_initialized = True
        if sp.arena.dtype == torch.float32:
            for _, p in sp.arena.named:
                if p.grad is None:
                    p.grad = p.main_grad

    def _backward_weight_native(self, mb):
        sp = self._program
        prog = sp.mbs[mb]
        self._start_accumulation_if_cleared(sp)
        sp.set_accumulate_mode(prog, init=not sp.acc_initialized)
        prog.W.run()
        self._after_weight_pass(sp)

    def _grad_from(self, consumer: "PipelineStageBase", pos: int, mb: int):
        if not consumer._bwd_done.get(mb):
            raise RuntimeError(
                f"{self.log_prefix} gradient of microbatch {mb} from stage {consumer.stage_index} has not been produced")
        if consumer.is_native:
            return consumer._program.mbs[mb].input_grad
        return consumer._input_grads[mb][pos]

    def _backward_eager(self, mb, loss):
        stage_output, input_values = self.fwd_cache.pop(mb)
        consumers = getattr(self, "_out_consumers", None)
        if self.is_last:
            bwd_kwargs = {"stage_output": loss, "output_grads": None, "input_values": input_values}
        elif consumers is not None:
            # every output with its gradient: the sum over the stages that consumed it (the reference
            # stops at one consumer per output, ``_PipelineStage.py:790-793``)
            outs, grads = [], []
            for out_idx, users in consumers.items():
                total = None
                for dst, pos in users:
                    g = self._grad_from(self._stages[dst], pos, mb)
                    if g is not None:
                        total = g if total is None else total + g
                if total is not None:
                    if out_idx is not None:
                        outs.append(stage_output[out_idx])
                    elif isinstance(stage_output, (tuple, list)) and len(stage_output) == 1:
                        outs.append(stage_output[0])  # the cache holds a single output as a 1-tuple
                    else:
                        outs.append(stage_output)
                    grads.append(total)
            bwd_kwargs = {"stage_output": tuple(outs), "output_grads": tuple(grads), "input_values": input_values}
        else:
            nxt = self._next
            if nxt is None:
                raise RuntimeError(f"{self.log_prefix} is not linked to stage {self.stage_index + 1}")
            grads = (self._grad_from(nxt, 0, mb),) if nxt.is_native else None
            if grads is None:
                if not nxt._bwd_done.get(mb):
                    raise RuntimeError(f"{self.log_prefix} gradient of microbatch {mb} has not been produced")
                grads = tuple(nxt._input_grads[mb])
            bwd_kwargs = {"stage_output": stage_output, "output_grads": grads, "input_values": input_values}
        self.grads_input = stage_backward(**bwd_kwargs)
        self._input_grads[mb] = list(self.grads_input)
        self._bwd_done[mb] = True


def _stage_wiring(pipe, stage_index: int):
    """How the pipe's graph feeds stage ``stage_index`` and who consumes its outputs
    (reference ``_PipelineStage.py:649-768``).  Returns (routes, consumers, is_chain):
    routes: per positional input (source stage, output index or None), None for the first stage whose
    inputs are the user's; consumers: output index (None: the single output) -> [(stage, input
    position)]; is_chain: the only input is the whole output of the previous stage and the only
    consumer of the output is the next stage."""
    import operator
    nodes = [n for n in pipe.split_gm.graph.nodes if n.op == "call_module" and str(n.target).startswith("submod_")]
    index_of = {n: i for i, n in enumerate(nodes)}
    node = nodes[stage_index]

    def source(arg):
        out_idx = None
        while arg.op == "call_function" and arg.target is operator.getitem:
            out_idx = arg.args[1] if out_idx is None else out_idx
            arg = arg.args[0]
        return arg, out_idx

    routes = []
    for arg in node.args:
        src, out_idx = source(arg)
        if src.op == "placeholder":
            if stage_index != 0:
                raise NotImplementedError(
                    f"stage {stage_index} reads the model input '{src.name}': only the first stage may "
                    "(reference _PipelineStage.py:462-470)")
            routes = None
            break
        if src not in index_of:
            raise RuntimeError(f"stage {stage_index}: unsupported input node {src.format_node()}")
        routes.append((index_of[src], out_idx))
    consumers = {}
    for user in node.users:
        if user.op == "call_function" and user.target is operator.getitem:
            dsts = consumers.setdefault(user.args[1], [])
            for gu in user.users:
                if gu in index_of:
                    dsts += [(index_of[gu], pos) for pos, a in enumerate(gu.args) if a is user]
        elif user in index_of:
            consumers.setdefault(None, [])
            consumers[None] += [(index_of[user], pos) for pos, a in enumerate(user.args) if a is node]
    chain_in = stage_index == 0 or routes == [(stage_index - 1, None)]
    chain_out = stage_index == len(nodes) - 1 or consumers == {None: [(stage_index + 1, 0)]}
    if stage_index == 0 and len(node.args) != 1:
        chain_in = True  # the lowering itself checks that a native first stage takes one tensor
    return routes, consumers, chain_in and chain_out


class PipelineStage(PipelineStageBase):
    """A stage built from a ``Pipe`` (reference ``_PipelineStage.py:818-833``).  Inputs follow the
    pipe's graph: a stage may take several values, from any earlier stage (skip connections,
    reference ``test/test_skip_conn.py:20-45``); such a stage runs through autograd, and so does one
    whose output feeds more than the next stage."""

    def __init__(self, pipe, stage_index: int, device, group=None, **kw):
        self.pipe = pipe
        self.pipe_info = pipe.info()
        submod = pipe.get_stage_module(stage_index)
        routes, consumers, is_chain = _stage_wiring(pipe, stage_index)
        if not is_chain:
            kw["force_eager"] = True
        super().__init__(submod, stage_index, pipe.num_stages, device, self.pipe_info.num_chunks,
                         group, **kw)
        if not is_chain or not self.is_native:
            self._arg_routes = routes
            self._out_consumers = consumers if stage_index != pipe.num_stages - 1 else None


class ManualPipelineStage(PipelineStageBase):
    """A stage built from a hand-written module (reference ``ManualPipelineStage.py:178-307``).
    ``input_args`` / ``output_args`` are example microbatch values; the reference sizes its receive
    buffers from them and compares them between neighbouring ranks (``ManualPipelineStage.py:342-439``).
    Here buffers take their shapes from the live tensors, and the examples are a contract that is
    checked: every forward compares the shape and dtype of what the stage receives and produces with
    the examples and raises ``ValueError`` on a mismatch; ``validate_stage_shapes`` compares the
    examples of consecutive stages."""

    def __init__(self, submodule: nn.Module, stage_index: int, num_stages: int, device,
                 num_microbatches: int, input_args=None, output_args=None, group=None, **kw):
        super().__init__(submodule, stage_index, num_stages, device, num_microbatches, group, **kw)
        self.inputs = _to_tuple(input_args)
        self.outputs = _to_tuple(output_args)

    @staticmethod
    def _meta(values):
        return [(tuple(v.shape), v.dtype) for v in values if isinstance(v, torch.Tensor)]

    def _check_live_shapes(self, flat_inputs, output_tuple) -> None:
        for what, examples, live in (("input", self.inputs, flat_inputs), ("output", self.outputs, output_tuple)):
            want = self._meta(examples)
            if not want:
                continue
            got = self._meta(live)
            if got != want:
                raise ValueError(
                    f"{self.log_prefix} {what} of microbatch {self.fwd_chunk_id} has shape/dtype {got}, "
                    f"but the stage was built with example {what}s {want}")


def validate_stage_shapes(pipeline_stages: List["ManualPipelineStage"]) -> None:
    """Checks that the example values the stages were built with fit together (reference
    ``ManualPipelineStage.py:342-439``, without its all-gather: every stage lives in this process):
    all stages agree on the number of stages, and the example output of stage i has the shapes of the
    example input of stage i + 1 wherever both were given.  Raises ``ValueError``."""
    if len(pipeline_stages) == 0:
        raise ValueError("No pipeline stages provided.")
    ordered = sorted(pipeline_stages, key=lambda st: st.stage_index)
    num_stages = ordered[0].num_stages
    for st in ordered:
        if st.num_stages != num_stages:
            raise ValueError(
                f"Stage id {st.stage_index} has num stages ({st.num_stages}) which does not match num stages "
                f"({num_stages}) of other stages.")
    for a, b in zip(ordered, ordered[1:]):
        if b.stage_index != a.stage_index + 1:
            continue
        out = [list(s) for s, _ in ManualPipelineStage._meta(a.outputs)]
        inp = [list(s) for s, _ in ManualPipelineStage._meta(b.inputs)]
        if out and inp and out != inp:
            raise ValueError(
                f"Stage_id {a.stage_index} output shape {out} at does not match stage_id {b.stage_index} "
                f"input shape {inp}.")


def _to_tuple(v):
    if v is None:
        return ()
    return tuple(v) if isinstance(v, (tuple, list)) else (v,)


def link_stages(stages: List[PipelineStageBase]) -> List[PipelineStageBase]:
    """Wires the device-local hand-off between consecutive stages and returns them sorted."""
    ordered = sorted(stages, key=lambda s: s.stage_index)
    idx = [s.stage_index for s in ordered]
    if len(set(idx)) != len(idx):
        raise ValueError(f"duplicate stage indices {idx}")
    by_index = {s.stage_index: s for s in ordered}
    for s in ordered:
        s._prev = by_index.get(s.stage_index - 1)
        s._next = by_index.get(s.stage_index + 1)
        s._stages = by_index
    return ordered
