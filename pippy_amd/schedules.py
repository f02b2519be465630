"""Pipeline schedules (mirrors ``pippy/PipelineSchedule.py`` of the reference).

Same classes, constructor arguments, ``step`` / ``_step_microbatches`` contract and error types.
The difference is where stages live: the reference runs one process per pipeline rank and each
process executes the loop of its own rank; here all stages are virtual stages of one GPU, so a
schedule builds the per-rank programs from the reference's index formulas
(``_schedule_order.py``), merges them into one dependency-respecting order and executes that.
Per-stage forward order and backward order are unchanged (microbatches ascending), hence so are
all results, including the fp32 gradient accumulation order.

Single-stage schedule classes (``ScheduleGPipe``, ``Schedule1F1B``) accept, besides one stage as
in the reference, the list of all stages of the pipeline: that is how a multi-stage pipeline is
run on one device.
"""
from __future__ import annotations

import logging
import os
from abc import ABC, abstractmethod
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple, Union

import torch
from torch.profiler import record_function
from contextlib import nullcontext

from . import _schedule_order as order
from . import microbatch as _microbatch
from .microbatch import TensorChunkSpec, copy_into_rows, merge_chunks, split_args_kwargs_into_chunks
from .stage import PipelineStageBase, link_stages

logger = logging.getLogger(__name__)


class _RunningMerge:
    """Builds the merged output of a step while the step is still running: every microbatch output of
    the last stage is copied into its rows of the result as soon as its forward pass has been issued,
    on a stream of its own (an HBM-bound copy next to the MFMA-bound kernels of the other passes),
    instead of all of them after the last backward pass.  The result is the same freshly allocated
    contiguous tensor that ``merge_chunks`` returns.  Used when the output is one tensor merged along
    dimension 0 and all microbatches have the same size; anything else is merged at the end as before."""

    def __init__(self, n_microbatches: int, device):
        self.n = n_microbatches
        self.stream = torch.cuda.Stream(device=device)
        self.out: Optional[torch.Tensor] = None
        self.rows = 0
        self.done = 0
        self.ok = True
        self.wrap = None

    def reset(self):
        self.out, self.rows, self.done, self.ok, self.wrap = None, 0, 0, True, None

    def add(self, m: int, chunk, produced_on: "torch.cuda.Stream", main: "torch.cuda.Stream"):
        if not self.ok:
            return
        if type(chunk) in (tuple, list) and len(chunk) == 1:     # exported models return 1-tuples
            self.wrap, chunk = type(chunk), chunk[0]
        if not isinstance(chunk, torch.Tensor) or not chunk.is_cuda or chunk.dim() == 0 or m != self.done:
            self.ok = False
            return
        if self.out is None:
            self.rows = chunk.shape[0]
            with torch.cuda.stream(main):      # allocated (and later freed) under the caller's stream
                self.out = torch.empty((self.n * self.rows,) + tuple(chunk.shape[1:]), dtype=chunk.dtype,
                                       device=chunk.device)
            self.out.record_stream(self.stream)
        elif chunk.shape != (self.rows,) + tuple(self.out.shape[1:]) or chunk.dtype != self.out.dtype:
            self.ok = False
            return
        ready = torch.cuda.Event()
        ready.record(produced_on)
        self.stream.wait_event(ready)
        with torch.cuda.stream(self.stream):
            copy_into_rows(self.out, m * self.rows, chunk)
        self.done += 1

    def result(self, main: "torch.cuda.Stream") -> Optional[torch.Tensor]:
        """The merged tensor once every microbatch has been added (the caller's stream then waits for
        the copies), else None."""
        if not self.ok or self.out is None or self.done != self.n:
            return None
        main.wait_stream(self.stream)
        return self.out if self.wrap is None else self.wrap([self.out])


class PipelineSchedule(ABC):
    def __init__(self, n_microbatches: int, loss_fn: Optional[Callable[..., torch.Tensor]] = None,
                 output_merge_spec: Optional[Union[Dict[str, Any], Tuple[Any]]] = None):
        self._n_microbatches = n_microbatches
        self._loss_fn = loss_fn
        self._output_merge_spec = output_merge_spec
        self._has_backward = self._loss_fn is not None
        self._pipe_info = None
        self._internal_losses: List[torch.Tensor] = []
        self._stages: List[PipelineStageBase] = []
        self._by_index: Dict[int, PipelineStageBase] = {}
        #: spread the virtual stages over two HIP streams (natively lowered stages only): True, False, or
        #: None = when a stage pass holds enough work for it (see ``_stage_streams``)
        self.concurrent_stages: Optional[bool] = None
        self._small_step: Dict[Any, bool] = {}
        self._streams = None
        self._w_streams = None
        self._events: Dict[Any, Any] = {}
        #: run the weight-gradient passes of a stage as ONE batched pass after its last input-gradient pass
        #: (every weight-gradient GEMM once over all microbatches, bit-identical accumulators, see
        #: ``_program.BatchedW``).  None: where it pays - stages with expert weights, whose fp32 accumulators
        #: outweigh a microbatch's operands (53.2 against 58.3 ms per Mixtral-style step), and a schedule's
        #: only native stage, whose passes have no other stage's kernels to run beside (the accumulators then
        #: move once per step instead of once per microbatch: 375 against 386 ms per Llama-stage step); with
        #: several stages on this device the batched pass at the end of the step no longer hides behind other
        #: stages' kernels (43.5 against 43.2 ms per GPT-2-small step);
        #: True / False: every native stage / none
        self.batch_weight_grads: Optional[bool] = None
        #: copy microbatch outputs into the merged result while the step runs (see ``_RunningMerge``)
        self.merge_while_running = True
        self._running_merge: Optional[_RunningMerge] = None
        self._merge_active: Optional[_RunningMerge] = None
        logger.info(f"Using {self.__class__.__name__}")

    # -- losses (reference ``PipelineSchedule.py:39-80``) -------------------------------------------
    def _maybe_compute_loss(self, stage, output, target_mbs, mb_index):
        if not (stage.is_last and self._has_backward):
            return
        if target_mbs is None:
            raise RuntimeError("a loss function was given but no target")
        self._internal_losses.append(self._compute_loss(stage, output, target_mbs[mb_index], mb_index))

    def _maybe_get_loss(self, stage, mb_index):
        """The loss that the backward pass of microbatch ``mb_index`` starts from: only the last
        stage of a training schedule has one."""
        held = len(self._internal_losses)
        if 0 <= mb_index < held:
            return self._internal_losses[mb_index] if (stage.is_last and self._has_backward) else None
        if held:
            raise RuntimeError(
                f"Loss for microbatch {mb_index} is not available. "
                f"Available losses for microbatches: {self._internal_losses}")
        return None

    def _update_losses(self, stages, losses):
        """Hands the step's losses to the caller's list and forgets them."""
        stages = stages if isinstance(stages, list) else [stages]
        if losses is not None and any(st.is_last for st in stages):
            if len(self._internal_losses) != self._n_microbatches:
                raise RuntimeError(
                    f"Expecting {self._n_microbatches} losses but got {len(self._internal_losses)}")
            losses[:] = self._internal_losses
        self._internal_losses.clear()

    def _compute_loss(self, stage, output, target, mb_index):
        return stage.compute_loss(self._loss_fn, output, target, mb_index)

    # -- input checks (reference ``PipelineSchedule.py:114-152``) -----------------------------------
    def _require_microbatch_list(self, mbs, name: str):
        if not isinstance(mbs, list):
            raise TypeError(f"{name} must be a list but got a {type(mbs)}")
        if len(mbs) != self._n_microbatches:
            raise ValueError(f"Expecting {self._n_microbatches} {name} but got {len(mbs)}")

    def _check_inputs(self, arg_mbs=None, kwarg_mbs=None, target_mbs=None, losses=None):
        """Validates the per-microbatch lists; absent positional / keyword lists become empty ones."""
        given = {"arg_mbs": arg_mbs, "kwarg_mbs": kwarg_mbs, "target_mbs": target_mbs}
        for name, mbs in given.items():
            if mbs is not None:
                self._require_microbatch_list(mbs, name)
        if losses is not None and not isinstance(losses, list):
            raise TypeError(f"losses must be a list but got a {type(losses)}")
        n = self._n_microbatches
        return (arg_mbs if arg_mbs is not None else [()] * n,
                kwarg_mbs if kwarg_mbs is not None else [{}] * n)

    def _split_inputs(self, args: Tuple[Any, ...], kwargs: Optional[Dict[str, Any]] = None):
        """Full batch -> microbatches (reference ``PipelineSchedule.py:157-187``): the chunk specs are
        those the pipe was traced with, dimension 0 everywhere without a pipe."""
        n = self._n_microbatches
        if not args and not kwargs:
            return [()] * n, [{}] * n
        info = self._pipe_info
        return split_args_kwargs_into_chunks(args, kwargs, n,
                                             info.args_chunk_spec if info is not None else None,
                                             info.kwargs_chunk_spec if info is not None else None)

    def _merge_outputs(self, output_chunks: List[Any]) -> Any:
        """Microbatch outputs -> full batch (reference ``PipelineSchedule.py:189-197``)."""
        return merge_chunks(output_chunks, self._output_merge_spec)

    # -- execution of a merged action order on the device -------------------------------------------
    def _stage_streams(self, arg_mbs=None):
        """The HIP stream of every virtual stage (two streams, half of the stages on each), or None
        when the actions run on the caller's stream.

        Stages are independent between hand-offs, exactly like ranks of a real pipeline, so their
        launch lists may overlap on the device: a kernel that leaves CUs idle (a GEMM with fewer
        tiles than CUs, the tail of any grid, the dependent chain of a causal attention block)
        shares the machine with a kernel of another stage.  Only natively lowered stages qualify:
        their buffers are allocated once, so no allocator block changes hands between streams."""
        if self.concurrent_stages is False or os.environ.get("PIPPY_AMD_SERIAL_STAGES") == "1":
            return None
        if len(self._stages) < 2 or not all(getattr(st, "is_native", False) for st in self._stages):
            return None
        if self.concurrent_stages is None and os.environ.get("PIPPY_AMD_CONCURRENT_STAGES") != "1" \
                and self._is_small_step(arg_mbs):
            return None
        dev = self._stages[0].device
        if torch.device(dev).type != "cuda":
            return None
        if self._streams is None or len(self._streams) != len(self._stages):
            # two streams, the first half of the stages on one and the second half on the other: a
            # second kernel in flight fills the idle CUs of the first, more of them only contend
            # (GPT-2-small, 4 stages: 46.6 ms per step against 47.1 with a stream per stage; the
            # BERT-base inference step 11.1 against 11.5 ms)
            n = len(self._stages)
            pool = [torch.cuda.Stream(device=dev) for _ in range(min(n, 2))]
            order_ = sorted(st.stage_index for st in self._stages)
            self._streams = {s: pool[(k * len(pool)) // n] for k, s in enumerate(order_)}
            # deferred weight-gradient passes ("W" actions) read per-microbatch buffers only, so they
            # get a stream of their own next to the stage's forward / input-gradient stream
            self._w_streams = {st.stage_index: torch.cuda.Stream(device=dev) for st in self._stages}
            self._events = {}
        return self._streams

    #: below this many floating-point operations per stage pass (2 x parameters x rows of a microbatch) the
    #: kernels of a pass are shorter than what switching streams and recording events costs the host
    #: (about 50 us per pass): the README-sized MLP runs 0.5 ms per step on one stream, 1.1 ms on two
    _CONCURRENT_MIN_FLOP = 1.0e10

    def _is_small_step(self, arg_mbs) -> bool:
        first = None
        if arg_mbs:
            first = next((a for a in arg_mbs[0] if isinstance(a, torch.Tensor)), None)
        if first is None:
            return False
        rows = first.numel() if not first.is_floating_point() or first.dim() < 2 else first.numel() // first.shape[-1]
        got = self._small_step.get(rows)
        if got is None:
            params = max(sum(p.numel() for p in st.submod.parameters()) for st in self._stages)
            got = self._small_step[rows] = 2.0 * params * rows < self._CONCURRENT_MIN_FLOP
        return got

    def _event(self, key):
        ev = self._events.get(key)
        if ev is None:
            ev = self._events[key] = torch.cuda.Event()
        return ev

    def _execute(self, actions: Sequence[order.Action], arg_mbs, kwarg_mbs, target_mbs):
        streams = self._stage_streams(arg_mbs)
        self._choose_weight_grad_batching()
        if streams is None:
            for kind, s, m in actions:
                self._run_action(kind, s, m, arg_mbs, kwarg_mbs, target_mbs)
                if kind in ("B", "I"):
                    self._flush_if_last(s)
            return
        # hand-offs become events: forward (s, m) waits for forward (s-1, m), backward (s, m) for
        # backward (s+1, m); everything of one stage stays in order on that stage's stream
        main = torch.cuda.current_stream()
        start = self._event("start")
        start.record(main)
        merger = self._merger(main)
        w_streams = self._w_streams
        for st in list(streams.values()) + list(w_streams.values()):
            st.wait_event(start)
        last = max(streams)
        used_w = set()
        for kind, s, m in actions:
            if kind == "W":
                if self._by_index[s].batch_weight_grads:
                    continue        # covered by the batched pass behind the stage's last input-gradient pass
                # after the input-gradient pass of the same microbatch; W passes of a stage stay in
                # microbatch order among themselves, which keeps the accumulation order
                wm = self._by_index[s].bwd_weight_chunk_id
                st = w_streams[s]
                used_w.add(s)
                with torch.cuda.stream(st):
                    st.wait_event(self._event(("B", s, wm)))
                    self._run_action(kind, s, m, arg_mbs, kwarg_mbs, target_mbs)
                continue
            st = streams[s]
            with torch.cuda.stream(st):
                if kind == "F":
                    if s > 0:
                        st.wait_event(self._event(("F", s - 1, m)))
                elif kind in ("B", "I"):
                    if s < last:
                        st.wait_event(self._event(("B", s + 1, m)))
                self._run_action(kind, s, m, arg_mbs, kwarg_mbs, target_mbs)
                if kind == "F":
                    self._event(("F", s, m)).record(st)
                    if merger is not None and s == last:
                        merger.add(m, self._by_index[s].output_chunks[m], st, main)
                elif kind in ("B", "I"):
                    self._event(("B", s, m)).record(st)
                    if kind == "B":
                        self._flush_if_last(s)
            if kind == "I" and self._by_index[s].batch_weight_grads and \
                    self._by_index[s].bwd_chunk_id == self._n_microbatches:
                # deferred weight gradients: the batched pass runs beside the stage's stream
                wst = w_streams[s]
                used_w.add(s)
                with torch.cuda.stream(wst):
                    wst.wait_event(self._event(("B", s, m)))
                    self._flush_if_last(s)
        for s, st in streams.items():
            done = self._event(("done", s))
            done.record(st)
            main.wait_event(done)
        for s in used_w:
            done = self._event(("done_w", s))
            done.record(w_streams[s])
            main.wait_event(done)
        if merger is not None:
            # also for a caller that drives _step_microbatches itself and never asks for the merged result:
            # the copies read the per-microbatch output buffers that the next step overwrites
            main.wait_stream(merger.stream)

    def _choose_weight_grad_batching(self):
        """Sets ``batch_weight_grads`` (and with it ``split_backward``: per-microbatch gradient buffers) on
        the stages, before the step's first forward pass builds their launch lists."""
        n_native = sum(1 for st in self._stages if getattr(st, "is_native", False))
        for st in self._stages:
            if not getattr(st, "is_native", False) or not self._has_backward:
                continue
            want = self.batch_weight_grads
            if want is None:
                want = st.prefers_batched_weight_grads or n_native == 1
            if want and not st.split_backward:
                st.split_backward = True
            st.batch_weight_grads = bool(want)

    def _flush_if_last(self, s: int):
        stage = self._by_index[s]
        if getattr(stage, "batch_weight_grads", False) and stage.bwd_chunk_id == self._n_microbatches:
            with self._range(f"Stage {s} BackwardWeight batched"):
                stage.flush_weight_grads()

    def _merger(self, main) -> Optional[_RunningMerge]:
        """The running merge of this step, or None when outputs are merged at the end."""
        default_spec = self._output_merge_spec is None or (
            isinstance(self._output_merge_spec, TensorChunkSpec) and self._output_merge_spec.split_dim == 0)
        self._merge_active = None
        if not self.merge_while_running or os.environ.get("PIPPY_AMD_MERGE_AT_END") == "1" or not default_spec \
                or _microbatch._debug_mask_minibatches:
            return None
        if self._running_merge is None or self._running_merge.n != self._n_microbatches:
            self._running_merge = _RunningMerge(self._n_microbatches, main.device)
        self._running_merge.stream.wait_stream(main)
        self._running_merge.reset()
        self._merge_active = self._running_merge
        return self._running_merge

    @staticmethod
    def _range(name: str):
        """A profiler range with the reference's names (``PipelineSchedule.py:540,557``); entering one
        costs tens of microseconds, so it is only opened while a torch profiler is recording."""
        return record_function(name) if torch.autograd.profiler._is_profiler_enabled else nullcontext()

    def _run_action(self, kind, s, m, arg_mbs, kwarg_mbs, target_mbs):
        stage = self._by_index[s]
        if kind == "F":
            with self._range(f"Stage {s} Forward {m}"):
                if stage.fwd_chunk_id != m:
                    raise RuntimeError(f"stage {s}: forward order broken ({stage.fwd_chunk_id} != {m})")
                a = arg_mbs[m] if stage.is_first else ()
                k = kwarg_mbs[m] if stage.is_first else {}
                output = stage.forward_one_chunk(a, k)
                self._maybe_compute_loss(stage, output, target_mbs, m)
        elif kind == "B":
            with self._range(f"Stage {s} Backward {m}"):
                if stage.bwd_chunk_id != m:
                    raise RuntimeError(f"stage {s}: backward order broken ({stage.bwd_chunk_id} != {m})")
                stage.backward_one_chunk(loss=self._maybe_get_loss(stage, m))
        elif kind == "I":
            with self._range(f"Stage {s} BackwardInput {m}"):
                stage.backward_input_one_chunk(loss=self._maybe_get_loss(stage, m))
        elif kind == "W":
            with self._range(f"Stage {s} BackwardWeight {m}"):
                stage.backward_weight_one_chunk()
        else:
            raise ValueError(f"unknown action {kind}")

    @abstractmethod
    def _rank_programs(self) -> List[List[order.Action]]:
        """One action program per virtual pipeline rank."""

    def _step_microbatches(self, arg_mbs: Optional[List] = None, kwarg_mbs: Optional[List] = None,
                           target_mbs: Optional[List] = None, losses: Optional[List] = None):
        """Runs one iteration over lists of microbatches (reference ``PipelineSchedule.py:83-98``)."""
        arg_mbs, kwarg_mbs = self._check_inputs(arg_mbs, kwarg_mbs, target_mbs, losses)
        num_stages = self._stages[0].num_stages
        present = sorted(s.stage_index for s in self._stages)
        if present != list(range(num_stages)):
            raise RuntimeError(
                f"this schedule holds stages {present} of a {num_stages}-stage pipeline; all stages "
                "run as virtual stages on one device, so every stage must be given to the schedule "
                "(there is no inter-process transport)")
        actions = order.merge_rank_programs(self._rank_programs(), num_stages)
        self._execute(actions, arg_mbs, kwarg_mbs, target_mbs)
        self._update_losses(self._stages, losses)

    def step(self, *args, target=None, losses: Optional[List] = None, **kwargs):
        """Runs one iteration on a whole batch: split, run the microbatches, merge
        (reference ``PipelineSchedule.py:254-276,490-514``)."""
        for stage in self._stages:
            stage.clear_runtime_states()
        args_split, kwargs_split = self._split_inputs(args, kwargs)
        if target is not None:
            targets_split = list(torch.tensor_split(target, self._n_microbatches))
        else:
            targets_split = None
        self._merge_active = None
        self._step_microbatches(args_split, kwargs_split, targets_split, losses)
        for stage in self._stages:
            if stage.is_last:
                if self._merge_active is not None:
                    merged = self._merge_active.result(torch.cuda.current_stream())
                    self._merge_active.out = None
                    if merged is not None:
                        return merged
                return self._merge_outputs(stage.output_chunks)
        return None

    def zero_grad(self):
        for stage in self._stages:
            stage.zero_grad()

    def _adopt_stages(self, stages: List[PipelineStageBase]):
        self._stages = link_stages(stages)
        self._by_index = {st.stage_index: st for st in self._stages}
        self._streams = None
        self._num_stages = self._stages[0].num_stages
        self._pipe_info = getattr(self._stages[0], "pipe_info", None)
        for stage in self._stages:
            stage.has_backward = self._has_backward
            # a pipe built from the inputs of ONE microbatch (``pipeline(mod, mb_args=...)``) leaves the
            # microbatch count to the schedule
            stage.chunks = max(stage.chunks, self._n_microbatches)


class PipelineScheduleSingle(PipelineSchedule):
    """Schedules whose ranks own one stage each (reference ``PipelineSchedule.py:225-276``)."""

    def __init__(self, stage: Union[PipelineStageBase, List[PipelineStageBase]], n_microbatches: int,
                 loss_fn: Optional[Callable] = None,
                 output_merge_spec: Optional[Union[Dict[str, Any], Tuple[Any]]] = None):
        super().__init__(n_microbatches=n_microbatches, loss_fn=loss_fn, output_merge_spec=output_merge_spec)
        stages = list(stage) if isinstance(stage, (list, tuple)) else [stage]
        self._adopt_stages(stages)
        self._stage = self._stages[0]


class ScheduleGPipe(PipelineScheduleSingle):
    """All forwards, then all backwards (reference ``PipelineSchedule.py:279-355``)."""

    def _rank_programs(self):
        return [order.gpipe_rank_program(s.stage_index, self._n_microbatches, self._has_backward)
                for s in self._stages]


class Schedule1F1B(PipelineScheduleSingle):
    """One-forward-one-backward (reference ``PipelineSchedule.py:358-449``)."""

    def _rank_programs(self):
        return [order.one_f_one_b_rank_program(s.stage_index, self._num_stages, self._n_microbatches,
                                               self._has_backward) for s in self._stages]


class ScheduleZeroBubble(PipelineScheduleSingle):
    """1F1B with the backward split into an input-gradient and a deferred weight-gradient pass.
    Not part of the reference (its backward is one fused autograd call); needs native stages."""

    def __init__(self, stage, n_microbatches, loss_fn=None, output_merge_spec=None):
        super().__init__(stage, n_microbatches, loss_fn, output_merge_spec)
        if not self._has_backward:
            raise ValueError("a zero-bubble schedule needs a loss function")
        for s in self._stages:
            if not s.is_native:
                raise RuntimeError("zero-bubble needs stages that lower to native input/weight passes")
            s.split_backward = True

    def _rank_programs(self):
        return [order.zero_bubble_rank_program(s.stage_index, self._num_stages, self._n_microbatches)
                for s in self._stages]


class PipelineScheduleMulti(PipelineSchedule):
    """Schedules whose ranks own several stages (reference ``PipelineSchedule.py:452-514``)."""

    def __init__(self, stages: List[PipelineStageBase], n_microbatches: int,
                 loss_fn: Optional[Callable] = None,
                 output_merge_spec: Optional[Union[Dict[str, Any], Tuple[Any]]] = None):
        if len(stages) <= 1:
            raise ValueError(f"Multi-stage schedule expects at least two stages but got {len(stages)}")
        super().__init__(n_microbatches=n_microbatches, loss_fn=loss_fn, output_merge_spec=output_merge_spec)
        self._adopt_stages(list(stages))
        self.pp_group_size = self._stages[0].group_size

    def _local_stages(self, rank: int) -> List[int]:
        return [s.stage_index for s in self._stages if s.group_rank == rank]


class ScheduleLoopedBFS(PipelineScheduleMulti):
    """Breadth-first over the local stages (reference ``PipelineSchedule.py:517-569``)."""

    def _rank_programs(self):
        return [order.looped_bfs_rank_program(self._local_stages(r), self._n_microbatches, self._has_backward)
                for r in range(self.pp_group_size)]


class ScheduleInterleaved1F1B(PipelineScheduleMulti):
    """Interleaved 1F1B (reference ``PipelineSchedule.py:572-778``)."""

    def __init__(self, stages: List[PipelineStageBase], n_microbatches: int,
                 loss_fn: Optional[Callable] = None,
                 output_merge_spec: Optional[Union[Dict[str, Any], Tuple[Any]]] = None):
        if len(stages) > 0:
            group_size = stages[0].group_size
            if n_microbatches % group_size != 0:
                raise ValueError(
                    "Interleaved 1F1B requires the number of microbatches to be a "
                    f"multiple of the number of pipeline ranks ({group_size}), "
                    f"but got {n_microbatches}.")
        super().__init__(stages=stages, n_microbatches=n_microbatches, loss_fn=loss_fn,
                         output_merge_spec=output_merge_spec)
        self.n_local_stages = len(self._local_stages(0))
        self.rank = 0

    def _rank_programs(self):
        return [order.interleaved_rank_program(r, self.pp_group_size, self._local_stages(r),
                                               self._n_microbatches, self._has_backward)
                for r in range(self.pp_group_size)]
