"""Per-rank action programs of the pipeline schedules, and their merge into one device order.

The reference runs one OS process per pipeline rank; each executes the loop of its schedule and
ranks synchronise only through blocking receives.  Here every stage is a virtual stage on one
GPU, so the per-rank programs (same index formulas as the reference) are merged into a single
deterministic sequence that respects the data dependencies the receives used to enforce.

An action is ``(kind, stage_index, microbatch)`` with kind ``"F"`` (forward), ``"B"`` (full
backward), ``"I"`` (input-gradient pass) or ``"W"`` (weight-gradient pass).
"""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

Action = Tuple[str, int, int]


def gpipe_rank_program(stage: int, n_microbatches: int, has_backward: bool) -> List[Action]:
    """All forwards, then all backwards in ascending microbatch order
    (reference ``PipelineSchedule.py:295-348``)."""
    prog: List[Action] = [("F", stage, m) for m in range(n_microbatches)]
    if has_backward:
        prog += [("B", stage, m) for m in range(n_microbatches)]
    return prog


def one_f_one_b_phases(stage: int, num_stages: int, n_microbatches: int) -> Tuple[int, int, int]:
    """(warm-up, steady 1F1B, cool-down) step counts (reference ``PipelineSchedule.py:379-387``).
    4 stages x 8 microbatches gives 6/2/6, 4/4/4, 2/6/2, 0/8/0."""
    warmup = min(n_microbatches, 2 * (num_stages - stage - 1))
    main = n_microbatches - warmup
    cooldown = 2 * n_microbatches - (warmup + 2 * main)
    return warmup, main, cooldown


def one_f_one_b_rank_program(stage: int, num_stages: int, n_microbatches: int,
                             has_backward: bool) -> List[Action]:
    """Reference ``PipelineSchedule.py:403-438``: step i runs forward i (while i < M) and, from
    step ``warmup`` on, the next backward."""
    warmup, main, cooldown = one_f_one_b_phases(stage, num_stages, n_microbatches)
    prog: List[Action] = []
    bwd = 0
    for i in range(warmup + main + cooldown):
        if i < n_microbatches:
            prog.append(("F", stage, i))
        if i >= warmup and has_backward:
            prog.append(("B", stage, bwd))
            bwd += 1
    return prog


def looped_bfs_rank_program(local_stages: Sequence[int], n_microbatches: int,
                            has_backward: bool) -> List[Action]:
    """Stage by stage all forwards, then in reverse stage order all backwards
    (reference ``PipelineSchedule.py:538-567``)."""
    prog: List[Action] = []
    for s in local_stages:
        prog += [("F", s, m) for m in range(n_microbatches)]
    if has_backward:
        for s in reversed(list(local_stages)):
            prog += [("B", s, m) for m in range(n_microbatches)]
    return prog


def interleaved_phases(rank: int, group_size: int, n_local: int,
                       n_microbatches: int) -> Tuple[int, int, int]:
    """(warm-up, 1F1B, cool-down) step counts (reference ``PipelineSchedule.py:623-634``)."""
    warmup = (n_local - 1) * group_size + 2 * ((group_size - 1) - rank)
    warmup = min(warmup, n_microbatches * n_local)
    fwd_bwd = n_local * n_microbatches - warmup
    cooldown = n_local * n_microbatches - fwd_bwd
    return warmup, fwd_bwd, cooldown


def interleaved_rank_program(rank: int, group_size: int, local_stages: Sequence[int],
                             n_microbatches: int, has_backward: bool = True) -> List[Action]:
    """Reference ``PipelineSchedule.py:651-771``: the forward stage of step t is
    ``(t // G) % n_local``; the backward stage is ``n_local - 1 - ((t - warmup) // G) % n_local``;
    every stage counts its own microbatches."""
    n_local = len(local_stages)
    warmup, fwd_bwd, cooldown = interleaved_phases(rank, group_size, n_local, n_microbatches)
    fwd_mb: Dict[int, int] = {s: 0 for s in local_stages}
    bwd_mb: Dict[int, int] = {s: 0 for s in local_stages}

    def fwd_stage(step):
        return local_stages[(step // group_size) % n_local]

    def bwd_stage(step):
        return local_stages[n_local - 1 - ((step - warmup) // group_size) % n_local]

    prog: List[Action] = []
    for step in range(warmup):
        s = fwd_stage(step)
        prog.append(("F", s, fwd_mb[s]))
        fwd_mb[s] += 1
    for step in range(warmup, warmup + fwd_bwd):
        s = fwd_stage(step)
        prog.append(("F", s, fwd_mb[s]))
        fwd_mb[s] += 1
        if has_backward:
            s = bwd_stage(step)
            prog.append(("B", s, bwd_mb[s]))
            bwd_mb[s] += 1
    if has_backward:
        for step in range(warmup + fwd_bwd, warmup + fwd_bwd + cooldown):
            s = bwd_stage(step)
            prog.append(("B", s, bwd_mb[s]))
            bwd_mb[s] += 1
    return prog


def zero_bubble_rank_program(stage: int, num_stages: int, n_microbatches: int) -> List[Action]:
    """Zero-bubble (ZB-H1 style) program with the backward split into an input-gradient pass I and
    a weight-gradient pass W.  Not in the reference, whose backward is one fused autograd call
    (``pippy/_backward.py:67-69``).  Warm-up as 1F1B's textbook form, then F/I pairs with each W
    deferred by ``stage`` slots so that it fills the bubble; W runs in ascending microbatch order,
    which keeps the fp32 accumulation order equal to the fused schedule's."""
    M = n_microbatches
    warmup = min(M, num_stages - stage - 1)
    prog: List[Action] = [("F", stage, m) for m in range(warmup)]
    f, i, w = warmup, 0, 0
    delay = stage  # number of I passes that may run ahead of W on this stage
    while i < M:
        if f < M:
            prog.append(("F", stage, f))
            f += 1
        prog.append(("I", stage, i))
        i += 1
        if i - w > delay:
            prog.append(("W", stage, w))
            w += 1
    while w < M:
        prog.append(("W", stage, w))
        w += 1
    return prog


def merge_rank_programs(programs: Sequence[Sequence[Action]], num_stages: int) -> List[Action]:
    """Interleaves per-rank programs into one order.  An action is ready when its inputs exist:
    F(s, m) after F(s-1, m); B/I(s, m) after F(s, m) and after B/I(s+1, m); W(s, m) after I(s, m).
    Ranks are scanned round-robin from rank 0 and each ready head is issued, which is
    deterministic and cannot dead-lock on programs that are valid multi-process schedules."""
    done = set()
    heads = [0] * len(programs)
    order: List[Action] = []
    total = sum(len(p) for p in programs)

    def ready(act: Action) -> bool:
        kind, s, m = act
        if kind == "F":
            return s == 0 or ("F", s - 1, m) in done
        if kind in ("B", "I"):
            if ("F", s, m) not in done:
                return False
            return s == num_stages - 1 or ("B", s + 1, m) in done or ("I", s + 1, m) in done
        if kind == "W":
            return ("I", s, m) in done
        raise ValueError(f"unknown action kind {kind}")

    while len(order) < total:
        progressed = False
        for r, prog in enumerate(programs):
            while heads[r] < len(prog) and ready(prog[heads[r]]):
                act = prog[heads[r]]
                order.append(act)
                done.add(act)
                heads[r] += 1
                progressed = True
                break  # one action per rank per sweep keeps ranks in lock step
        if not progressed:
            stuck = [prog[heads[r]] for r, prog in enumerate(programs) if heads[r] < len(prog)]
            raise RuntimeError(f"schedule dead-lock: no rank can proceed; waiting actions {stuck}")
    return order
