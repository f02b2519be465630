"""Execution order of the reference's schedules, by simulating its processes.

Each pipeline rank of the reference is an OS process running the loop of its schedule
(pippy/PipelineSchedule.py:280-355 GPipe, :359-449 1F1B, :518-569 LoopedBFS, :599-778 interleaved
1F1B) and blocking in ``work.wait()`` on receives until the neighbour has sent.  This module
re-states those loops as Python generators that yield the actions in program order and a tiny
round-robin scheduler that lets a rank proceed only when the data its next action receives has
been produced.  The result is one legal global order and, per rank, the exact program.

Pinned by tests/test_oracle.py: the 4-stage x 8-microbatch phase table quoted in the reference
(pippy/PipelineSchedule.py:373-377), the single-rank interleaved order for 2 local stages
(warm-up 1, then forward/backward pairs, cool-down 1), and the invariants every pipeline order
must satisfy (each (stage, microbatch) forward and backward exactly once, data dependencies
respected, per-stage microbatch order ascending).
"""
from collections import defaultdict
from typing import Dict, Iterator, List, Sequence, Tuple

Action = Tuple[str, int, int]  # ("F" | "B", stage, microbatch)


def gpipe_rank(stage: int, M: int, backward: bool = True) -> Iterator[Action]:
    for i in range(M):                       # pippy/PipelineSchedule.py:295-312
        yield ("F", stage, i)
    if backward:
        for i in range(M):                   # :327-348
            yield ("B", stage, i)


def one_f_one_b_counts(stage: int, S: int, M: int) -> Tuple[int, int, int]:
    warmup = min(M, 2 * (S - stage - 1))     # :379-382
    main = M - warmup                        # :384
    cooldown = 2 * M - (warmup + 2 * main)   # :386
    return warmup, main, cooldown


def one_f_one_b_rank(stage: int, S: int, M: int, backward: bool = True) -> Iterator[Action]:
    warmup, main, cooldown = one_f_one_b_counts(stage, S, M)
    bwd = 0
    for i in range(warmup + main + cooldown):  # :403
        if i < M:                              # :404-418
            yield ("F", stage, i)
        if i >= warmup and backward:           # :420-438
            yield ("B", stage, bwd)
            bwd += 1


def looped_bfs_rank(local_stages: Sequence[int], M: int, backward: bool = True) -> Iterator[Action]:
    for s in local_stages:                     # :538-550
        for i in range(M):
            yield ("F", s, i)
    if backward:
        for s in reversed(list(local_stages)):  # :552-567
            for i in range(M):
                yield ("B", s, i)


def interleaved_rank(rank: int, G: int, local_stages: Sequence[int], M: int) -> Iterator[Action]:
    n_local = len(local_stages)
    warmup = (n_local - 1) * G + 2 * ((G - 1) - rank)   # :624-625
    warmup = min(warmup, M * n_local)                   # :626-628
    fwd_bwd = n_local * M - warmup                      # :629-631
    cooldown = n_local * M - fwd_bwd                    # :632-634
    fwd_mb: Dict[int, int] = defaultdict(int)
    bwd_mb: Dict[int, int] = defaultdict(int)

    def fstage(step):                                   # :651-652
        return local_stages[(step // G) % n_local]

    def bstage(step):                                   # :654-660
        return local_stages[n_local - 1 - ((step - warmup) // G) % n_local]

    for step in range(warmup):                          # :672-704
        s = fstage(step)
        yield ("F", s, fwd_mb[s])
        fwd_mb[s] += 1
    for step in range(warmup, warmup + fwd_bwd):        # :707-742
        s = fstage(step)
        yield ("F", s, fwd_mb[s])
        fwd_mb[s] += 1
        s = bstage(step)
        yield ("B", s, bwd_mb[s])
        bwd_mb[s] += 1
    for step in range(warmup + fwd_bwd, warmup + fwd_bwd + cooldown):  # :745-771
        s = bstage(step)
        yield ("B", s, bwd_mb[s])
        bwd_mb[s] += 1


def simulate(rank_programs: Sequence[Iterator[Action]], S: int) -> List[Action]:
    """Runs the rank generators like concurrent processes: a forward of stage s > 0 blocks until
    stage s-1 has sent microbatch m's activation, a backward of stage s < S-1 blocks until stage
    s+1 has sent microbatch m's gradient.  Raises on dead-lock."""
    progs = [list(p) for p in rank_programs]
    pos = [0] * len(progs)
    done = set()
    order: List[Action] = []
    remaining = sum(len(p) for p in progs)
    while remaining:
        moved = False
        for r, prog in enumerate(progs):
            if pos[r] >= len(prog):
                continue
            kind, s, m = prog[pos[r]]
            if kind == "F":
                ok = s == 0 or ("F", s - 1, m) in done
            else:
                ok = ("F", s, m) in done and (s == S - 1 or ("B", s + 1, m) in done)
            if ok:
                done.add((kind, s, m))
                order.append((kind, s, m))
                pos[r] += 1
                remaining -= 1
                moved = True
        if not moved:
            raise RuntimeError("dead-lock in simulated schedule")
    return order
