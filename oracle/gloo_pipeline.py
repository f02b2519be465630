"""The reference's way of running a pipeline on host cores: one CPU process per stage over gloo.

Test and measurement infrastructure (the CPU baseline of ``bench.py``); nothing in the product
imports it.  Every process owns one stage of the same GPT-2-shaped decoder (built from seed 0, so all
ranks hold the same weights without exchanging them) and executes the program of its own rank of
``Schedule1F1B`` (pippy/PipelineSchedule.py:359-449: ``warmup = min(M, 2 (S - s - 1))`` forwards, then
forward / backward pairs, then the remaining backwards).  Hand-offs are what the reference posts as
``dist.P2POp`` pairs (pippy/_PipelineStage.py:210-341): a blocking receive of the activation before a
forward and of the output gradient before a backward, an asynchronous send after them; the backward
of a (stage, microbatch) is one ``torch.autograd.backward`` (pippy/_backward.py:67-69), so parameter
gradients accumulate in ``param.grad`` in the parameter dtype as they do in the reference.  The
process group is started as in the reference's tests (test/test_fwd.py:117-129: backend gloo on CPU).

Run as ``python -m oracle.gloo_pipeline --rank R --world S ...`` with MASTER_ADDR / MASTER_PORT set;
rank 0 prints one JSON line with the wall times of the timed steps (their median is the figure).
"""
import argparse
import json
import os
import sys
import time

import torch
import torch.distributed as dist
import torch.nn as nn
import torch.nn.functional as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle.schedules import one_f_one_b_rank  # noqa: E402


def build_stage(args, rank: int, dtype) -> nn.Module:
    from pippy_amd.configs import DecoderLM
    torch.manual_seed(0)
    model = DecoderLM(vocab=args.vocab, max_seq=args.seq, dim=args.dim, n_layers=args.layers,
                      n_heads=args.heads, ffn=args.ffn, dtype=dtype)
    per = args.layers // args.world
    mods = ([model.embed] if rank == 0 else []) + [model.h[i] for i in range(per * rank, per * (rank + 1))]
    if rank == args.world - 1:
        mods.append(model.head)
    return nn.Sequential(*mods)


def run_step(stage: nn.Module, rank: int, world: int, M: int, ids_mbs, target_mbs, act_shape, dtype):
    """One 1F1B step of this rank.  Returns the losses (last rank) of the step."""
    first, last = rank == 0, rank == world - 1
    inputs, outputs, losses, sends = {}, {}, {}, []
    for kind, _s, m in one_f_one_b_rank(rank, world, M):
        if kind == "F":
            if first:
                x = ids_mbs[m]
            else:
                x = torch.empty(act_shape, dtype=dtype)
                dist.recv(x, src=rank - 1)
                x.requires_grad_(True)
            out = stage(x)
            inputs[m], outputs[m] = x, out
            if last:
                losses[m] = F.cross_entropy(out.reshape(-1, out.shape[-1]).float(), target_mbs[m].reshape(-1))
            else:
                sends.append(dist.isend(out.detach(), dst=rank + 1))
        else:
            if last:
                torch.autograd.backward(losses[m])
            else:
                g = torch.empty(act_shape, dtype=dtype)
                dist.recv(g, src=rank + 1)
                torch.autograd.backward(outputs[m], grad_tensors=g)
            if not first:
                sends.append(dist.isend(inputs[m].grad, dst=rank - 1))
            del inputs[m], outputs[m]
    for w in sends:
        w.wait()
    return [losses[m].detach() for m in sorted(losses)]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--rank", type=int, required=True)
    ap.add_argument("--world", type=int, required=True)
    ap.add_argument("--threads", type=int, default=1)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--vocab", type=int, default=50257)
    ap.add_argument("--seq", type=int, default=1024)
    ap.add_argument("--dim", type=int, default=768)
    ap.add_argument("--layers", type=int, default=12)
    ap.add_argument("--heads", type=int, default=12)
    ap.add_argument("--ffn", type=int, default=3072)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--microbatches", type=int, default=8)
    ap.add_argument("--warmup-microbatches", type=int, default=1)
    ap.add_argument("--warmup-steps", type=int, default=1, help="untimed full steps before the timed ones")
    ap.add_argument("--timed-steps", type=int, default=3, help="timed full steps; the median is reported")
    ap.add_argument("--budget-seconds", type=float, default=0.0,
                    help="if > 0 and the warm-up microbatch says that the warm-up and timed steps would "
                         "overrun it: one timed step without a warm-up step, over the first M' = M, M/2, "
                         "M/4 ... microbatches, the largest count that stays within the budget")
    args = ap.parse_args()

    torch.set_num_threads(max(1, args.threads))
    dist.init_process_group("gloo", rank=args.rank, world_size=args.world)
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    stage = build_stage(args, args.rank, dtype)
    mb = args.batch // args.microbatches
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, args.vocab, (args.batch, args.seq), generator=g)
    target = torch.randint(0, args.vocab, (args.batch, args.seq), generator=g)
    ids_mbs = list(torch.tensor_split(ids, args.microbatches))
    target_mbs = list(torch.tensor_split(target, args.microbatches))
    act_shape = (mb, args.seq, args.dim)

    # warm-up: a short step (thread pools, allocator, first-touch of the weights), gradients dropped
    w = max(1, args.warmup_microbatches)
    dist.barrier()
    t0 = time.perf_counter()
    run_step(stage, args.rank, args.world, w, ids_mbs[:w], target_mbs[:w], act_shape, dtype)
    dist.barrier()
    warm_s = time.perf_counter() - t0
    for p in stage.parameters():
        p.grad = None

    # how much is timed: by default whole steps (warm-up steps, then timed steps); when the warm-up
    # microbatch says that this would overrun the budget, one step, or the first half (quarter ...) of
    # its microbatches (a pipelined step of M microbatches over S stages lasts about (M + S - 1) / S
    # single-microbatch passes through the whole pipeline, which is what the warm-up timed)
    n_timed, warm_steps, timed_steps = args.microbatches, max(0, args.warmup_steps), max(1, args.timed_steps)
    if args.budget_seconds > 0:
        per_pass = warm_s / w
        est = lambda n: per_pass * (n + args.world - 1) / args.world  # noqa: E731
        if est(n_timed) * (warm_steps + timed_steps) > args.budget_seconds:
            warm_steps, timed_steps = 0, 1
            while n_timed > 1 and est(n_timed) > args.budget_seconds:
                n_timed //= 2
    decided = torch.tensor([n_timed, warm_steps, timed_steps])
    dist.broadcast(decided, src=0)
    n_timed, warm_steps, timed_steps = (int(v) for v in decided)

    def zero_grads():
        for p in stage.parameters():
            p.grad = None

    step_times, losses = [], None
    for it in range(warm_steps + timed_steps):
        zero_grads()
        dist.barrier()
        t0 = time.perf_counter()
        got = run_step(stage, args.rank, args.world, n_timed, ids_mbs[:n_timed], target_mbs[:n_timed], act_shape,
                       dtype)
        dist.barrier()
        if it >= warm_steps:
            step_times.append(time.perf_counter() - t0)
        if losses is None:
            losses = got  # of the first step run after the gradients were cleared: what a test compares
    step_s = sorted(step_times)[len(step_times) // 2]
    if args.rank == args.world - 1 and args.world > 1:
        # the last rank holds the losses; rank 0 reports, so send them over
        dist.send(torch.stack(losses).float(), dst=0)
    if args.rank == 0:
        got = torch.empty(n_timed)
        if args.world > 1:
            dist.recv(got, src=args.world - 1)
        else:
            got = torch.stack(losses).float()
        print(json.dumps({"step_s": step_s, "step_times_s": step_times, "warmup_steps": warm_steps,
                          "warmup_s": warm_s, "warmup_microbatches": w,
                          "losses": [float(v) for v in got],
                          "tokens": n_timed * mb * args.seq, "microbatches_timed": n_timed,
                          "microbatches": args.microbatches, "threads_per_rank": torch.get_num_threads(),
                          "world": args.world, "dtype": args.dtype,
                          "loss_microbatch0": float(got[0])}), flush=True)
    dist.destroy_process_group()


if __name__ == "__main__":
    main()
