"""CPU statement of one ``schedule.step()`` of the reference, in fp32.

Control flow follows the reference: split the batch with ``torch.tensor_split``
(pippy/microbatch.py:139-141, pippy/PipelineSchedule.py:262-265), run every microbatch forward
through the stages in order (pippy/_PipelineStage.py:452-510), compute the loss of microbatch m
right after its last-stage forward (pippy/PipelineSchedule.py:39-45), run the backwards in
ascending microbatch order (pippy/PipelineSchedule.py:327-348, 401-438) with one
``torch.autograd.backward`` per (stage, microbatch) that accumulates into ``param.grad``
(pippy/_backward.py:67-69), and concatenate the outputs (pippy/microbatch.py:415).  Stage
boundaries detach and re-attach activations exactly like the receive buffers of the reference
(pippy/_PipelineStage.py:246-249); they do not change any number, which the oracle's own test
checks against an un-staged run.

Pinned by tests/test_oracle.py: sum of per-microbatch losses == full-batch loss for a
sum-reduction loss (pippy test_grad.py:123-126), gradients == un-pipelined gradients
(test_grad.py:103-136), merged output == un-pipelined output (test_fwd.py:80-84).
"""
from typing import Callable, List, Optional, Sequence

import torch
import torch.nn as nn


def step(stages: Sequence[nn.Module], x: torch.Tensor, target: Optional[torch.Tensor],
         n_microbatches: int, loss_fn: Optional[Callable]):
    """Returns (merged_output, losses).  Parameter gradients accumulate into ``p.grad``."""
    xs = list(torch.tensor_split(x, n_microbatches))
    ts = list(torch.tensor_split(target, n_microbatches)) if target is not None else None
    S = len(stages)
    acts: List[List[torch.Tensor]] = []   # per microbatch: input of every stage
    outs: List[List[torch.Tensor]] = []   # per microbatch: output of every stage
    losses = []
    for m, xm in enumerate(xs):
        ins, os_ = [], []
        h = xm
        for s, stage in enumerate(stages):
            if s > 0:
                h = h.detach()
                if loss_fn is not None and h.is_floating_point():
                    h.requires_grad_(True)
            ins.append(h)
            h = stage(h)
            os_.append(h)
        acts.append(ins)
        outs.append(os_)
        if loss_fn is not None:
            losses.append(loss_fn(h, ts[m]))
    if loss_fn is not None:
        for m in range(len(xs)):
            grad = None
            for s in reversed(range(S)):
                if s == S - 1:
                    torch.autograd.backward(losses[m])
                else:
                    torch.autograd.backward(outs[m][s], grad_tensors=grad)
                g = acts[m][s].grad if acts[m][s].is_floating_point() else None
                grad = g
    merged = torch.cat([o[-1].detach() for o in outs], dim=0)
    return merged, [l.detach() for l in losses]
