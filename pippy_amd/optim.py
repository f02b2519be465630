"""Optimizer step on the fp32 gradient accumulators of natively lowered stages.

The reference's users build a ``torch.optim`` optimizer over ``stage.submod.parameters()`` and call
``optimizer.step()`` after ``schedule.step()`` (reference ``test/test_optim.py:83-99``).  A lowered
stage keeps its parameters, and the fp32 sums of their microbatch gradients, in flat arenas, so the
same update is one HIP launch per stage: ``FusedSGD`` and ``FusedAdamW`` follow ``torch.optim.SGD``
and ``torch.optim.AdamW`` (same hyper-parameters, same arithmetic operation by operation), read the
fp32 accumulators instead of ``param.grad`` and keep their state in fp32.

    opt = FusedAdamW(stages, lr=3e-4, weight_decay=0.1)
    for batch, target in data:
        opt.zero_grad()
        schedule.step(batch, target=target, losses=losses)
        opt.step()
"""
from __future__ import annotations

import math
from typing import Iterable, List, Optional

import torch

from . import _native as N


class _FusedOptimizer:
    def __init__(self, stages, master_weights: bool):
        stages = list(stages) if isinstance(stages, (list, tuple)) else [stages]
        if not stages:
            raise ValueError("optimizer got no stages")
        self._stages = stages
        self._arenas = []
        for st in stages:
            if not getattr(st, "is_native", False):
                raise RuntimeError(
                    f"stage {getattr(st, 'stage_index', '?')} is not lowered to HIP launch lists; use a "
                    "torch.optim optimizer on stage.submod.parameters() after stage.materialize_grads()")
            self._arenas.append(st.param_arena())
        self._master: List[Optional[torch.Tensor]] = []
        for a in self._arenas:
            if master_weights and a.dtype == torch.bfloat16:
                self._master.append(a.params.to(torch.float32))
            else:
                self._master.append(None)
        self._steps = 0

    def zero_grad(self, set_to_none: bool = True):
        """Clears the accumulated gradients of every stage (the next weight-gradient pass starts
        the sums afresh)."""
        for st in self._stages:
            st.zero_grad()

    def _after_update(self):
        for a in self._arenas:
            a.mark_updated()

    def _has_grads(self, k: int) -> bool:
        """False for a stage whose gradients were cleared and not produced again: its accumulators
        hold the sums of an earlier step, and torch.optim skips parameters without a gradient."""
        prog = self._stages[k]._program
        return prog is not None and prog.acc_initialized

    @property
    def master_weights(self) -> List[Optional[torch.Tensor]]:
        return self._master

    # -- checkpointing: state per parameter, keyed by the name it has in its stage module (which is
    # the name in the un-split model), so that a state dict survives a different split
    def _flat_state(self) -> dict:
        """name -> list of flat fp32 state tensors, one per stage arena (None where unused)."""
        return {"master": self._master}

    def state_dict(self) -> dict:
        state = {}
        flats = self._flat_state()
        for st, arena, k in zip(self._stages, self._arenas, range(len(self._arenas))):
            for name, p in st.submod.named_parameters():
                entry = {}
                for key, per_stage in flats.items():
                    if per_stage[k] is not None:
                        entry[key] = arena._slice(per_stage[k], p, False).detach().cpu().clone()
                state[name] = entry
        return {"step": self._steps, "state": state}

    def load_state_dict(self, sd: dict) -> None:
        flats = self._flat_state()
        for st, arena, k in zip(self._stages, self._arenas, range(len(self._arenas))):
            for name, p in st.submod.named_parameters():
                if name not in sd["state"]:
                    raise KeyError(f"optimizer state of {name} is missing")
                for key, per_stage in flats.items():
                    if per_stage[k] is not None:
                        arena._slice(per_stage[k], p, False).copy_(sd["state"][name][key])
        self._steps = int(sd["step"])


class FusedSGD(_FusedOptimizer):
    """``torch.optim.SGD`` over the arenas of lowered stages."""

    def __init__(self, stages, lr: float, momentum: float = 0.0, dampening: float = 0.0,
                 weight_decay: float = 0.0, nesterov: bool = False, *, maximize: bool = False,
                 master_weights: bool = False):
        if lr < 0.0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if momentum < 0.0:
            raise ValueError(f"Invalid momentum value: {momentum}")
        if weight_decay < 0.0:
            raise ValueError(f"Invalid weight_decay value: {weight_decay}")
        if nesterov and (momentum <= 0 or dampening != 0):
            raise ValueError("Nesterov momentum requires a momentum and zero dampening")
        super().__init__(stages, master_weights)
        self.lr, self.momentum, self.dampening = lr, momentum, dampening
        self.weight_decay, self.nesterov, self.maximize = weight_decay, nesterov, maximize
        self._buf = [torch.zeros_like(a.acc) if momentum != 0 else None for a in self._arenas]

    def _flat_state(self):
        return {"momentum_buffer": self._buf, "master": self._master}

    @torch.no_grad()
    def step(self):
        for k, (a, buf, master) in enumerate(zip(self._arenas, self._buf, self._master)):
            if not self._has_grads(k):
                continue
            N.sgd_step(a.params, a.acc, buf, master=master, lr=self.lr, momentum=self.momentum,
                       dampening=self.dampening, weight_decay=self.weight_decay, nesterov=self.nesterov,
                       first_step=self._steps == 0, maximize=self.maximize)
        self._steps += 1
        self._after_update()


class FusedAdamW(_FusedOptimizer):
    """``torch.optim.AdamW`` (no amsgrad) over the arenas of lowered stages."""

    def __init__(self, stages, lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 1e-2, *, maximize: bool = False, master_weights: bool = False):
        if lr < 0.0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if eps < 0.0:
            raise ValueError(f"Invalid epsilon value: {eps}")
        if not 0.0 <= betas[0] < 1.0 or not 0.0 <= betas[1] < 1.0:
            raise ValueError(f"Invalid betas: {betas}")
        if weight_decay < 0.0:
            raise ValueError(f"Invalid weight_decay value: {weight_decay}")
        super().__init__(stages, master_weights)
        self.lr, self.betas, self.eps = lr, tuple(betas), eps
        self.weight_decay, self.maximize = weight_decay, maximize
        self._m = [torch.zeros_like(a.acc) for a in self._arenas]
        self._v = [torch.zeros_like(a.acc) for a in self._arenas]

    def _flat_state(self):
        return {"exp_avg": self._m, "exp_avg_sq": self._v, "master": self._master}

    @torch.no_grad()
    def step(self):
        self._steps += 1
        b1, b2 = self.betas
        bc1 = 1.0 - b1 ** self._steps
        bc2_sqrt = math.sqrt(1.0 - b2 ** self._steps)
        for k, (a, m, v, master) in enumerate(zip(self._arenas, self._m, self._v, self._master)):
            if not self._has_grads(k):
                continue
            N.adamw_step(a.params, a.acc, m, v, master=master, lr=self.lr, beta1=b1, beta2=b2, eps=self.eps,
                         weight_decay=self.weight_decay, bias_correction1=bc1, bias_correction2_sqrt=bc2_sqrt,
                         maximize=self.maximize)
        self._after_update()
