"""Loss functions the last stage can run as HIP kernels.

The reference calls the user's ``loss_fn(output, target)`` right after the last stage's forward
(``pippy/PipelineSchedule.py:39-45,154-155``) and lets autograd differentiate it later.  A loss
object from this module is recognised by the stage runtime and replaced by one fused kernel that
returns the loss and leaves its gradient in the stage's output-gradient slot.  Any other callable
still works: it runs under autograd on the stage output and its gradient is copied into the slot.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


class NativeLoss:
    """Marker base class."""


class CrossEntropyLoss(NativeLoss):
    """Mean cross entropy over the non-ignored positions of one microbatch.  ``output`` is
    ``[..., vocab]`` logits and ``target`` the matching ``[...]`` int64 class ids (already shifted
    for next-token prediction)."""

    def __init__(self, ignore_index: int = -100):
        self.ignore_index = ignore_index

    def __call__(self, output: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
        # torch statement (used when the loss runs outside a native stage)
        return F.cross_entropy(output.reshape(-1, output.shape[-1]).float(), target.reshape(-1),
                               ignore_index=self.ignore_index)


def as_native_loss(loss_fn):
    """Maps a loss callable to its native form, or None.  ``torch.nn.CrossEntropyLoss`` with
    default options on 2-d logits is the same function as ``CrossEntropyLoss`` above."""
    if isinstance(loss_fn, NativeLoss):
        return loss_fn
    if isinstance(loss_fn, torch.nn.CrossEntropyLoss):
        if (loss_fn.reduction == "mean" and loss_fn.weight is None
                and getattr(loss_fn, "label_smoothing", 0.0) == 0.0):
            native = CrossEntropyLoss(ignore_index=loss_fn.ignore_index)
            native._requires_2d = True  # torch's class dimension is dim 1, not the last one
            return native
    return None
