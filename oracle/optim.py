"""Optimizer updates restated on numpy fp32 arrays (TEST INFRASTRUCTURE ONLY).

The reference's users step ``torch.optim`` optimizers on stage parameters after ``schedule.step()``
(reference ``test/test_optim.py:83-99``).  These functions restate torch.optim's single-tensor SGD
and AdamW updates, one numpy fp32 operation per torch operation; ``tests/test_oracle.py`` pins them
against ``torch.optim.SGD`` / ``torch.optim.AdamW`` themselves on CPU fp32 tensors.
"""
from __future__ import annotations

import numpy as np

f32 = np.float32


def sgd_step(p, g, buf, *, lr, momentum=0.0, dampening=0.0, weight_decay=0.0, nesterov=False,
             first_step=False, maximize=False):
    """Returns (new_p, new_buf).  p, g, buf: fp32 arrays (buf may be None when momentum == 0)."""
    p = np.asarray(p, dtype=f32)
    d = np.asarray(g, dtype=f32)
    if maximize:
        d = -d
    if weight_decay != 0:
        d = d + f32(weight_decay) * p
    if momentum != 0:
        if first_step or buf is None:
            buf = d.copy()
        else:
            buf = f32(momentum) * np.asarray(buf, dtype=f32) + f32(1.0 - dampening) * d
        d = d + f32(momentum) * buf if nesterov else buf
    return p - f32(lr) * d, buf


def adamw_step(p, g, m, v, *, lr, beta1, beta2, eps, weight_decay, step, maximize=False):
    """Returns (new_p, new_m, new_v); ``step`` counts from 1."""
    p = np.asarray(p, dtype=f32)
    d = np.asarray(g, dtype=f32)
    if maximize:
        d = -d
    m = np.asarray(m, dtype=f32)
    v = np.asarray(v, dtype=f32)
    p = p * f32(1.0 - lr * weight_decay)
    m = m + f32(1.0 - beta1) * (d - m)
    v = f32(beta2) * v + f32(1.0 - beta2) * d * d
    bc1 = 1.0 - beta1 ** step
    bc2_sqrt = (1.0 - beta2 ** step) ** 0.5
    denom = np.sqrt(v) / f32(bc2_sqrt) + f32(eps)
    p = p - f32(lr / bc1) * (m / denom)
    return p, m, v


def round_bf16(x):
    """fp32 array -> nearest-even bf16, returned as fp32."""
    u = np.asarray(x, dtype=f32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(f32)
