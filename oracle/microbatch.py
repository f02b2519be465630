"""numpy statement of the reference's microbatch split and merge.

Split: pippy/microbatch.py:139-141 calls ``torch.tensor_split(v, n, dim)``, whose documented rule
is: the first ``size % n`` chunks have ``size // n + 1`` elements along ``dim``, the rest
``size // n``.  Merge: pippy/microbatch.py:415 calls ``torch.cat(values, dim)``.  Both only move
elements, so any dtype can be checked bit for bit on its raw bytes.

Pinned by tests/test_oracle.py against torch.tensor_split / torch.cat themselves, the shapes the
reference's own test holds (test/test_microbatch.py:17-34) and the round trip
merge(split(x)) == x (test/test_microbatch.py:37-51).
"""
from typing import List, Sequence

import numpy as np


def chunk_bounds(size: int, n: int) -> List[range]:
    base, extra = divmod(size, n)
    out, lo = [], 0
    for i in range(n):
        d = base + (1 if i < extra else 0)
        out.append(range(lo, lo + d))
        lo += d
    return out


def split(x: np.ndarray, n: int, dim: int = 0) -> List[np.ndarray]:
    idx = [slice(None)] * x.ndim
    chunks = []
    for r in chunk_bounds(x.shape[dim], n):
        idx[dim] = slice(r.start, r.stop)
        chunks.append(np.ascontiguousarray(x[tuple(idx)]))
    return chunks


def merge(chunks: Sequence[np.ndarray], dim: int = 0) -> np.ndarray:
    first = chunks[0]
    shape = list(first.shape)
    shape[dim] = sum(c.shape[dim] for c in chunks)
    out = np.empty(shape, dtype=first.dtype)
    idx = [slice(None)] * first.ndim
    lo = 0
    for c in chunks:
        idx[dim] = slice(lo, lo + c.shape[dim])
        out[tuple(idx)] = c
        lo += c.shape[dim]
    return out


def accumulate_fp32(grads_bf16_bits: Sequence[np.ndarray]) -> np.ndarray:
    """Sequential fp32 accumulation of bf16 gradients given as uint16 bit patterns, in list order:
    acc = float(g0); acc = acc + float(g_m).  bf16 -> fp32 is exact (bits << 16).  This is the
    autograd accumulation of pippy/_backward.py:67-69 with an fp32 accumulator."""
    def widen(bits):
        return (bits.astype(np.uint32) << 16).view(np.float32)
    acc = widen(grads_bf16_bits[0]).copy()
    for g in grads_bf16_bits[1:]:
        acc = (acc + widen(g)).astype(np.float32)
    return acc
