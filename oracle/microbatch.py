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


def round_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns, round to nearest even (finite inputs)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def embedding_grad(ids: np.ndarray, dy_bf16_bits: np.ndarray, vocab: int, round_bf16: bool) -> np.ndarray:
    """Gradient of ``F.embedding`` w.r.t. its table for one microbatch (reached from
    pippy/_backward.py:67-69): row v is the sum of dy[t] over the tokens with ids[t] == v, formed in
    fp32 in ascending t; ``round_bf16`` rounds it to bf16, the dtype of the table.  Returned as fp32.
    ``np.add.at`` applies the additions one by one in index order."""
    dy = (dy_bf16_bits.astype(np.uint32) << 16).view(np.float32)
    g = np.zeros((vocab, dy.shape[1]), dtype=np.float32)
    np.add.at(g, ids.reshape(-1), dy)
    if round_bf16:
        g = (round_to_bf16_bits(g).astype(np.uint32) << 16).view(np.float32)
    return g
