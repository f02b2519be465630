"""Microbatch split and merge (mirrors ``pippy/microbatch.py`` of the reference).

Same names, argument meaning and error behaviour as the reference; the data movement runs on the
GPU through the row-copy kernels:

* split (reference ``microbatch.py:139-141``, ``torch.tensor_split``): a chunk that is already a
  contiguous slab of its source (any split of a contiguous tensor along its first non-unit
  dimension) stays a zero-copy view, exactly as in the reference; every other chunk of a device
  tensor is materialised contiguous by ``pp_split_copy`` so that stage kernels can consume it.
* merge (reference ``microbatch.py:415``, ``torch.cat``): one ``pp_copy_rows`` launch gathers all
  chunks into a fresh tensor.

Host tensors are only ever viewed (a split of a CPU tensor moves no bytes); merging CPU tensors
raises, because this package has no CPU data path.
"""
from __future__ import annotations

import logging
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch
from torch.utils._pytree import tree_flatten, tree_unflatten

from . import _native

logger = logging.getLogger(__name__)

# When set, every microbatch is presented as a full-size tensor that is zero outside its own slice
# (reference ``microbatch.py:16,143-163``): GEMM shapes then equal the un-pipelined run.
_debug_mask_minibatches = False


class _CustomReducer:
    """Fold-left reduction of one output leaf over the microbatches (``microbatch.py:19-33``)."""

    def __init__(self, init_value, reduce_fn):
        self.init_value = init_value
        self.reduce_fn = reduce_fn


class _LossReducer(_CustomReducer):
    pass


sum_reducer = _LossReducer(torch.tensor(0.0), lambda a, b: a + b)

DEFAULT_CHUNK_DIM = 0


class TensorChunkSpec:
    """Says along which dimension a tensor argument is split (``microbatch.py:48-58``)."""

    def __init__(self, split_dim):
        self.split_dim = split_dim

    split_dim: int

    def __repr__(self):
        return f"{self.__class__.__module__}.{self.__class__.__name__}({self.split_dim})"

    def __str__(self):
        return f"TensorChunkSpec({self.split_dim})"


class _Replicate:
    """Marks an argument that every microbatch receives unchanged (``microbatch.py:62-63``)."""


# ---- pure host logic (no device work) -----------------------------------------------------------
def chunk_sizes(dim_size: int, n_chunks: int) -> List[int]:
    """Sizes ``torch.tensor_split(x, n)`` gives along a dimension of ``dim_size``: the first
    ``dim_size % n`` chunks get ``ceil(dim_size / n)``, the rest ``floor``."""
    if n_chunks <= 0:
        raise ValueError(f"number of chunks must be positive, got {n_chunks}")
    base, extra = divmod(dim_size, n_chunks)
    return [base + (1 if i < extra else 0) for i in range(n_chunks)]


def _is_slab(t: torch.Tensor, dim: int) -> bool:
    """True if slicing ``t`` along ``dim`` yields contiguous chunks (all leading dims are 1)."""
    if not t.is_contiguous():
        return False
    return all(s == 1 for s in t.shape[:dim])


def _split_tensor(v: torch.Tensor, n: int, dim: int) -> Sequence[torch.Tensor]:
    views = torch.tensor_split(v, n, dim)
    if not v.is_cuda:
        return views  # host tensors: views only, nothing to compute
    dim = dim % max(v.dim(), 1)
    if _is_slab(v, dim) or v.numel() == 0:
        return views
    src = v
    if not v.is_contiguous():
        src = torch.empty(v.shape, dtype=v.dtype, device=v.device)
        _native.strided_copy_nd(src, v)
    outs = [torch.empty(c.shape, dtype=v.dtype, device=v.device) for c in views]
    _native.split_copy(src, outs, dim)
    return tuple(outs)


class _Leaf:
    """One flattened value of an argument and what the spec says to do with it: ``dim`` is the
    dimension a tensor is cut along, or None for a value that every microbatch receives as it is."""

    __slots__ = ("value", "dim")

    def __init__(self, value, dim):
        self.value = value
        self.dim = dim


def _plan_leaves(arg, chunk_spec) -> Tuple[List[_Leaf], Any]:
    """Flattens one argument next to its spec (reference ``microbatch.py:97-113,169``)."""
    values, tree = tree_flatten(arg)
    rules, _ = tree_flatten(chunk_spec)
    if len(values) != len(rules):
        raise ValueError(
            f"Argument value {arg} did not have the same number of "
            f"values as as chunk spec {chunk_spec}")
    leaves = []
    for value, rule in zip(values, rules):
        if rule is _Replicate or not isinstance(value, torch.Tensor):
            leaves.append(_Leaf(value, None))
        elif isinstance(rule, TensorChunkSpec):
            leaves.append(_Leaf(value, rule.split_dim))
        else:
            raise TypeError(f"Unrecognized chunk spec: {rule}")
    return leaves, tree


def _settle_chunk_count(plans, num_chunks: int) -> int:
    """How many chunks the arguments really give (reference ``microbatch.py:118-137``): the first
    tensor that is cut may be shorter than ``num_chunks`` along its dimension, which lowers the count
    with a warning; a later tensor that is shorter than the count is an error."""
    count = num_chunks
    seen_tensor = False
    for key, leaves, _tree in plans:
        for leaf in leaves:
            if leaf.dim is None:
                continue
            extent = leaf.value.size(leaf.dim)
            if extent < count:
                if seen_tensor:
                    raise RuntimeError(
                        f"Arg {key} on chunking dimension has a size of {extent}, "
                        f"smaller than the number of chunks {num_chunks}. "
                        "PiPPy cannot reduce the number of chunks because "
                        "other arguments have bigger chunk-dimension sizes. "
                        "Please adjust your num_chunks setting.")
                logger.warning(
                    f"Tensor size on chunking dimension is {extent}, "
                    f"downsizing the number of chunks from {num_chunks} to {extent}.")
                count = extent
            seen_tensor = True
    return count


def _shard_dict_of_args(args_dict, args_chunk_spec, num_chunks):
    """Cuts a dict of arguments into a list of per-microbatch dicts (reference
    ``microbatch.py:66-194``).  Three passes: pair every flattened value with its rule, settle the
    chunk count, then cut each tensor once and deal the pieces out."""
    assert len(args_dict) == len(args_chunk_spec), (
        f"args_dict.keys() = {list(args_dict.keys())} "
        f"args_chunk_spec.keys() = {list(args_chunk_spec.keys())}")
    plans = []
    for key, arg in args_dict.items():
        rule = args_chunk_spec[key]
        assert rule is not None
        leaves, tree = _plan_leaves(arg, rule)
        plans.append((key, leaves, tree))
    count = _settle_chunk_count(plans, num_chunks)
    cut = _masked_chunks if _debug_mask_minibatches else _split_tensor

    microbatches: List[Dict[Any, Any]] = [{} for _ in range(count)]
    for key, leaves, tree in plans:
        pieces = [cut(leaf.value, count, leaf.dim) if leaf.dim is not None else None for leaf in leaves]
        for m, mb_args in enumerate(microbatches):
            flat = [leaf.value if piece is None else piece[m] for leaf, piece in zip(leaves, pieces)]
            mb_args[key] = tree_unflatten(flat, tree)
    return microbatches


def _masked_chunks(v: torch.Tensor, n: int, dim: int) -> List[torch.Tensor]:
    """Full-size zero tensors with one chunk written in place (``microbatch.py:143-163``)."""
    out = []
    lo = 0
    for size in chunk_sizes(v.size(dim), n):
        full = torch.zeros_like(v)
        idx = [slice(None)] * v.dim()
        idx[dim] = slice(lo, lo + size)
        if v.is_cuda and size > 0:
            src = v[tuple(idx)]
            tmp = torch.empty(src.shape, dtype=v.dtype, device=v.device)
            _native.strided_copy_nd(tmp, src)
            _copy_into_slice(full, tmp, dim, lo)
        else:
            full[tuple(idx)] = v[tuple(idx)]
        out.append(full)
        lo += size
    return out


def _rows(shape: Sequence[int], dim: int, elem: int) -> Tuple[int, int]:
    outer = 1
    for s in shape[:dim]:
        outer *= s
    inner = elem
    for s in shape[dim + 1:]:
        inner *= s
    return outer, inner


def _copy_into_slice(dst: torch.Tensor, chunk: torch.Tensor, dim: int, lo: int) -> None:
    """dst[..., lo:lo+chunk.size(dim), ...] = chunk, both contiguous, via the row-copy kernel."""
    outer, inner = _rows(dst.shape, dim, dst.element_size())
    d = chunk.size(dim)
    _native.copy_rows([(chunk.data_ptr(), dst.data_ptr() + lo * inner, outer, d * inner, d * inner,
                        dst.size(dim) * inner)])


def split_args_kwargs_into_chunks(
    args: Tuple[Any, ...],
    kwargs: Optional[Dict[str, Any]],
    chunks: int,
    args_chunk_spec: Optional[Tuple[TensorChunkSpec, ...]] = None,
    kwargs_chunk_spec: Optional[Dict[str, TensorChunkSpec]] = None,
) -> Tuple[List[Tuple], List[Dict]]:
    """Split ``args`` / ``kwargs`` into ``chunks`` microbatches (reference ``microbatch.py:197-300``).
    Without a spec every tensor is cut along dimension 0.  Positional and keyword arguments must end
    up with the same number of chunks; when the keyword arguments settle on fewer, the positional
    ones are cut again to that number."""
    kwargs = {} if kwargs is None else kwargs
    by_position = dict(enumerate(args))
    default = TensorChunkSpec(DEFAULT_CHUNK_DIM)
    position_rules = dict(enumerate(args_chunk_spec if args_chunk_spec is not None else (default,) * len(args)))
    keyword_rules = kwargs_chunk_spec if kwargs_chunk_spec is not None else dict.fromkeys(kwargs, default)

    positional = _shard_dict_of_args(by_position, position_rules, chunks)
    keyword = _shard_dict_of_args(kwargs, keyword_rules, len(positional))
    if len(keyword) < len(positional):
        positional = _shard_dict_of_args(by_position, position_rules, len(keyword))
    if len(positional) != len(keyword):
        raise RuntimeError(
            "args and kwargs are split into different number of chunks: "
            f"{len(positional)}, {len(keyword)}")
    return [tuple(mb[i] for i in range(len(args))) for mb in positional], keyword


# ---- merge -------------------------------------------------------------------------------------
def _collapse(t: torch.Tensor, dims: Sequence[int]):
    """(count, stride) if the listed dims of ``t`` walk memory with one uniform stride, else None
    (size-1 dims are ignored; an empty walk is (1, 0))."""
    stride = None
    count = 1
    for d in reversed(list(dims)):
        if t.size(d) == 1:
            continue
        if stride is None:
            stride = t.stride(d)
        elif t.stride(d) != stride * count:
            return None
        count *= t.size(d)
    return (count, stride if stride is not None else 0)


def _row_view(t: torch.Tensor, dim: int):
    """Describes ``t`` as uniformly strided rows for a concatenation along ``dim``.  Returns
    (n_rows, row_bytes, row_stride_bytes, rows_per_outer) or None.  ``rows_per_outer`` is how many
    consecutive rows belong to one index of the dims before ``dim`` (the destination jumps after
    that many rows unless there is a single outer index)."""
    es = t.element_size()
    nd = t.dim()
    # k = first dim of the densely packed trailing block
    expect = 1
    k = nd
    for d in range(nd - 1, -1, -1):
        if t.size(d) != 1 and t.stride(d) != expect:
            break
        expect *= t.size(d)
        k = d
    outer = 1
    for s_ in t.shape[:dim]:
        outer *= s_
    if k <= dim:
        # whole [dim..] slabs are contiguous: one row per outer index
        row_elems = 1
        for s_ in t.shape[dim:]:
            row_elems *= s_
        col = _collapse(t, range(0, dim))
        if col is None:
            return None
        count, stride = col
        if count > 1 and stride < row_elems:
            return None
        return (outer, row_elems * es, (stride if count > 1 else row_elems) * es, 1)
    # the dense block is smaller than a slab: rows are the dense blocks; the destination is only
    # uniformly strided when a single outer index exists
    if outer != 1:
        return None
    row_elems = 1
    for s_ in t.shape[k:]:
        row_elems *= s_
    col = _collapse(t, range(0, k))
    if col is None:
        return None
    count, stride = col
    if count > 1 and stride < row_elems:
        return None
    return (count, row_elems * es, (stride if count > 1 else row_elems) * es, count)


def cat_chunks(values: Sequence[torch.Tensor], dim: int) -> torch.Tensor:
    """``torch.cat(values, dim)`` on the GPU with one row-copy launch per 64 chunks."""
    if not values:
        raise ValueError("expected a non-empty list of tensors to concatenate")
    first = values[0]
    for v in values:
        if not isinstance(v, torch.Tensor):
            raise TypeError(f"cannot concatenate a {type(v)}")
    if not first.is_cuda:
        raise RuntimeError(
            "merge_chunks: microbatch outputs are on the host; pippy_amd merges device tensors "
            "only (there is no CPU data path)")
    if first.dim() == 0:
        raise RuntimeError("zero-dimensional tensor cannot be concatenated")
    dim = dim % first.dim()
    total = 0
    for v in values:
        if v.dim() != first.dim() or v.dtype != first.dtype or v.device != first.device:
            raise RuntimeError("merge_chunks: chunks disagree in rank, dtype or device")
        for d in range(first.dim()):
            if d != dim and v.size(d) != first.size(d):
                raise RuntimeError(
                    f"Sizes of tensors must match except in dimension {dim}. "
                    f"Expected size {first.size(d)} but got size {v.size(d)} in dimension {d}")
        total += v.size(dim)
    shape = list(first.shape)
    shape[dim] = total
    out = torch.empty(shape, dtype=first.dtype, device=first.device)
    if out.numel() == 0:
        return out
    outer, inner = _rows(shape, dim, first.element_size())
    segs = []
    keep_alive = []  # staging tensors must outlive the enqueue of the copy that reads them
    lo = 0
    for v in values:
        d = v.size(dim)
        if v.numel():
            segs.append(_segment(v, out.data_ptr() + lo * inner, dim, total, outer, inner, keep_alive))
        lo += d
    _native.copy_rows(segs)
    del keep_alive
    return out


def _segment(v: torch.Tensor, dst_ptr: int, dim: int, total: int, outer: int, inner: int, keep_alive: list):
    """The row-copy segment that writes ``v`` into its place along ``dim`` of a contiguous tensor whose
    size along ``dim`` is ``total`` (``outer`` / ``inner`` as ``_rows`` gives them for that tensor)."""
    d = v.size(dim)
    rv = _row_view(v, dim)
    if rv is None:  # arbitrary strides: gather into a contiguous staging tensor first
        tmp = torch.empty(v.shape, dtype=v.dtype, device=v.device)
        _native.strided_copy_nd(tmp, v)
        keep_alive.append(tmp)
        v = tmp
        rv = (outer, d * inner, d * inner, 1)
    n_rows, row_bytes, src_stride, rows_per_outer = rv
    if rows_per_outer == 1:
        assert row_bytes == d * inner and n_rows == outer
        dst_stride = total * inner
    else:
        assert outer == 1 and n_rows * row_bytes == d * inner
        dst_stride = row_bytes
    return (v.data_ptr(), dst_ptr, n_rows, row_bytes, src_stride, dst_stride)


def copy_into_rows(out: torch.Tensor, lo: int, v: torch.Tensor) -> None:
    """``out[lo : lo + v.size(0)] = v`` for a contiguous device tensor ``out`` and a chunk ``v`` of any
    strides, on the current stream: one microbatch's share of ``cat_chunks(values, 0)``."""
    assert out.is_contiguous() and out.is_cuda and v.shape[1:] == out.shape[1:] and v.dtype == out.dtype
    if not v.numel():
        return
    outer, inner = _rows(list(out.shape), 0, out.element_size())
    keep_alive = []
    _native.copy_rows([_segment(v, out.data_ptr() + lo * inner, 0, out.size(0), outer, inner, keep_alive)])
    del keep_alive


def _own_slices(values: Sequence[torch.Tensor], dim: int) -> List[torch.Tensor]:
    """Debug-mask mode: every microbatch value has the full batch shape and only the slice that the
    split gave its microbatch is meaningful (reference ``microbatch.py:380-410``)."""
    shape = values[0].shape
    for v in values[1:]:
        assert v.shape == shape
    out, lo = [], 0
    for v, size in zip(values, chunk_sizes(shape[dim], len(values))):
        out.append(v.narrow(dim, lo, size))
        lo += size
    return out


def _merge_leaf(rule, column: Sequence[Any]):
    """One output leaf from its per-microbatch values (reference ``microbatch.py:374-429``)."""
    if isinstance(rule, TensorChunkSpec):
        values = _own_slices(column, rule.split_dim) if _debug_mask_minibatches else column
        return cat_chunks(values, rule.split_dim)
    if isinstance(rule, _CustomReducer):
        total = rule.init_value
        for value in column:
            total = rule.reduce_fn(total, value)
        return total
    # anything else was replicated: every microbatch must hold the same value
    for value in column[1:]:
        assert value == column[0]
    return column[0]


def merge_chunks(chunks: List[Any], chunk_spec):
    """Inverse of the split: per-microbatch values back into one (reference
    ``microbatch.py:303-432``).  ``chunk_spec`` mirrors the structure of one chunk; None concatenates
    every leaf along dimension 0."""
    if chunk_spec is None:
        leaves0, tree = tree_flatten(chunks[0])
        rules = [TensorChunkSpec(DEFAULT_CHUNK_DIM)] * len(leaves0)
    else:
        rules, tree = tree_flatten(chunk_spec)
    columns: List[List[Any]] = [[] for _ in rules]
    for chunk in chunks:
        leaves, _ = tree_flatten(chunk)
        if len(leaves) != len(rules):
            raise ValueError(f"Chunk {chunk} did not match chunk spec {chunk_spec}")
        for column, leaf in zip(columns, leaves):
            column.append(leaf)
    return tree_unflatten([_merge_leaf(rule, column) for rule, column in zip(rules, columns)], tree)
