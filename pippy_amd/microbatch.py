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


def _shard_dict_of_args(args_dict, args_chunk_spec, num_chunks):
    """Flatten, split or replicate, regroup per chunk (``microbatch.py:66-194``)."""
    args_sharded_replicated = {}
    arg_specs = []
    real_num_chunks = num_chunks
    first_tensor = True

    assert len(args_dict) == len(args_chunk_spec), (
        f"args_dict.keys() = {list(args_dict.keys())} "
        f"args_chunk_spec.keys() = {list(args_chunk_spec.keys())}")

    for arg_key, arg in args_dict.items():
        flat, spec = tree_flatten(arg)
        arg_specs.append(spec)
        chunk_spec = args_chunk_spec[arg_key]
        assert chunk_spec is not None
        chunk_spec_flat, _ = tree_flatten(chunk_spec)
        if len(flat) != len(chunk_spec_flat):
            raise ValueError(
                f"Argument value {arg} did not have the same number of "
                f"values as as chunk spec {chunk_spec}")

        sharded_arg_flat = []
        for v, chunk_v in zip(flat, chunk_spec_flat):
            if chunk_v is _Replicate or not isinstance(v, torch.Tensor):
                sharded_arg_flat.append([v] * real_num_chunks)
            elif isinstance(chunk_v, TensorChunkSpec):
                v_split_dim_size = v.size(chunk_v.split_dim)
                if v_split_dim_size < real_num_chunks:
                    if first_tensor:
                        logger.warning(
                            f"Tensor size on chunking dimension is {v_split_dim_size}, "
                            f"downsizing the number of chunks from {num_chunks} to {v_split_dim_size}.")
                        real_num_chunks = v_split_dim_size
                    else:
                        raise RuntimeError(
                            f"Arg {arg_key} on chunking dimension has a size of {v_split_dim_size}, "
                            f"smaller than the number of chunks {num_chunks}. "
                            "PiPPy cannot reduce the number of chunks because "
                            "other arguments have bigger chunk-dimension sizes. "
                            "Please adjust your num_chunks setting.")

                if _debug_mask_minibatches:
                    chunk_tensors = _masked_chunks(v, real_num_chunks, chunk_v.split_dim)
                else:
                    chunk_tensors = _split_tensor(v, real_num_chunks, chunk_v.split_dim)
                sharded_arg_flat.append(chunk_tensors)
                first_tensor = False
            else:
                raise TypeError(f"Unrecognized chunk spec: {chunk_v}")
        args_sharded_replicated[arg_key] = sharded_arg_flat

    args_split = []
    for chunk_idx in range(real_num_chunks):
        per_chunk_args = {}
        for (key, arg), arg_spec in zip(args_sharded_replicated.items(), arg_specs):
            per_chunk_args[key] = tree_unflatten([v_flat[chunk_idx] for v_flat in arg], arg_spec)
        args_split.append(per_chunk_args)
    return args_split


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
    """Split ``args`` / ``kwargs`` into ``chunks`` microbatches (``microbatch.py:197-300``)."""
    if kwargs is None:
        kwargs = {}
    if args_chunk_spec is None:
        args_chunk_spec = (TensorChunkSpec(DEFAULT_CHUNK_DIM),) * len(args)
    if kwargs_chunk_spec is None:
        kwargs_chunk_spec = dict.fromkeys(kwargs, TensorChunkSpec(DEFAULT_CHUNK_DIM))

    args_split_dict = _shard_dict_of_args(dict(enumerate(args)), dict(enumerate(args_chunk_spec)), chunks)
    real_num_chunks = len(args_split_dict)
    kwargs_split = _shard_dict_of_args(kwargs, kwargs_chunk_spec, real_num_chunks)

    if len(kwargs_split) < real_num_chunks:
        # kwargs forced a smaller chunk count (e.g. args held no tensor): re-shard args to match
        real_num_chunks = len(kwargs_split)
        args_split_dict = _shard_dict_of_args(
            dict(enumerate(args)), dict(enumerate(args_chunk_spec)), real_num_chunks)

    if len(args_split_dict) != len(kwargs_split):
        raise RuntimeError(
            "args and kwargs are split into different number of chunks: "
            f"{len(args_split_dict)}, {len(kwargs_split)}")

    args_split = [tuple(chunk_args[i] for i in range(len(chunk_args))) for chunk_args in args_split_dict]
    return args_split, kwargs_split


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
            segs.append((v.data_ptr(), out.data_ptr() + lo * inner, n_rows, row_bytes, src_stride,
                         dst_stride))
        lo += d
    _native.copy_rows(segs)
    del keep_alive
    return out


def merge_chunks(chunks: List[Any], chunk_spec):
    """Inverse of the split: merge per-microbatch values into one (``microbatch.py:303-432``)."""
    if chunk_spec is not None:
        spec_flattened, flatten_spec = tree_flatten(chunk_spec)
    else:
        # default: every output leaf is concatenated along dim 0 (``microbatch.py:348-354``)
        chunk0_flat, flatten_spec = tree_flatten(chunks[0])
        spec_flattened = [TensorChunkSpec(DEFAULT_CHUNK_DIM)] * len(chunk0_flat)

    chunks_flattened = []
    for chunk in chunks:
        chunk_flattened, _ = tree_flatten(chunk)
        if len(chunk_flattened) != len(spec_flattened):
            raise ValueError(f"Chunk {chunk} did not match chunk spec {chunk_spec}")
        chunks_flattened.append(chunk_flattened)

    args_flattened = []
    for arg_idx, arg in enumerate(spec_flattened):
        if isinstance(arg, TensorChunkSpec):
            partial_values = [c[arg_idx] for c in chunks_flattened]
            if _debug_mask_minibatches:
                # every chunk is full size; keep only its own slice (``microbatch.py:380-410``)
                overall_shape = partial_values[0].shape
                for val in partial_values[1:]:
                    assert val.shape == overall_shape
                sizes = chunk_sizes(overall_shape[arg.split_dim], len(partial_values))
                values_to_cat = []
                lo = 0
                for val, size in zip(partial_values, sizes):
                    idx = [slice(None)] * val.dim()
                    idx[arg.split_dim] = slice(lo, lo + size)
                    values_to_cat.append(val[tuple(idx)])
                    lo += size
            else:
                values_to_cat = partial_values
            args_flattened.append(cat_chunks(values_to_cat, arg.split_dim))
        elif isinstance(arg, _CustomReducer):
            reduced_val = arg.init_value
            for chunk in chunks_flattened:
                reduced_val = arg.reduce_fn(reduced_val, chunk[arg_idx])
            args_flattened.append(reduced_val)
        else:
            value = chunks_flattened[0][arg_idx]
            for chunk in chunks_flattened[1:]:
                assert chunk[arg_idx] == value
            args_flattened.append(value)

    return tree_unflatten(args_flattened, flatten_spec)
