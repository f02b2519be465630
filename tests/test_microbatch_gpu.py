"""The reference's split / merge API (``pippy/microbatch.py``) on device tensors: every result must
equal, bit for bit, what ``torch.tensor_split`` / ``torch.cat`` give for the same arguments
(``microbatch.py:139-141,415``), also where the chunks are not slabs of their source (split along an
inner dimension, non-contiguous inputs), in debug-mask mode (``microbatch.py:143-163,380-410``), with
replicated leaves and with a reducer."""
import pytest
import torch

import pippy_amd.microbatch as mb
from pippy_amd.microbatch import (TensorChunkSpec, _Replicate, merge_chunks, split_args_kwargs_into_chunks,
                                  sum_reducer)

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _make(shape, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    if dtype.is_floating_point:
        return torch.randn(shape, generator=g).to(dtype).to(DEV)
    return torch.randint(-1000, 1000, shape, generator=g).to(dtype).to(DEV)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.int64, torch.uint8])
@pytest.mark.parametrize("shape,dim,n", [((6, 10, 7), 1, 4), ((3, 5, 16), 2, 3), ((4, 9), 1, 9),
                                         ((2, 3, 4, 10), 2, 2), ((8, 33, 50), 1, 8), ((5, 4, 1001), 2, 7)])
def test_split_along_inner_dims_matches_tensor_split(dtype, shape, dim, n):
    x = _make(shape, dtype)
    args_split, kwargs_split = split_args_kwargs_into_chunks((x,), {"k": x}, n, (TensorChunkSpec(dim),),
                                                             {"k": TensorChunkSpec(dim)})
    expect = torch.tensor_split(x, n, dim)
    assert len(args_split) == len(kwargs_split) == n
    for m in range(n):
        got = args_split[m][0]
        assert got.is_cuda and got.is_contiguous()
        assert torch.equal(got, expect[m])
        assert torch.equal(kwargs_split[m]["k"], expect[m])
    # and back
    merged = merge_chunks([a[0] for a in args_split], TensorChunkSpec(dim))
    assert torch.equal(merged, x)


@pytest.mark.parametrize("dim", [0, 1, 2])
def test_split_of_non_contiguous_inputs(dim):
    base = _make((12, 10, 14), torch.bfloat16)
    views = {"transposed": base.transpose(0, 2), "strided": base[::2, :, 1::3], "offset": base[1:, 2:, :]}
    for name, v in views.items():
        assert not v.is_contiguous()
        n = 3
        got = split_args_kwargs_into_chunks((v,), None, n, (TensorChunkSpec(dim),))[0]
        expect = torch.tensor_split(v, n, dim)
        for m in range(n):
            assert torch.equal(got[m][0], expect[m]), (name, dim, m)


def test_replicated_and_non_tensor_leaves_and_nested_structures():
    x = _make((8, 6), torch.float32)
    w = _make((3, 3), torch.float32, seed=1)
    args = ((x, {"w": w, "flag": 7}),)
    spec = ((TensorChunkSpec(1), {"w": _Replicate, "flag": _Replicate}),)
    chunks, _ = split_args_kwargs_into_chunks(args, None, 3, spec)
    expect = torch.tensor_split(x, 3, 1)
    for m, (arg,) in enumerate(chunks):
        xs, d = arg
        assert torch.equal(xs, expect[m])
        assert d["w"] is w and d["flag"] == 7
    # merged back: the tensor is concatenated, replicated leaves are taken from the first chunk
    merged = merge_chunks([(c[0][0], c[0][1]["flag"]) for c in chunks], (TensorChunkSpec(1), None))
    assert torch.equal(merged[0], x) and merged[1] == 7


@pytest.mark.parametrize("dim", [0, 1, 2])
def test_debug_mask_layout_and_round_trip(dim, monkeypatch):
    """Each microbatch is the full-size tensor, zero outside its own slice
    (layout of the reference's test_ir.py:696-709); the merge keeps each chunk's own slice."""
    monkeypatch.setattr(mb, "_debug_mask_minibatches", True)
    x = _make((6, 5, 8), torch.bfloat16)
    n = 3
    chunks, _ = split_args_kwargs_into_chunks((x,), None, n, (TensorChunkSpec(dim),))
    lo = 0
    for m, size in enumerate(mb.chunk_sizes(x.size(dim), n)):
        full = chunks[m][0]
        assert full.shape == x.shape
        expect = torch.zeros_like(x)
        expect.narrow(dim, lo, size).copy_(x.narrow(dim, lo, size))
        assert torch.equal(full, expect)
        lo += size
    merged = merge_chunks([c[0] for c in chunks], TensorChunkSpec(dim))
    assert torch.equal(merged, x)


def test_merge_with_reducer_and_non_contiguous_chunks():
    x = _make((4, 6, 10), torch.float32)
    parts = list(torch.tensor_split(x.transpose(1, 2), 3, 2))  # non-contiguous chunks, cut along dim 2
    assert not parts[0].is_contiguous()
    losses = [torch.tensor(float(m + 1), device=DEV) for m in range(3)]
    chunks = [(parts[m], losses[m]) for m in range(3)]
    merged, total = merge_chunks(chunks, (TensorChunkSpec(2), sum_reducer))
    assert torch.equal(merged, torch.cat(parts, 2))
    assert merged.is_contiguous()
    assert float(total) == 6.0
    # sliced chunks whose rows are strided in memory
    y = _make((9, 8), torch.bfloat16)
    cols = [y[:, 0:3], y[:, 3:4], y[:, 4:8]]
    assert torch.equal(merge_chunks(cols, TensorChunkSpec(1)), y)
    rows = [y[0:9:2], y[1:9:2]]
    assert torch.equal(merge_chunks(rows, TensorChunkSpec(0)), torch.cat(rows, 0))


def test_chunk_count_shrinks_on_the_first_tensor_only():
    x = _make((2, 16), torch.float32)
    y = _make((8, 16), torch.float32)
    chunks, kw = split_args_kwargs_into_chunks((x,), {"y": y}, 4)
    assert len(chunks) == len(kw) == 2
    assert torch.equal(kw[1]["y"], torch.tensor_split(y, 2)[1])
    with pytest.raises(RuntimeError, match="smaller than the number of chunks"):
        split_args_kwargs_into_chunks((y, x), None, 4)
