"""Host bookkeeping helpers (mirrors ``pippy/_utils.py:13-53`` of the reference)."""
from typing import Any, List

import torch
from torch.utils._pytree import tree_flatten, tree_map


def flatten_args(args) -> List[Any]:
    """Flattens nested args into a list of leaves (reference ``_utils.py:37-53``)."""
    flat, _ = tree_flatten(args)
    return flat


def flatten_args_detach(args):
    """Detaches every tensor leaf, keeping ``requires_grad`` (reference ``_utils.py:13-34``).
    Returns (new_args, flat_detached_tensors)."""
    flat_detached = []

    def detach(a):
        if isinstance(a, torch.Tensor):
            d = a.detach().requires_grad_(a.requires_grad)
            flat_detached.append(d)
            return d
        flat_detached.append(a)
        return a

    return tree_map(detach, args), flat_detached
