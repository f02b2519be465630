"""Stage backward (mirrors ``pippy/_backward.py`` of the reference).

``stage_backward`` keeps the reference signature and semantics for autograd-traced stage outputs
(eager stages).  Native stages do not go through autograd: their backward is the pair of launch
lists run by ``PipelineStageBase.backward_input_one_chunk`` / ``backward_weight_one_chunk``.
"""
from typing import List, Optional

import torch


def _debug_info(v):
    if isinstance(v, torch.Tensor):
        return f"Tensor({tuple(v.shape)}, grad={v.requires_grad}, dtype={v.dtype})"
    if isinstance(v, (list, tuple)):
        return type(v)(_debug_info(x) for x in v)
    if isinstance(v, dict):
        return {k: _debug_info(x) for k, x in v.items()}
    return repr(v)


def stage_backward(stage_output, output_grads, input_values,
                   outputs_with_grads_idxs: Optional[List[int]] = None):
    """Computes the gradients of the stage inputs and accumulates the parameter gradients
    (reference ``_backward.py:9-102``): walk outputs and their gradients in parallel, keep the
    tensors that take part in autograd, run one ``torch.autograd.backward`` and read ``.grad`` of
    the inputs."""
    if outputs_with_grads_idxs is not None:  # deprecated argument kept for signature parity
        stage_output = [stage_output[i] for i in outputs_with_grads_idxs]
        output_grads = [output_grads[i] for i in outputs_with_grads_idxs]
    try:
        outs: List[torch.Tensor] = []
        grads: List[Optional[torch.Tensor]] = []

        def collect(o, g):
            if isinstance(o, torch.Tensor):
                if not o.requires_grad and o.grad_fn is None:
                    return
                assert isinstance(g, (torch.Tensor, type(None))), \
                    f"Expected Tensor or None gradient but got {type(g)}"
                outs.append(o)
                grads.append(g)
            elif isinstance(o, (tuple, list)):
                if g is None:
                    return
                assert isinstance(g, (tuple, list)), \
                    f"grad_value expected to have type {type(o)} but got {type(g)}"
                assert len(o) == len(g)
                for oo, gg in zip(o, g):
                    collect(oo, gg)
            elif isinstance(o, dict):
                if g is None:
                    return
                assert isinstance(g, dict)
                assert set(o.keys()) == set(g.keys())
                for k in o.keys():
                    collect(o[k], g[k])

        collect(stage_output, output_grads)
        torch.autograd.backward(outs, grad_tensors=grads)
        grad_inputs = [v.grad if isinstance(v, torch.Tensor) else None for v in input_values]
    except Exception as e:
        raise RuntimeError(
            "Failed to run stage backward:\n"
            f"Stage output: {_debug_info(stage_output)}\n"
            f"Output gradient: {_debug_info(output_grads)}\n"
            f"Input: {_debug_info(input_values)}") from e
    return grad_inputs


def _null_coalesce_accumulate(lhs, rhs):
    """Adds two values either of which may be None (reference ``_backward.py:107-117``)."""
    if lhs is None:
        return rhs
    if rhs is None:
        return lhs
    return torch.add(lhs, rhs)
