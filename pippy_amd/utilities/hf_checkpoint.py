"""Sharded checkpoints keyed by the original model's parameter names, with a Hugging Face style
index file.

Same surface as the reference utility (``pippy/utilities/hf_checkpoint.py``: ``save_checkpoint``
at ``:424-452``, ``load_checkpoint`` at ``:64-144``, index layout at ``:350-392``, name matching at
``:205-241``): one binary per pipeline stage, ``pytorch_model-0000i-of-0000S.bin``, holding that
stage's parameters and buffers under the names they have in the un-split model (stage modules here
keep those names, reference ``test/test_fwd.py:86-92``), plus ``pytorch_model.bin.index.json`` with
``metadata.total_size`` and the ``weight_map`` from name to file.

Differences that follow from running every stage in one process on one GPU: ``save_checkpoint``
takes all stages at once instead of being called once per rank; binaries hold plain tensors and are
read back with ``torch.load(weights_only=True)``; loading copies *into* the existing parameters
(``param.copy_``) instead of replacing them, because the parameters of a lowered stage are views of
the stage's flat arena that its launch lists point to.
"""
from __future__ import annotations

import json
import os
import pathlib
import tempfile
from typing import Dict, Iterable, List, Optional, Sequence, Tuple, Union

import torch
from torch import nn

CKPT_INDEX_JSON_FILENAME = "pytorch_model.bin.index.json"

# prefixes that checkpoints of common model families put in front of, or leave out of, the names
TYPICAL_PREFIXES = ["model", "transformer"]
# a tied output projection may be stored only under the name of the embedding it shares
TYPICAL_SHARER_WEIGHTS = ["lm_head.weight", "encoder_embed_tokens.weight"]
TYPICAL_SHAREE_WEIGHTS = ["decoder.embed_tokens.weight", "word_embeddings.weight", "shared.weight", "wte.weight"]


def _binary_filename(idx: int, count: int, is_optim: bool = False) -> str:
    kind = "optim" if is_optim else "model"
    return f"pytorch_{kind}-{str(idx + 1).zfill(5)}-of-{str(count).zfill(5)}.bin"


def _module_of(stage) -> nn.Module:
    return stage.submod if hasattr(stage, "submod") else stage


def _named_tensors(module: nn.Module) -> Iterable[Tuple[str, torch.Tensor]]:
    yield from module.named_parameters()
    yield from module.named_buffers()


def _atomic_write(text: str, path: str) -> None:
    """Writes through a temporary file in the same directory, then renames."""
    tmp = tempfile.NamedTemporaryFile("w", delete=False, dir=os.path.dirname(path) or ".")
    try:
        with tmp as f:
            f.write(text)
            f.flush()
            os.fsync(f.fileno())
        os.replace(tmp.name, path)
    finally:
        if os.path.exists(tmp.name):
            os.unlink(tmp.name)


def save_checkpoint(stages, checkpoint_dir: str = "checkpoints", optimizer=None) -> str:
    """Writes one binary per stage and the index; returns the index path.  ``stages``: a list of
    pipeline stages (or stage modules), or a ``Pipe``.  ``optimizer``: anything with
    ``state_dict()``; its state goes to ``pytorch_optim-00001-of-00001.bin``."""
    if hasattr(stages, "num_stages") and hasattr(stages, "get_stage_module"):
        stages = [stages.get_stage_module(i) for i in range(stages.num_stages)]
    modules = [_module_of(s) for s in (stages if isinstance(stages, (list, tuple)) else [stages])]
    pathlib.Path(checkpoint_dir).mkdir(parents=True, exist_ok=True)
    weight_map: Dict[str, str] = {}
    total_size = 0
    for idx, mod in enumerate(modules):
        fname = _binary_filename(idx, len(modules))
        shard = {}
        for name, t in _named_tensors(mod):
            if name not in weight_map:
                total_size += t.numel() * t.element_size()
            weight_map[name] = fname
            shard[name] = t.detach().to("cpu", copy=True).contiguous()
        torch.save(shard, os.path.join(checkpoint_dir, fname))
    index = {"metadata": {"total_size": total_size}, "weight_map": weight_map}
    index_path = os.path.join(checkpoint_dir, CKPT_INDEX_JSON_FILENAME)
    _atomic_write(json.dumps(index, indent=4), index_path)
    if optimizer is not None:
        torch.save(optimizer.state_dict(), os.path.join(checkpoint_dir, _binary_filename(0, 1, is_optim=True)))
    return index_path


def _match_checkpoint_name(name: str, index: Dict[str, str], prefixes: Sequence[str]) -> Tuple[Optional[str], bool]:
    """Name under which ``name`` is stored and whether the tensor is shared with another weight.
    Tried in order: the name itself; the name without, or with, one of ``prefixes``; for a tied
    output projection, the embedding it shares."""
    if name in index:
        return name, False
    for prefix in prefixes:
        if name.startswith(prefix + ".") and name[len(prefix) + 1:] in index:
            return name[len(prefix) + 1:], False
        if prefix + "." + name in index:
            return prefix + "." + name, False
    if name in TYPICAL_SHARER_WEIGHTS or name.split(".", 1)[-1] in TYPICAL_SHARER_WEIGHTS:
        for sharee in TYPICAL_SHAREE_WEIGHTS:
            for key in index:
                if key == sharee or key.endswith("." + sharee):
                    return key, True
    return None, False


def load_checkpoint(model, index_filename: Union[str, os.PathLike], optim=None, device=None, dtype=None,
                    checkpoint_prefix: Optional[str] = None):
    """Loads the tensors that ``model`` (a stage, a stage module or a whole model) owns from the
    checkpoint behind ``index_filename``; only the binaries that hold them are opened.  Values are
    cast to the dtype of the tensor they replace and copied in place (stage tensors are views of the
    stage's flat arenas and keep their dtype: a floating-point ``dtype`` that differs from it raises
    ``RuntimeError``).  Also raises ``RuntimeError`` when a tensor of ``model`` is not in the index."""
    module = _module_of(model)
    folder = os.path.split(index_filename)[0]
    with open(index_filename, "r") as f:
        index = json.load(f)
    index = index.get("weight_map", index)
    prefixes = [checkpoint_prefix] if checkpoint_prefix else TYPICAL_PREFIXES
    file_to_weights: Dict[str, List[Tuple[torch.Tensor, str, str]]] = {}
    for name, tensor in _named_tensors(module):
        stored, _shared = _match_checkpoint_name(name, index, prefixes)
        if stored is None:
            raise RuntimeError(f"Weight {name} is not found in checkpoint index")
        file_to_weights.setdefault(index[stored], []).append((tensor, name, stored))
    for fname, weights in file_to_weights.items():
        shard = torch.load(os.path.join(folder, fname), map_location="cpu", weights_only=True)
        for tensor, name, stored in weights:
            if stored not in shard:
                raise RuntimeError(f"{stored} not in {fname}")
            value = shard[stored]
            if tuple(value.shape) != tuple(tensor.shape):
                raise RuntimeError(f"{name}: checkpoint shape {tuple(value.shape)} != {tuple(tensor.shape)}")
            with torch.no_grad():
                if dtype is not None and tensor.dtype != dtype and tensor.is_floating_point():
                    raise RuntimeError(f"{name}: a stage tensor keeps its dtype {tensor.dtype} (asked for {dtype})")
                if device is not None and torch.device(device).type != tensor.device.type:
                    raise RuntimeError(f"{name} lives on {tensor.device}; move the model before loading")
                tensor.copy_(value.to(tensor.dtype))   # in place: bumps the version launch lists watch
        del shard
    if optim is not None:
        optim.load_state_dict(torch.load(os.path.join(folder, _binary_filename(0, 1, is_optim=True)),
                                         map_location="cpu", weights_only=True))
        return model, optim
    return model
