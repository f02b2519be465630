"""Checkpoint I/O keyed by the names of the un-split model (reference
pippy/utilities/hf_checkpoint.py; name invariant of test/test_fwd.py:86-92)."""
import json
import os

import pytest
import torch
import torch.nn as nn


class _Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.layer0 = nn.Linear(8, 16)
        self.layer1 = nn.Linear(16, 16)
        self.norm = nn.LayerNorm(16)
        self.register_buffer("scale", torch.full((16,), 0.5))
        self.out = nn.Linear(16, 4)

    def forward(self, x):
        x = torch.relu(self.layer0(x))
        x = torch.relu(self.layer1(x))
        return self.out(self.norm(x) * self.scale)


def _pipe(seed):
    import pippy_amd as pp
    torch.manual_seed(seed)
    model = _Net()
    pipe = pp.pipeline(model, 2, (torch.randn(4, 8),), split_spec={"layer1": pp.SplitPoint.BEGINNING})
    return model, pipe


def test_save_writes_one_binary_per_stage_and_an_index_of_original_names(tmp_path):
    from pippy_amd.utilities.hf_checkpoint import CKPT_INDEX_JSON_FILENAME, save_checkpoint
    model, pipe = _pipe(0)
    index_path = save_checkpoint(pipe, str(tmp_path))
    assert os.path.basename(index_path) == CKPT_INDEX_JSON_FILENAME
    index = json.load(open(index_path))
    names = set(model.state_dict().keys())
    assert set(index["weight_map"].keys()) == names
    assert index["metadata"]["total_size"] == sum(t.numel() * t.element_size() for t in model.state_dict().values())
    files = sorted(set(index["weight_map"].values()))
    assert files == ["pytorch_model-00001-of-00002.bin", "pytorch_model-00002-of-00002.bin"]
    assert index["weight_map"]["layer0.weight"] == files[0] and index["weight_map"]["out.bias"] == files[1]
    shard = torch.load(tmp_path / files[1], weights_only=True)
    assert torch.equal(shard["out.weight"], model.out.weight)


def test_load_restores_each_stage_in_place_and_only_opens_its_own_file(tmp_path):
    from pippy_amd.utilities.hf_checkpoint import load_checkpoint, save_checkpoint
    model, pipe = _pipe(0)
    index_path = save_checkpoint(pipe, str(tmp_path))
    other, other_pipe = _pipe(1)
    assert not torch.equal(other.layer1.weight, model.layer1.weight)
    stage1 = other_pipe.get_stage_module(1)
    before = {n: p for n, p in stage1.named_parameters()}
    os.remove(tmp_path / "pytorch_model-00001-of-00002.bin")       # stage 1 does not need it
    load_checkpoint(stage1, index_path)
    for n, p in stage1.named_parameters():
        assert p is before[n]                                       # same objects, new values
        assert torch.equal(p, model.state_dict()[n])
    assert torch.equal(dict(stage1.named_buffers())["scale"], model.scale)
    with pytest.raises(FileNotFoundError):
        load_checkpoint(other_pipe.get_stage_module(0), index_path)


def test_name_matching_prefixes_shared_weights_and_missing_names(tmp_path):
    from pippy_amd.utilities.hf_checkpoint import _match_checkpoint_name, load_checkpoint
    index = {"h.0.w": "a.bin", "transformer.ln.weight": "a.bin", "wte.weight": "b.bin"}
    assert _match_checkpoint_name("h.0.w", index, ["model", "transformer"]) == ("h.0.w", False)
    assert _match_checkpoint_name("transformer.h.0.w", index, ["model", "transformer"]) == ("h.0.w", False)
    assert _match_checkpoint_name("ln.weight", index, ["model", "transformer"]) == ("transformer.ln.weight", False)
    assert _match_checkpoint_name("lm_head.weight", index, ["model"]) == ("wte.weight", True)
    assert _match_checkpoint_name("missing", index, ["model"]) == (None, False)
    torch.save({"h.weight": torch.ones(2, 2)}, tmp_path / "a.bin")
    json.dump({"weight_map": {"h.weight": "a.bin"}}, open(tmp_path / "index.json", "w"))
    m = nn.Module()
    m.model = nn.Module()
    m.model.h = nn.Linear(2, 2, bias=False)
    load_checkpoint(m, str(tmp_path / "index.json"))
    assert torch.equal(m.model.h.weight, torch.ones(2, 2))
    m.extra = nn.Linear(2, 2)
    with pytest.raises(RuntimeError, match="not found in checkpoint index"):
        load_checkpoint(m, str(tmp_path / "index.json"))
    m2 = nn.Module()
    m2.h = nn.Linear(3, 2, bias=False)
    with pytest.raises(RuntimeError, match="shape"):
        load_checkpoint(m2, str(tmp_path / "index.json"))
