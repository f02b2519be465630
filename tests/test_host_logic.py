"""Host-side logic that needs no GPU: microbatch bookkeeping, schedule orders, the splitting
front end, error behaviour, and the C ABI surface of the built library."""
import ctypes
import os
import re
import subprocess
import sys
from collections import namedtuple

import pytest
import torch
import torch.nn as nn

import pippy_amd as pp
from oracle import schedules as OS
from pippy_amd import _native, _schedule_order as order
from pippy_amd import microbatch as MB
from pippy_amd._lowering import lower_stage_module
from pippy_amd.microbatch import (TensorChunkSpec, _Replicate, chunk_sizes, merge_chunks,
                                  split_args_kwargs_into_chunks, sum_reducer)
from pippy_amd.stage import ManualPipelineStage

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- microbatch split (views of host tensors; no data movement) -----------------------------------
def _golden(name):
    import json
    with open(os.path.join(ROOT, "tests", "golden", name)) as f:
        return json.load(f)


def test_split_shapes_of_the_reference_test():
    """The chunk shapes that test/test_microbatch.py:17-34 of the reference asserts."""
    gold = _golden("microbatch_split_shapes.json")
    d, n = gold["width"], gold["chunks"]
    xs = [torch.randn(r, d) for r in gold["rows"]]
    args, kwargs = tuple(xs), {f"x{i}": x for i, x in enumerate(xs)}
    a, k = split_args_kwargs_into_chunks(args, kwargs, n)
    assert len(a) == n and len(k) == n
    for c in range(n):
        assert [tuple(t.shape) for t in a[c]] == [(r, d) for r in gold["chunk_rows"][c]]
        assert [tuple(k[c][f"x{i}"].shape) for i in range(len(xs))] == [(r, d) for r in gold["chunk_rows"][c]]
    # chunks are views of the caller's tensors, as in the reference (no bytes move)
    assert a[1][0].data_ptr() == xs[0][64:].data_ptr()
    for i, x in enumerate(args):
        assert torch.equal(torch.cat([c[i] for c in a]), x)


@pytest.mark.parametrize("size,n", [(10, 4), (3, 3), (8, 8), (1, 1), (50257, 8), (0, 3)])
def test_chunk_sizes_match_tensor_split(size, n):
    ref = [t.shape[0] for t in torch.tensor_split(torch.empty(size, device="meta"), n)]
    assert chunk_sizes(size, n) == ref


def test_replicate_and_namedtuple_chunking():
    """test/test_ir.py:598-680 of the reference (the split part)."""
    NT = namedtuple("NT", ["my_tensor", "my_integer"])
    x, nt = torch.randn(5, 3), NT(torch.randn(5, 3), 42)
    a, k = split_args_kwargs_into_chunks((x,), {"input_nt": nt}, chunks=5, args_chunk_spec=(_Replicate,),
                                         kwargs_chunk_spec={"input_nt": NT(TensorChunkSpec(0), _Replicate)})
    assert len(a) == 5 and len(k) == 5
    for i in range(5):
        assert a[i][0] is x
        assert isinstance(k[i]["input_nt"], NT) and k[i]["input_nt"].my_integer == 42
        assert torch.equal(k[i]["input_nt"].my_tensor, nt.my_tensor[i:i + 1])


def test_fewer_rows_than_chunks_shrinks_or_raises():
    a, k = split_args_kwargs_into_chunks((torch.randn(3, 2),), None, 8)
    assert len(a) == 3  # first tensor decides (reference microbatch.py:120-129)
    with pytest.raises(RuntimeError, match="smaller than the number of chunks"):
        split_args_kwargs_into_chunks((torch.randn(8, 2), torch.randn(3, 2)), None, 8)


def test_split_error_types():
    with pytest.raises(ValueError):
        split_args_kwargs_into_chunks(((torch.randn(4, 2), torch.randn(4, 2)),), None, 2,
                                      args_chunk_spec=(TensorChunkSpec(0),))
    with pytest.raises(TypeError, match="Unrecognized chunk spec"):
        split_args_kwargs_into_chunks((torch.randn(4, 2),), None, 2, args_chunk_spec=(object(),))


def test_debug_mask_layout_on_host():
    """test/test_ir.py:696-709 of the reference: full-size chunks, zero outside the own slice."""
    x = torch.randn(5, 3)
    MB._debug_mask_minibatches = True
    try:
        a, _ = split_args_kwargs_into_chunks((x,), None, 5)
    finally:
        MB._debug_mask_minibatches = False
    for i, (c,) in enumerate(a):
        assert c.shape == x.shape
        assert torch.equal(c[i:i + 1], x[i:i + 1])
        assert float(c[:i].abs().sum()) == 0 and float(c[i + 1:].abs().sum()) == 0


def test_merge_reducer_and_replicated_leaves_on_host():
    chunks = [{"loss": torch.tensor(float(i)), "tag": "same"} for i in range(4)]
    out = merge_chunks(chunks, {"loss": sum_reducer, "tag": None})
    assert out["tag"] == "same" and float(out["loss"]) == 6.0
    with pytest.raises(ValueError, match="did not match chunk spec"):
        merge_chunks([(torch.zeros(1), torch.zeros(1))], (TensorChunkSpec(0),))
    with pytest.raises(RuntimeError, match="no CPU data path"):
        merge_chunks([torch.zeros(2, 2), torch.zeros(2, 2)], None)


def test_row_view_descriptions():
    buf = torch.empty(256, 1024, dtype=torch.bfloat16)
    v = buf.view(2, 128, 1024)[..., :1000]          # padded logits rows
    assert MB._row_view(v, 0) == (256, 2000, 2048, 256)
    c = torch.empty(4, 5, 6)
    assert MB._row_view(c, 0) == (1, 480, 480, 1)
    assert MB._row_view(c, 1) == (4, 120, 120, 1)
    assert MB._row_view(torch.empty(4, 6, 5).transpose(1, 2), 0) is None


# ---- schedule orders ----------------------------------------------------------------------------------
def test_1f1b_phases_known_answer():
    """The worked example in the reference's comment at PipelineSchedule.py:373-377."""
    gold = _golden("schedule_1f1b_phases.json")
    S, M = gold["num_stages"], gold["num_microbatches"]
    assert [list(order.one_f_one_b_phases(s, S, M)) for s in range(S)] == gold["phases_per_stage"]


@pytest.mark.parametrize("S,M", [(1, 1), (2, 4), (4, 8), (4, 2), (3, 7)])
def test_rank_programs_equal_the_simulated_reference(S, M):
    for s in range(S):
        assert order.gpipe_rank_program(s, M, True) == list(OS.gpipe_rank(s, M))
        assert order.one_f_one_b_rank_program(s, S, M, True) == list(OS.one_f_one_b_rank(s, S, M))
        assert order.one_f_one_b_rank_program(s, S, M, False) == list(OS.one_f_one_b_rank(s, S, M, False))


@pytest.mark.parametrize("G,n_local,M", [(1, 2, 8), (2, 2, 4), (2, 2, 8), (4, 2, 8), (2, 3, 4)])
def test_multi_stage_rank_programs_equal_the_simulated_reference(G, n_local, M):
    S = G * n_local
    for r in range(G):
        local = [s for s in range(S) if s % G == r]
        assert order.interleaved_rank_program(r, G, local, M) == list(OS.interleaved_rank(r, G, local, M))
        assert order.looped_bfs_rank_program(local, M, True) == list(OS.looped_bfs_rank(local, M))


def _invariants(actions, S, M, split=False):
    pos = {a: i for i, a in enumerate(actions)}
    assert len(pos) == len(actions)
    bk = "I" if split else "B"
    for s in range(S):
        for m in range(M):
            if s > 0:
                assert pos[("F", s - 1, m)] < pos[("F", s, m)]
            if s < S - 1:
                assert pos[(bk, s + 1, m)] < pos[(bk, s, m)]
            assert pos[("F", s, m)] < pos[(bk, s, m)]
            if split:
                assert pos[("I", s, m)] < pos[("W", s, m)]
            if m > 0:
                assert pos[("F", s, m - 1)] < pos[("F", s, m)]
                assert pos[(bk, s, m - 1)] < pos[(bk, s, m)]
                if split:
                    assert pos[("W", s, m - 1)] < pos[("W", s, m)]


@pytest.mark.parametrize("S,M", [(1, 3), (2, 4), (4, 8), (4, 16), (3, 2)])
def test_merged_orders_respect_dependencies(S, M):
    progs = [order.one_f_one_b_rank_program(s, S, M, True) for s in range(S)]
    merged = order.merge_rank_programs(progs, S)
    assert len(merged) == 2 * S * M
    _invariants(merged, S, M)
    zb = order.merge_rank_programs([order.zero_bubble_rank_program(s, S, M) for s in range(S)], S)
    assert len(zb) == 3 * S * M
    _invariants(zb, S, M, split=True)


def test_merge_detects_deadlock():
    with pytest.raises(RuntimeError, match="dead-lock"):
        order.merge_rank_programs([[("B", 0, 0), ("F", 0, 0)]], 1)


# ---- front end ------------------------------------------------------------------------------------------
class _Block(nn.Module):
    def __init__(self, i, o):
        super().__init__()
        self.lin = nn.Linear(i, o)

    def forward(self, x):
        return torch.relu(self.lin(x))


class _Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.num_layers = 3
        prev = 16
        for i, d in enumerate([16, 32, 8]):
            self.add_module(f"layer{i}", _Block(prev, d))
            prev = d
        self.output_proj = nn.Linear(prev, 4)

    def forward(self, x):
        for i in range(self.num_layers):
            x = getattr(self, f"layer{i}")(x)
        return self.output_proj(x)


def test_pipeline_splits_and_keeps_parameter_names():
    """test/test_pipe.py:78-110 of the reference: stage count, output equality, stage state_dict
    keys are a partition of the original keys."""
    torch.manual_seed(0)
    mod = _Net()
    x = torch.randn(8, 16)
    pipe = pp.pipeline(mod, 4, (x,), split_spec={"layer1": pp.SplitPoint.BEGINNING,
                                                 "layer2": pp.SplitPoint.END})
    assert pipe.num_stages == 3
    assert torch.equal(pipe(x), mod(x))
    old = set(mod.state_dict().keys())
    seen = set()
    for i in range(pipe.num_stages):
        keys = set(pipe.get_stage_module(i).state_dict().keys())
        assert keys <= old and not (keys & seen)
        seen |= keys
    assert seen == old
    info = pipe.info()
    assert info.num_stages == 3 and info.num_chunks == 4
    assert all(lower_stage_module(pipe.get_stage_module(i)) is not None for i in range(3))


def test_pipe_split_calls_in_forward():
    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.a, self.b = nn.Linear(4, 4), nn.Linear(4, 4)

        def forward(self, x):
            x = self.a(x)
            pp.pipe_split()
            return self.b(x)

    m = M()
    x = torch.randn(2, 4)
    pipe = pp.pipeline(m, 2, (x,))
    assert pipe.num_stages == 2 and torch.equal(pipe(x), m(x))


def test_annotate_split_points_and_errors():
    m = _Net()
    pp.annotate_split_points(m, {"layer2": pp.SplitPoint.BEGINNING})
    x = torch.randn(4, 16)
    ref = m(x)
    pipe = pp.pipeline(m, 2, (x,))
    assert pipe.num_stages == 2 and torch.equal(pipe(x), ref)
    with pytest.raises(ValueError, match="Cannot specify both"):
        pp.pipeline(_Net(), 2, (x,), split_spec={"layer1": pp.SplitPoint.END}, split_policy=lambda g: g)
    with pytest.raises(ValueError, match="not a module called"):
        pp.pipeline(_Net(), 2, (x,), split_spec={"nope": pp.SplitPoint.END})
    with pytest.raises(ValueError, match="Invalid stage index"):
        pipe.get_stage_module(5)


def test_root_level_parameters_and_buffers_move_into_the_stage_that_reads_them():
    """A tensor that the model's forward reads itself (not through a child module) belongs to the
    stage that uses it, under its original name (reference ``_IR.py:785-895`` sinks them)."""
    import pippy_amd as pp

    class Scaled(nn.Module):
        def __init__(self):
            super().__init__()
            self.a = nn.Linear(4, 4)
            self.b = nn.Linear(4, 4)
            self.gain = nn.Parameter(torch.full((4,), 2.0))
            self.register_buffer("shift", torch.arange(4.0))

        def forward(self, x):
            x = self.a(x) + self.shift
            pp.pipe_split()
            return self.b(x) * self.gain

    torch.manual_seed(0)
    model = Scaled()
    x = torch.randn(6, 4)
    pipe = pp.pipeline(model, 2, (x,))
    s0, s1 = pipe.get_stage_module(0), pipe.get_stage_module(1)
    assert set(s0.state_dict()) == {"a.weight", "a.bias", "shift"}
    assert set(s1.state_dict()) == {"b.weight", "b.bias", "gain"}
    assert dict(s1.named_parameters())["gain"] is model.gain
    assert len([n for n in s1.graph.nodes if n.op == "placeholder"]) == 1
    assert torch.equal(pipe(x), model(x))


def test_shared_parameters_are_rejected():
    class Tied(nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = nn.Linear(4, 4, bias=False)
            self.mid = nn.Linear(4, 4)

        def forward(self, x):
            x = self.emb(x)
            pp.pipe_split()
            return self.emb(self.mid(x))

    with pytest.raises(NotImplementedError, match="shared"):
        pp.pipeline(Tied(), 2, (torch.randn(2, 4),))


def test_chunk_spec_context_managers():
    """test/test_chunkspec.py:42-62 of the reference."""
    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = nn.Linear(4, 4)

        def forward(self, x, y, z=None):
            return self.lin(x) + y + z

    x, y, z = torch.randn(6, 4), torch.randn(6, 4), torch.randn(6, 4)
    with pp.ArgsChunkSpec((0, 0)), pp.KwargsChunkSpec({"z": 0}):
        pipe = pp.pipeline(M(), 3, (x, y), {"z": z})
    info = pipe.info()
    assert [s.split_dim for s in info.args_chunk_spec] == [0, 0]
    assert info.kwargs_chunk_spec["z"].split_dim == 0
    assert pp.Pipe.args_chunk_spec is None and pp.Pipe.kwargs_chunk_spec is None


def test_lowering_decisions():
    from pippy_amd.configs import DecoderLM
    m = DecoderLM(vocab=64, max_seq=16, dim=64, n_layers=2, n_heads=1, ffn=128)
    names = [type(b).__name__ for b in lower_stage_module(m)]
    assert names == ["TokenEmbedding", "TransformerLayer", "TransformerLayer", "LMHead"]
    assert [type(b).__name__ for b in lower_stage_module(_Net())] == ["LinearAct"] * 4

    class Skip(nn.Module):
        def __init__(self):
            super().__init__()
            self.a = nn.Linear(4, 4)

        def forward(self, x):
            return x + self.a(x)

    assert lower_stage_module(Skip()) is None  # not a chain: runs through autograd instead


# ---- stage / schedule argument checking (reference test_pipeline_schedule.py:477-521) ----------------
def _host_stages(n):
    mods = [nn.Linear(4, 4) for _ in range(n)]
    return [ManualPipelineStage(mods[i], i, n, "cpu", 8, input_args=torch.zeros(1, 4)) for i in range(n)]


def test_stage_constructor_errors():
    with pytest.raises(ValueError, match="out of range"):
        ManualPipelineStage(nn.Linear(2, 2), 3, 2, "cpu", 4)
    with pytest.raises(RuntimeError, match="cannot be larger than number of stages"):
        ManualPipelineStage(nn.Linear(2, 2), 0, 2, "cpu", 4, group=4)


def test_schedule_input_checks():
    sched = pp.Schedule1F1B(_host_stages(1), 8)
    with pytest.raises(ValueError):
        sched._step_microbatches([(i,) for i in range(7)])
    with pytest.raises(TypeError):
        sched._step_microbatches(torch.ones(8, 4, 8))
    with pytest.raises(TypeError):
        sched._step_microbatches([(torch.zeros(1, 4),)] * 8, losses=1)
    with pytest.raises(ValueError, match="at least two stages"):
        pp.ScheduleInterleaved1F1B(_host_stages(1), 8)
    stages = [ManualPipelineStage(nn.Linear(4, 4), i, 4, "cpu", 8, group=2) for i in range(4)]
    with pytest.raises(ValueError, match="multiple of the number of pipeline ranks"):
        pp.ScheduleInterleaved1F1B(stages, 7)
    partial = [ManualPipelineStage(nn.Linear(4, 4), 1, 3, "cpu", 8)]
    with pytest.raises(RuntimeError, match="every stage must be given"):
        pp.ScheduleGPipe(partial, 8)._step_microbatches([()] * 8)


def test_product_code_never_imports_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "pippy_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, re.M), f


# ---- C ABI --------------------------------------------------------------------------------------------
def _header_functions():
    text = open(os.path.join(ROOT, "include", "pippy_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pp_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _header_functions()
    assert names and set(names) == set(_native.EXPORTED_SYMBOLS)
    lib = ctypes.CDLL(str(_native.LIB_PATH))
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"
    assert _native.lib().pp_abi_version() == 1


def test_ctypes_structs_match_the_header(tmp_path):
    src = tmp_path / "sizes.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "pippy_amd.h"\n'
                   'int main(void){printf("%zu %zu %zu %zu %zu %zu %zu\\n", sizeof(pp_copy_seg), '
                   'sizeof(pp_gemm_desc), sizeof(pp_attn_desc), sizeof(pp_op), offsetof(pp_op, i), '
                   'offsetof(pp_op, j), offsetof(pp_gemm_desc, bias));return 0;}\n')
    exe = tmp_path / "sizes"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    got = [int(v) for v in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()]
    N = _native
    want = [ctypes.sizeof(N.CopySeg), ctypes.sizeof(N.GemmDesc), ctypes.sizeof(N.AttnDesc), ctypes.sizeof(N.Op),
            N.Op.i.offset, N.Op.j.offset, N.GemmDesc.bias.offset]
    assert got == want


def test_verbosity_from_the_environment():
    """PIPPY_VERBOSITY sets the package logger's level; an unknown value falls back to WARNING
    (reference ``pippy/_debug.py:13-18``)."""
    import logging
    from pippy_amd import _debug
    try:
        assert _debug.configure("DEBUG") == "DEBUG"
        assert logging.getLogger("pippy_amd").level == logging.DEBUG
        assert logging.getLogger("pippy_amd.schedules").getEffectiveLevel() == logging.DEBUG
        assert _debug.configure("LOUD") == "WARNING"
        assert logging.getLogger("pippy_amd").level == logging.WARNING
    finally:
        _debug.configure()
    assert _debug.map_debug_info([torch.zeros(2, 3), 5]) == ["Tensor((2, 3), grad=False)", "5"]


def test_pipeline_accepts_the_microbatch_spelling_and_build_stage():
    """``pipeline(module, mb_args=...)`` and ``pipe.build_stage(i, device)``, as the reference's examples
    call them (examples/huggingface/pippy_gpt2.py:50-65, examples/llama/pippy_llama.py:36-39)."""
    torch.manual_seed(0)
    model = _Net()
    x = torch.randn(8, 16)
    a = pp.pipeline(model, 4, (x,), split_spec={"layer1": pp.SplitPoint.BEGINNING})
    b = pp.pipeline(model, mb_args=(x[:2],), split_spec={"layer1": pp.SplitPoint.BEGINNING})
    assert a.num_stages == b.num_stages == 2
    for i in range(2):
        assert list(a.get_stage_module(i).state_dict()) == list(b.get_stage_module(i).state_dict())
    assert torch.equal(b(x), model(x))
    stage = b.build_stage(1, "cpu")
    assert isinstance(stage, pp.PipelineStage) and stage.stage_index == 1 and stage.num_stages == 2
    with pytest.raises(ValueError, match="either"):
        pp.pipeline(model, 4, (x,), mb_args=(x,))
    with pytest.raises(TypeError, match="num_chunks"):
        pp.pipeline(model)


# ---- example values of a hand-built stage are a checked contract (reference ManualPipelineStage.py:342-439)
def test_manual_stage_checks_live_shapes_against_its_examples():
    from pippy_amd.stage import validate_stage_shapes
    lin = nn.Linear(4, 6)
    kw = dict(force_eager=True)   # host tensors: the torch path (launch lists take device tensors)
    stage = ManualPipelineStage(lin, 0, 1, "cpu", 2, input_args=torch.zeros(3, 4), output_args=torch.zeros(3, 6), **kw)
    assert not stage.is_native and stage.eager_reason
    sched = pp.ScheduleGPipe([stage], 2)
    out = sched._step_microbatches([(torch.ones(3, 4),), (torch.ones(3, 4),)])
    assert out is None and len(stage.output_chunks) == 2
    stage.clear_runtime_states()
    with pytest.raises(ValueError, match="example inputs"):
        sched._step_microbatches([(torch.ones(2, 4),), (torch.ones(2, 4),)])
    wrong_out = ManualPipelineStage(lin, 0, 1, "cpu", 1, input_args=torch.zeros(3, 4), output_args=torch.zeros(3, 5), **kw)
    with pytest.raises(ValueError, match="example outputs"):
        pp.ScheduleGPipe([wrong_out], 1)._step_microbatches([(torch.ones(3, 4),)])
    wrong_dtype = ManualPipelineStage(lin, 0, 1, "cpu", 1, input_args=torch.zeros(3, 4, dtype=torch.float64), **kw)
    with pytest.raises(ValueError, match="example inputs"):
        pp.ScheduleGPipe([wrong_dtype], 1)._step_microbatches([(torch.ones(3, 4),)])

    a = ManualPipelineStage(nn.Linear(4, 6), 0, 2, "cpu", 1, input_args=torch.zeros(3, 4), output_args=torch.zeros(3, 6))
    b = ManualPipelineStage(nn.Linear(6, 2), 1, 2, "cpu", 1, input_args=torch.zeros(3, 6))
    validate_stage_shapes([a, b])
    c = ManualPipelineStage(nn.Linear(5, 2), 1, 2, "cpu", 1, input_args=torch.zeros(3, 5))
    with pytest.raises(ValueError, match="does not match stage_id 1 input shape"):
        validate_stage_shapes([a, c])
    d = ManualPipelineStage(nn.Linear(6, 2), 1, 3, "cpu", 1, input_args=torch.zeros(3, 6))
    with pytest.raises(ValueError, match="num stages"):
        validate_stage_shapes([a, d])
    with pytest.raises(ValueError, match="No pipeline stages"):
        validate_stage_shapes([])


def test_a_stage_that_cannot_be_lowered_says_why(caplog):
    class Branchy(nn.Module):
        def __init__(self):
            super().__init__()
            self.a = nn.Linear(4, 4)

        def forward(self, x):
            return x + self.a(x)

    import logging
    from pippy_amd._lowering import lower_stage_module
    why = []
    assert lower_stage_module(Branchy(), why) is None and "does not continue a chain" in why[0]
    with caplog.at_level(logging.WARNING, logger="pippy_amd.stage"):
        stage = ManualPipelineStage(Branchy(), 0, 1, "cpu", 1)
    assert not stage.is_native and stage.eager_reason
    assert any("runs eagerly" in r.getMessage() for r in caplog.records)
    why = []
    assert lower_stage_module(nn.Sequential(nn.Linear(4, 4), nn.ReLU(), nn.Linear(4, 2)), why) and not why
    assert lower_stage_module(nn.Linear(4, 2), why) and not why
    host = ManualPipelineStage(nn.Linear(4, 2), 0, 1, "cpu", 1)
    assert not host.is_native and "GPU only" in host.eager_reason


# ---- a transformer written with plain torch layers lowers to the same blocks --------------------------
def test_plain_torch_transformer_is_recognised_and_verified():
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import GPT, Block
    from pippy_amd._lowering import lower_stage_module
    torch.manual_seed(0)
    model = GPT(vocab=500, seq=64, d=128, h=2, L=4)
    why = []
    blocks = lower_stage_module(model, why)
    assert [type(b).__name__ for b in blocks] == ["WrappedTokenEmbedding"] + ["WrappedTransformerLayer"] * 4 + ["WrappedLMHead"]
    # the wrappers hold the model's own layers: nothing is copied or renamed
    assert blocks[1].attn.c_attn is model.h[0].c_attn and blocks[-1].lm_head is model.lm_head
    assert blocks[1].n_heads == 2 and blocks[1].causal and blocks[1].activation == "gelu_tanh"
    # stages cut by the front end lower too, with the model's parameter names
    ids = torch.randint(0, 500, (4, 64))
    pipe = pp.pipeline(model, 2, (ids,), split_spec={"h.2": pp.SplitPoint.BEGINNING})
    kinds = [[type(b).__name__ for b in lower_stage_module(pipe.get_stage_module(i))] for i in range(2)]
    assert kinds == [["WrappedTokenEmbedding"] + ["WrappedTransformerLayer"] * 2,
                     ["WrappedTransformerLayer"] * 2 + ["WrappedLMHead"]]
    assert "h.2.c_attn.weight" in pipe.get_stage_module(1).state_dict()

    # a model whose heads are not what the kernels are built for stays with torch, and says why
    why = []
    assert lower_stage_module(GPT(d=96, h=3), why) is None and "head dimension" in why[0]

    # a block that computes something else between the same layers fails the numerical check
    class Scaled(Block):
        def forward(self, x):
            return super().forward(x) * 1.5

    odd = GPT(vocab=500, seq=64, d=128, h=2, L=1)
    odd.h[0] = Scaled(128, 2)
    why = []
    assert lower_stage_module(odd, why) is None
    assert "residual" in why[0]


# ---- size-based split policies (reference pippy/ModelSplit.py:158-206) ---------------------------------
def test_split_policies_cut_by_parameter_count():
    from pippy_amd.configs import DecoderLM
    torch.manual_seed(0)
    model = DecoderLM(vocab=1000, max_seq=64, dim=128, n_layers=8, n_heads=2, ffn=512).float()
    ids = torch.randint(0, 1000, (4, 64))
    per_layer = sum(p.numel() for p in model.h[0].parameters())
    pipe = pp.pipeline(model, 2, (ids,), split_policy=pp.split_into_equal_size(4))
    assert pipe.num_stages == 4
    torch.testing.assert_close(pipe(ids), model(ids), rtol=0, atol=0)
    sizes = [sum(p.numel() for p in pipe.get_stage_module(i).parameters()) for i in range(4)]
    assert sum(sizes) == sum(p.numel() for p in model.parameters())
    assert all(s <= sum(sizes) // 4 for s in sizes[:-1])          # only the last stage may run over
    # a threshold of three layers: the embedding and two layers, then stages of three layers
    pipe = pp.pipeline(model, 2, (ids,), split_policy=pp.split_on_size_threshold(3 * per_layer))
    sizes = [sum(p.numel() for p in pipe.get_stage_module(i).parameters()) for i in range(pipe.num_stages)]
    assert all(s <= 3 * per_layer for s in sizes) and sizes[1] == 3 * per_layer
    torch.testing.assert_close(pipe(ids), model(ids), rtol=0, atol=0)
    with pytest.raises(ValueError):
        pp.pipeline(model, 2, (ids,), split_spec={"h.4": pp.SplitPoint.BEGINNING},
                    split_policy=pp.split_into_equal_size(2))
    with pytest.raises(NotImplementedError):
        pp.split_by_graph(2)


def test_whether_a_dropout_is_a_no_op_is_decided_when_the_stage_is_lowered():
    """A dropout with p > 0 is identity in eval mode only.  Lowering takes the decision once: in eval
    mode the stage becomes launch lists, in training mode it stays with torch autograd (and says why)."""
    from pippy_amd._lowering import lower_stage_module
    m = nn.Sequential(nn.Linear(16, 32), nn.ReLU(), nn.Dropout(0.1), nn.Linear(32, 16)).to(torch.bfloat16)
    m.eval()
    why = []
    assert lower_stage_module(m, why, for_kernels=True) is not None
    m.train()
    why = []
    assert lower_stage_module(m, why, for_kernels=True) is None
    assert "dropout" in why[0]
    # p == 0 is a no-op in either mode
    m[2].p = 0.0
    assert lower_stage_module(m, [], for_kernels=True) is not None


def test_a_launch_list_stage_refuses_to_run_after_its_dropout_was_switched_on():
    """The launch lists hold no dropout: a stage lowered in eval mode whose module is then put into
    training mode (p > 0) raises instead of training without dropout; back in eval mode it runs."""
    import pippy_amd as pp
    from pippy_amd import stage as stage_mod
    m = nn.Sequential(nn.Linear(16, 32), nn.ReLU(), nn.Dropout(0.1), nn.Linear(32, 16)).to(torch.bfloat16).eval()
    st = pp.ManualPipelineStage(m, 0, 1, "cpu", 1, input_args=(torch.zeros(2, 16, dtype=torch.bfloat16),))
    assert st._mode_bound_dropouts == []          # eager on the CPU: torch's own dropout applies, nothing to guard
    # the guard itself, on a stage object made to look lowered (launch lists need the GPU)
    st._mode_bound_dropouts = [m[2]]
    m.train()
    with pytest.raises(RuntimeError, match="dropout"):
        stage_mod.PipelineStageBase._forward_native(st, 0, (), {})


def test_size_policy_counts_a_layers_parameters_not_its_buffers():
    """Reference ``ModelSplit.py:45-52``: a layer call weighs what ``named_parameters`` holds.  The running
    statistics of a normalisation layer (buffers) must not move the cut."""
    import pippy_amd as pp
    model = nn.Sequential(nn.Linear(8, 8), nn.BatchNorm1d(8), nn.Linear(8, 8), nn.BatchNorm1d(8),
                          nn.Linear(8, 8), nn.BatchNorm1d(8), nn.Linear(8, 8), nn.BatchNorm1d(8)).eval()
    pair = (8 * 8 + 8) + 2 * 8           # a linear layer and the weight and bias of its normalisation
    # two pairs per stage by their parameters; with the 17 buffer elements of each BatchNorm counted too the
    # second pair would not fit
    pipe = pp.pipeline(model, 1, (torch.zeros(2, 8),), split_policy=pp.split_on_size_threshold(2 * pair))
    assert pipe.num_stages == 2
    keys0 = set(pipe.get_stage_module(0).state_dict())
    assert {k.split(".")[0] for k in keys0} == {"0", "1", "2", "3"}
