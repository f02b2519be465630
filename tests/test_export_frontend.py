"""The ``torch.export`` route of the front end (reference ``pippy/_IR.py:1141-1145,679-1125``): a model
that ``torch.fx`` symbolic tracing cannot follow is exported on the inputs of one microbatch and cut at
the markers.  Checked with the invariants of the reference's ``test/test_pipe.py:78-110`` (stage count,
``Pipe(x) == mod(x)``, the stages' state-dict keys partition the model's) and, end to end on the host,
with those of ``test/test_fwd.py:80-84`` / ``test/test_grad.py:103-136`` (pipelined output and gradients
equal the un-pipelined model's)."""
import copy

import pytest
import torch
import torch.fx as fx
import torch.nn as nn

import pippy_amd as pp


class _Block(nn.Module):
    def __init__(self, d):
        super().__init__()
        self.lin = nn.Linear(d, d)
        self.ln = nn.LayerNorm(d)

    def forward(self, x):
        h = self.lin(x)
        if h.shape[-1] > 4:      # Python control flow on a shape: symbolic tracing stops here
            h = torch.relu(h)
        return self.ln(h) + x


class _Model(nn.Module):
    def __init__(self, d=8, marker_at=None):
        super().__init__()
        self.scale = nn.Parameter(torch.rand(d) + 0.5)
        self.marker_at = marker_at
        self.layers = nn.ModuleList([_Block(d) for _ in range(4)])
        self.head = nn.Linear(d, 3)

    def forward(self, x):
        x = x * self.scale
        for i, layer in enumerate(self.layers):
            if self.marker_at == i:
                pp.pipe_split()
            x = layer(x)
        return self.head(x)


def _check_partition(pipe, model):
    keys = []
    for i in range(pipe.num_stages):
        stage_mod = pipe.get_stage_module(i)
        keys += list(stage_mod.state_dict().keys())
        for name, p in stage_mod.named_parameters():
            assert p is model.get_parameter(name), f"{name} is not the model's own parameter"
    assert sorted(keys) == sorted(model.state_dict().keys())


def test_symbolic_tracing_really_fails_on_this_model():
    with pytest.raises(Exception):
        fx.symbolic_trace(_Model())


@pytest.mark.parametrize("spec,marker_at,n_stages", [
    ({"layers.1": pp.SplitPoint.BEGINNING, "layers.2": pp.SplitPoint.END}, None, 3),
    (None, 2, 2),
    ({"layers.3": pp.SplitPoint.BEGINNING}, 1, 3),
])
def test_export_fallback_keeps_names_and_results(spec, marker_at, n_stages):
    torch.manual_seed(0)
    model = _Model(marker_at=marker_at)
    x = torch.randn(8, 8)
    pipe = pp.pipeline(model, 4, (x,), split_spec=spec)
    assert pipe.num_stages == n_stages
    _check_partition(pipe, model)
    assert torch.equal(pipe(x), model(x))
    # the marker does nothing when the model simply runs
    assert model(x).shape == (8, 3)


def test_export_fallback_pipeline_trains_like_the_unsplit_model():
    torch.manual_seed(1)
    model = _Model()
    ref = copy.deepcopy(model)
    x, target = torch.randn(8, 8), torch.randn(8, 3)
    pipe = pp.pipeline(model, 4, (x,), split_spec={"layers.2": pp.SplitPoint.BEGINNING})
    stages = [pp.PipelineStage(pipe, i, "cpu") for i in range(pipe.num_stages)]
    assert not any(st.is_native for st in stages)
    loss_fn = nn.MSELoss(reduction="sum")
    for cls in (pp.ScheduleGPipe, pp.Schedule1F1B):
        for p in model.parameters():
            p.grad = None
        losses = []
        # the microbatch lists are handed over directly: merging host tensors is not something this
        # package does (its merge is a device kernel), so the chunks are compared after a torch.cat
        for st in stages:
            st.clear_runtime_states()
        cls(stages, 4, loss_fn=loss_fn)._step_microbatches([(c,) for c in x.chunk(4)], None,
                                                           list(target.chunk(4)), losses)
        out = torch.cat(stages[-1].output_chunks)
        for p in ref.parameters():
            p.grad = None
        ref_out = ref(x)
        ref_loss = loss_fn(ref_out, target)
        ref_loss.backward()
        torch.testing.assert_close(out, ref_out)
        torch.testing.assert_close(sum(losses), ref_loss)
        for (n, p), (_, rp) in zip(model.named_parameters(), ref.named_parameters()):
            # microbatch sums against one full-batch sum: fp32 rounding only (the reference's own
            # backward test allows rtol 1e-2 / atol 5e-3, test/test_bwd.py:98)
            torch.testing.assert_close(p.grad, rp.grad, rtol=1e-4, atol=1e-4, msg=lambda m, n=n: f"{n}: {m}")


def test_split_point_that_is_not_in_the_model_raises_on_the_export_route_too():
    with pytest.raises(ValueError, match="not a module called by the model"):
        pp.pipeline(_Model(), 2, (torch.randn(4, 8),), split_spec={"nowhere": pp.SplitPoint.BEGINNING})


# ---- exported stages keep whole layers and lower to launch lists when their structure is recognised ----
def _lib_gpt():
    import os, sys
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import LibGPT
    torch.manual_seed(0)
    return LibGPT(vocab=500, seq=64, d=128, h=2, L=4)


def test_exported_stages_hold_the_models_own_layers_and_no_constant_computation():
    model = _lib_gpt()
    with pytest.raises(Exception):
        fx.symbolic_trace(model)
    ids = torch.randint(0, 500, (2, 32))
    pipe = pp.pipeline(model, 1, (ids,), split_spec={"h.2": pp.SplitPoint.BEGINNING})
    assert pipe.num_stages == 2
    torch.testing.assert_close(pipe(ids), model(ids), rtol=0, atol=0)
    _check_partition(pipe, model)
    for i in range(2):
        sm = pipe.get_stage_module(i)
        layers = {n.target for n in sm.graph.nodes if n.op == "call_module"}
        for name, layer in model.named_modules():
            if name and next(layer.children(), None) is None and name.startswith(("h.0.", "h.1.") if i == 0 else ("h.2.", "h.3.")):
                assert name in layers, f"{name} was not put back as a layer call"
                assert sm.get_submodule(name) is layer
        # one activation in, one activation out: the mask and the position indices are constants of the stage
        assert len([n for n in sm.graph.nodes if n.op == "placeholder"]) == 1
        assert not [n for n in sm.graph.nodes if n.op == "call_function" and "arange" in str(n.target)]
        assert not [k for k in sm.state_dict() if "_folded_constant" in k]


def test_exported_library_style_transformer_is_recognised_and_verified():
    from pippy_amd._lowering import lower_stage_module
    from pippy_amd.stage_modules import InOutLinear
    model = _lib_gpt()
    ids = torch.randint(0, 500, (2, 32))
    pipe = pp.pipeline(model, 1, (ids,), split_spec={"h.2": pp.SplitPoint.BEGINNING})
    why = []
    kinds = [[type(b).__name__ for b in lower_stage_module(pipe.get_stage_module(i), why)] for i in range(2)]
    assert not why
    assert kinds == [["WrappedTokenEmbedding"] + ["WrappedTransformerLayer"] * 2,
                     ["WrappedTransformerLayer"] * 2 + ["WrappedLMHead"]]
    layer = lower_stage_module(pipe.get_stage_module(1))[0]
    # [in, out] affine layers are wrapped, not copied; the constant mask was read as causal
    assert isinstance(layer.attn.c_attn, InOutLinear) and layer.attn.c_attn.layer is model.h[2].attn.c_attn
    assert layer.causal and layer.n_heads == 2 and layer.activation == "gelu_tanh"
    x = torch.randn(2, 32, 128)
    torch.testing.assert_close(layer(x), model.h[2](x, torch.ones(32, 32, dtype=torch.bool).tril()))


def test_a_mask_that_is_not_causal_keeps_the_stage_with_torch():
    from pippy_amd._lowering import lower_stage_module
    model = _lib_gpt()
    orig = model.forward

    def windowed(idx):
        t = idx.shape[-1]
        pos = torch.arange(t).unsqueeze(0)
        mask = ((pos.unsqueeze(-1) >= pos.unsqueeze(-2)) & (pos.unsqueeze(-1) - pos.unsqueeze(-2) < 8))[:, None]
        mask = mask.expand(idx.shape[0], 1, t, t)
        x = model.wte(idx) + model.wpe(pos)
        if t > 1:
            for blk in model.h:
                x = blk(x, mask)
        return model.lm_head(model.ln_f(x))

    model.forward = windowed
    ids = torch.randint(0, 500, (2, 32))
    pipe = pp.pipeline(model, 1, (ids,), split_spec={"h.2": pp.SplitPoint.BEGINNING})
    why = []
    assert lower_stage_module(pipe.get_stage_module(1), why) is None
    assert "mask" in why[0]


def test_shared_layers_mutated_buffers_and_keyword_inputs_survive_the_graph_passes():
    """A layer called twice is put back twice; buffers that the forward writes (batch-norm statistics, a
    step counter) are not mistaken for constants; keyword inputs reach the stage that reads them."""
    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.a, self.shared, self.b = nn.Linear(8, 8), nn.Linear(8, 8), nn.Linear(8, 4)
            self.bn = nn.BatchNorm1d(8)
            self.register_buffer("steps", torch.zeros(()))

        def forward(self, x, scale=None):
            if x.shape[0] > 1:
                x = self.a(x)
            x = self.bn(self.shared(torch.relu(self.shared(x))))
            self.steps += 1
            pp.pipe_split()
            if scale is not None:
                x = x * scale
            return self.b(x)

    torch.manual_seed(0)
    model, ref = Net(), Net()
    ref.load_state_dict(model.state_dict())
    x, scale = torch.randn(4, 8), torch.rand(4, 1)
    pipe = pp.pipeline(model, mb_args=(x,), mb_kwargs={"scale": scale})
    assert pipe.num_stages == 2
    calls = [n.target for n in pipe.get_stage_module(0).graph.nodes if n.op == "call_module"]
    assert calls == ["a", "shared", "shared"]
    for _ in range(2):
        torch.testing.assert_close(pipe(x, scale=scale), ref(x, scale=scale), rtol=0, atol=0)
    assert model.steps.item() == ref.steps.item() == 2      # (exporting runs the forward on fake tensors only)
    torch.testing.assert_close(model.bn.running_var, ref.bn.running_var)


def test_what_the_kernels_cannot_take_keeps_a_recognised_stage_with_torch():
    """The structure of an exported stage may be recognised and still not run as launch lists: float32
    parameters (the transformer kernels are bf16)."""
    from pippy_amd._lowering import lower_stage_module
    model = _lib_gpt()
    ids = torch.randint(0, 500, (2, 64))
    stage = pp.pipeline(model, 1, (ids,), split_spec={"h.2": pp.SplitPoint.BEGINNING}).get_stage_module(1)
    why = []
    assert lower_stage_module(stage, why) is not None
    assert lower_stage_module(stage, why, for_kernels=True) is None and "float32" in why[-1]
    model = _lib_gpt().to(torch.bfloat16)
    stage = pp.pipeline(model, 1, (ids,), split_spec={"h.2": pp.SplitPoint.BEGINNING}).get_stage_module(1)
    assert lower_stage_module(stage, why, for_kernels=True) is not None
    # any sequence length: the layers pad to a multiple of 64 by themselves
    stage = pp.pipeline(model, 1, (ids[:, :48],), split_spec={"h.2": pp.SplitPoint.BEGINNING}).get_stage_module(1)
    assert lower_stage_module(stage, why, for_kernels=True) is not None
    # widths: the bf16 kernels move groups of 8 values; fp32 chains of linear layers take any width; a
    # vocabulary projection keeps its rows padded and may have any number of them
    chain = nn.Sequential(nn.Linear(64, 100), nn.ReLU(), nn.Linear(100, 8))
    assert lower_stage_module(chain, why, for_kernels=True) is not None
    del why[:]
    assert lower_stage_module(chain.to(torch.bfloat16), why, for_kernels=True) is None
    assert "out width 100" in why[0] and "multiples of 8" in why[0]
    head = nn.Sequential(nn.Linear(64, 64), nn.LayerNorm(64), nn.Linear(64, 1001, bias=False)).to(torch.bfloat16)
    blocks = lower_stage_module(head, why, for_kernels=True)
    assert blocks is not None and type(blocks[-1]).__name__ == "WrappedLMHead"


def test_a_layer_subclass_with_a_forward_of_its_own_is_not_put_back_blindly():
    """OPT's position table is an ``nn.Embedding`` subclass whose forward shifts its indices by two.
    After constant folding, the exported nodes of that call are a plain look-up at the shifted constant:
    calling the subclass there would shift twice.  The look-up goes back as the base layer's view of the
    same parameter, the stage lowers with the table read from row 2 on, and a ReLU feed-forward lowers."""
    from pippy_amd._lowering import lower_stage_module
    model = _lib_gpt()

    class Shifted(nn.Embedding):
        def forward(self, pos):
            return super().forward(pos + 2)

    class Relu(nn.Module):
        def forward(self, x):
            return torch.relu(x)

    table = Shifted(66, 128)
    model.wpe = table
    for blk in model.h:
        blk.mlp.act = Relu()
    ids = torch.randint(0, 500, (2, 32))
    pipe = pp.pipeline(model, 1, (ids,), split_spec={"h.2": pp.SplitPoint.BEGINNING})
    torch.testing.assert_close(pipe(ids), model(ids), rtol=0, atol=0)
    _check_partition(pipe, model)
    sm = pipe.get_stage_module(0)
    assert type(sm.get_submodule("wpe")) is nn.Embedding and sm.get_submodule("wpe").weight is table.weight
    why = []
    blocks = lower_stage_module(sm, why)
    assert blocks is not None, why
    assert blocks[0].position_offset == 2 and blocks[0].wpe.weight is table.weight
    assert blocks[1].activation == "relu"
    x = ids
    with torch.no_grad():
        for b in blocks:
            x = b(x)
        torch.testing.assert_close(x, sm(ids), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("factor", ["default", "none", "queries"])
def test_attention_spelled_out_is_recognised_with_its_mask_and_factor(factor):
    """A model that writes attention as softmax(q k^T c, masked) v (the non-fused path of many code bases):
    the softmax stands for the attention call, the constant mask filled in where it is *set* is read as
    causal, and the factor on the scores — the default, none at all, or one applied to the queries
    beforehand — becomes the block's ``attn_scale``."""
    import math
    import torch.nn.functional as F
    from pippy_amd._lowering import lower_stage_module
    model = _lib_gpt()

    def spelled_out(self, x, mask):
        B, T, C = x.size()
        D = C // self.n_head
        q, k, v = (t.view(B, T, self.n_head, D).transpose(1, 2) for t in self.c_attn(x).split(C, dim=2))
        if factor == "queries":
            q = q * 0.2
        att = q @ k.transpose(-2, -1)
        if factor == "default":
            att = att / math.sqrt(D)
        att = att.masked_fill(~mask, float("-inf"))
        y = F.softmax(att, dim=-1) @ v
        return self.resid_dropout(self.c_proj(y.transpose(1, 2).reshape(B, T, C)))

    for blk in model.h:
        blk.attn.forward = spelled_out.__get__(blk.attn)
    ids = torch.randint(0, 500, (2, 32))
    pipe = pp.pipeline(model, 1, (ids,), split_spec={"h.2": pp.SplitPoint.BEGINNING})
    torch.testing.assert_close(pipe(ids), model(ids), rtol=0, atol=0)
    for i in range(2):
        sm = pipe.get_stage_module(i)
        why = []
        blocks = lower_stage_module(sm, why)
        assert blocks is not None, why
        layers = [b for b in blocks if type(b).__name__ == "WrappedTransformerLayer"]
        assert len(layers) == 2 and all(b.causal for b in layers)
        want = {"default": None, "none": 1.0, "queries": 0.2}[factor]
        assert all(b.attn_scale == want if want is None else abs(b.attn_scale - want) < 1e-9 for b in layers)


@pytest.mark.parametrize("norm_first,activation", [(True, "gelu"), (False, "relu")])
def test_torchs_own_encoder_layers_become_transformer_blocks(norm_first, activation):
    """``nn.TransformerEncoderLayer`` (batch first, called without a mask) is taken as a whole: a transformer
    block around its own parameters, the packed q|k|v projection of ``nn.MultiheadAttention`` seen through
    an ``nn.Linear`` view of the same parameter objects.  What it cannot take is said."""
    import os, sys
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import TorchEncoderLM
    from pippy_amd._lowering import lower_stage_module
    torch.manual_seed(0)
    model = TorchEncoderLM(vocab=500, seq=64, norm_first=norm_first, activation=activation)
    ids = torch.randint(0, 500, (2, 40))
    pipe = pp.pipeline(model, 1, (ids,), split_spec={"layers.2": pp.SplitPoint.BEGINNING})
    torch.testing.assert_close(pipe(ids), model(ids), rtol=0, atol=0)
    x = ids
    for i in range(2):
        why = []
        blocks = lower_stage_module(pipe.get_stage_module(i), why)
        assert blocks is not None, why
        layers = [b for b in blocks if type(b).__name__ == "WrappedTransformerLayer"]
        assert len(layers) == 2
        for b, own in zip(layers, model.layers[2 * i:2 * i + 2]):
            assert b.attn.c_attn.weight is own.self_attn.in_proj_weight and b.attn.c_attn.bias is own.self_attn.in_proj_bias
            assert b.attn.c_proj is own.self_attn.out_proj and b.mlp.c_fc is own.linear1 and b.ln_2 is own.norm2
            assert (b.pre_ln, b.causal, b.n_heads) == (norm_first, False, 2)
            assert b.activation == {"gelu": "gelu_erf", "relu": "relu"}[activation]
        with torch.no_grad():
            for b in blocks:
                x = b(x)
    torch.testing.assert_close(x, model(ids), rtol=1e-4, atol=1e-4)
    # a last projection onto a width that is no multiple of 8 becomes the head block (padded rows) in bf16
    odd = TorchEncoderLM(vocab=501, seq=64, norm_first=norm_first, activation=activation).to(torch.bfloat16)
    pipe = pp.pipeline(odd, 1, (ids,), split_spec={"layers.2": pp.SplitPoint.BEGINNING})
    tail = lower_stage_module(pipe.get_stage_module(1), [])[-1]
    assert type(tail).__name__ == "WrappedLMHead" and tail.lm_head is odd.head and tail.ln_f is odd.norm
    # sequence-major layers and head sizes the kernels do not have stay with torch, with the reason
    other = TorchEncoderLM(vocab=500, seq=64, d=96, h=2)
    pipe = pp.pipeline(other, 1, (ids,), split_spec={"layers.2": pp.SplitPoint.BEGINNING})
    why = []
    assert lower_stage_module(pipe.get_stage_module(1), why) is None and "head size 48" in why[0]
    other = TorchEncoderLM(vocab=500, seq=64)
    for layer in other.layers:
        layer.self_attn.batch_first = False
    pipe = pp.pipeline(other, 1, (ids,), split_spec={"layers.2": pp.SplitPoint.BEGINNING})
    why = []
    assert lower_stage_module(pipe.get_stage_module(1), why) is None and "batch_first" in why[0]


@pytest.mark.parametrize("norm_first", [True, False])
def test_torchs_encoder_stack_is_recognised_through_its_exported_graph(norm_first):
    """``nn.TransformerEncoder`` goes through torch.export; ``nn.MultiheadAttention`` applies its packed
    q|k|v parameters and its output projection as functions of parameters, which are taken as linear layers
    (views of the same parameter objects); the sequence-major reshaping inside is not parsed but checked."""
    import os, sys
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import TorchEncoderStackLM
    from pippy_amd._lowering import lower_stage_module
    torch.manual_seed(0)
    model = TorchEncoderStackLM(vocab=500, seq=64, norm_first=norm_first)
    ids = torch.randint(0, 500, (2, 40))
    pipe = pp.pipeline(model, 1, (ids,), split_spec={"encoder.layers.2": pp.SplitPoint.BEGINNING})
    torch.testing.assert_close(pipe(ids), model(ids), rtol=0, atol=0)
    _check_partition(pipe, model)
    x = ids
    for i in range(2):
        why = []
        blocks = lower_stage_module(pipe.get_stage_module(i), why)
        assert blocks is not None, why
        layers = [b for b in blocks if type(b).__name__ == "WrappedTransformerLayer"]
        assert len(layers) == 2
        for b, own in zip(layers, model.encoder.layers[2 * i:2 * i + 2]):
            assert b.attn.c_attn.weight is own.self_attn.in_proj_weight
            assert b.attn.c_proj.weight is own.self_attn.out_proj.weight and b.mlp.c_fc is own.linear1
            assert (b.pre_ln, b.causal, b.n_heads, b.activation) == (norm_first, False, 2, "gelu_erf")
        with torch.no_grad():
            for b in blocks:
                x = b(x)
    torch.testing.assert_close(x, model(ids), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("flag", [True, False])
def test_values_computed_from_shapes_do_not_travel_between_stages(flag, caplog):
    """torch.fx can trace this model (each encoder layer is one call), but the causal mask that forward
    builds from the sequence length would then be a second tensor on every stage boundary.  The front end
    notices, exports the model instead, where the mask is a constant of each stage, and says so; the
    stages are then recognised as causal transformer layers.  A real skip connection keeps the traced
    pipeline (its exported form has the same boundary)."""
    import logging, os, sys
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import TorchCausalLM
    from pippy_amd._lowering import lower_stage_module
    torch.manual_seed(0)
    model = TorchCausalLM(vocab=500, seq=64, flag=flag)
    ids = torch.randint(0, 500, (2, 40))
    with caplog.at_level(logging.WARNING, logger="pippy_amd._IR"):
        pipe = pp.pipeline(model, 1, (ids,), split_spec={"layers.2": pp.SplitPoint.BEGINNING})
    assert "more than one tensor" in caplog.text
    torch.testing.assert_close(pipe(ids), model(ids), rtol=0, atol=0)
    _check_partition(pipe, model)
    for i in range(2):
        sm = pipe.get_stage_module(i)
        assert len([n for n in sm.graph.nodes if n.op == "placeholder"]) == 1
        why = []
        blocks = lower_stage_module(sm, why)
        assert blocks is not None, why
        layers = [b for b in blocks if type(b).__name__ == "WrappedTransformerLayer"]
        assert len(layers) == 2 and all(b.causal and b.pre_ln for b in layers)

    class Skip(nn.Module):
        def __init__(self):
            super().__init__()
            self.a, self.b, self.c = nn.Linear(16, 16), nn.Linear(16, 16), nn.Linear(16, 16)

        def forward(self, x):
            first = torch.relu(self.a(x))
            pp.pipe_split()
            y = torch.relu(self.b(first))
            pp.pipe_split()
            return self.c(y + first)

    caplog.clear()
    with caplog.at_level(logging.WARNING, logger="pippy_amd._IR"):
        skip = pp.pipeline(Skip(), 1, (torch.randn(4, 16),))
    assert "more than one tensor" not in caplog.text and skip.num_stages == 3
    assert any(n.op == "call_module" and n.target == "b" for n in skip.get_stage_module(1).graph.nodes)


@pytest.mark.parametrize("bias,flash", [(True, True), (True, False), (False, True), (False, False)])
def test_a_teaching_style_gpt_with_its_own_layer_norm_is_recognised(bias, flash):
    """The GPT of small teaching code bases: a layer-norm class of its own (``F.layer_norm`` on its
    parameters, the bias optional) is taken as the ``nn.LayerNorm`` it amounts to (a view of the same
    parameter objects, the epsilon found by comparison), attention through the fused call or spelled out
    against a registered lower-triangular buffer, layers with or without biases."""
    import os, sys
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import TeachingGPT
    from pippy_amd._lowering import lower_stage_module
    from pippy_amd.stage_modules import layer_norm_like
    torch.manual_seed(0)
    model = TeachingGPT(vocab=500, seq=64, bias=bias, flash=flash)
    keys = set(model.state_dict())
    ids = torch.randint(0, 500, (2, 40))
    pipe = pp.pipeline(model, 1, (ids,), split_spec={"transformer.h.2": pp.SplitPoint.BEGINNING})
    torch.testing.assert_close(pipe(ids), model(ids), rtol=0, atol=0)
    _check_partition(pipe, model)
    x = ids
    for i in range(2):
        why = []
        blocks = lower_stage_module(pipe.get_stage_module(i), why)
        assert blocks is not None, why
        layers = [b for b in blocks if type(b).__name__ == "WrappedTransformerLayer"]
        assert len(layers) == 2 and all(b.causal and b.pre_ln and b.activation == "gelu_erf" for b in layers)
        own = model.transformer.h[2 * i]
        assert layers[0].ln_1.weight is own.ln_1.weight and layers[0].ln_1.eps == 1e-5
        assert (layers[0].ln_1.bias is own.ln_1.bias) if bias else layers[0].ln_1.bias is None
        with torch.no_grad():
            for b in blocks:
                x = b(x)
    torch.testing.assert_close(x, model(ids), rtol=1e-4, atol=1e-4)
    assert set(model.state_dict()) == keys          # recognising the layers left the model as it was
    view = layer_norm_like(model.transformer.ln_f)
    assert view is layer_norm_like(model.transformer.ln_f) and isinstance(view, nn.LayerNorm)
    assert layer_norm_like(nn.LayerNorm(8)) is None and layer_norm_like(nn.Linear(8, 8)) is None


@pytest.mark.parametrize("need_weights,causal", [(True, False), (True, True), (False, False), (False, True)])
def test_blocks_around_torchs_attention_layer_are_recognised(need_weights, causal):
    """``nn.MultiheadAttention`` inside a block of one's own.  Without a mask torch.fx keeps the layer as one
    call, which is taken as its packed projection, the attention and its output projection; with a mask
    built from the sequence length the model is exported, and with ``need_weights`` (the layer's default)
    the layer spells its attention out (the mask added by ``baddbmm``); the averaged weights, which nobody
    reads, are dropped."""
    import os, sys
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import MHAModel
    from pippy_amd._lowering import lower_stage_module
    torch.manual_seed(0)
    model = MHAModel(vocab=500, seq=64, need_weights=need_weights, causal=causal)
    ids = torch.randint(0, 500, (2, 40))
    pipe = pp.pipeline(model, 1, (ids,), split_spec={"blocks.2": pp.SplitPoint.BEGINNING})
    torch.testing.assert_close(pipe(ids), model(ids), rtol=0, atol=0)
    _check_partition(pipe, model)
    x = ids
    for i in range(2):
        why = []
        blocks = lower_stage_module(pipe.get_stage_module(i), why)
        assert blocks is not None, why
        layers = [b for b in blocks if type(b).__name__ == "WrappedTransformerLayer"]
        assert len(layers) == 2 and all(b.causal == causal and b.pre_ln and b.attn_scale is None for b in layers)
        own = model.blocks[2 * i].attn
        assert layers[0].attn.c_attn.weight is own.in_proj_weight and layers[0].attn.c_proj.weight is own.out_proj.weight
        with torch.no_grad():
            for b in blocks:
                x = b(x)
    torch.testing.assert_close(x, model(ids), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("boolean,flag", [(False, True), (True, False)])
def test_torchs_encoder_layers_called_with_a_registered_causal_mask(boolean, flag):
    """``layer(x, src_mask=self.mask)`` with the mask a registered buffer (additive, or boolean with True for
    what is masked), with or without ``is_causal=True``: torch.fx keeps the calls whole, the mask is read
    from the buffer, and the comparison with the stage runs at the mask's size."""
    from pippy_amd._lowering import lower_stage_module

    class Model(nn.Module):
        def __init__(self, vocab=300, d=128, h=2, L=4, seq=48):
            super().__init__()
            self.emb = nn.Embedding(vocab, d)
            self.layers = nn.ModuleList([nn.TransformerEncoderLayer(d, h, 2 * d, dropout=0.0, batch_first=True,
                                                                    norm_first=True) for _ in range(L)])
            self.head = nn.Linear(d, vocab, bias=False)
            mask = torch.triu(torch.ones(seq, seq, dtype=torch.bool), 1) if boolean else \
                nn.Transformer.generate_square_subsequent_mask(seq)
            self.register_buffer("mask", mask, persistent=False)

        def forward(self, ids):
            x = self.emb(ids)
            for layer in self.layers:
                x = layer(x, src_mask=self.mask, is_causal=True) if flag else layer(x, src_mask=self.mask)
            return self.head(x)

    torch.manual_seed(0)
    model = Model()
    ids = torch.randint(0, 300, (2, 48))
    pipe = pp.pipeline(model, 1, (ids,), split_spec={"layers.2": pp.SplitPoint.BEGINNING})
    torch.testing.assert_close(pipe(ids), model(ids), rtol=0, atol=0)
    x = ids
    for i in range(2):
        why = []
        blocks = lower_stage_module(pipe.get_stage_module(i), why)
        assert blocks is not None, why
        layers = [b for b in blocks if type(b).__name__ == "WrappedTransformerLayer"]
        assert len(layers) == 2 and all(b.causal for b in layers)
        with torch.no_grad():
            for b in blocks:
                x = b(x)
    torch.testing.assert_close(x, model(ids), rtol=1e-4, atol=1e-4)
    # a mask that is not causal keeps the stage with torch
    model.mask = torch.zeros(48, 48).fill_diagonal_(float("-inf"))
    pipe = pp.pipeline(model, 1, (ids,), split_spec={"layers.2": pp.SplitPoint.BEGINNING})
    why = []
    assert lower_stage_module(pipe.get_stage_module(1), why) is None and "not a constant causal mask" in why[0]
