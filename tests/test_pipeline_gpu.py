"""End-to-end parity of the pipeline (split -> staged forward/backward -> accumulate -> merge) on
the GPU against the fp32 CPU oracle, through the reference's own API surface."""
import copy
import math

import pytest
import torch

from _util import BF16_TOL, F32_TOL, assert_close_rel, check_gradients, max_rel
from oracle import ops as OO
from oracle import pipeline as OP

pytestmark = pytest.mark.gpu
DEV = "cuda"


def note(msg):
    print(msg, flush=True)


def _fp32_cpu_copy(model):
    ref = copy.deepcopy(model).float().cpu()
    return ref


def _build_decoder(n_stages, n_layers=4, M=4, vocab=1000, seq=128, dim=128, heads=2, ffn=512, seed=0,
                   fused=False, group=None):
    import pippy_amd as pp
    from pippy_amd.configs import DecoderLM, equal_split_spec
    torch.manual_seed(seed)
    model = DecoderLM(vocab=vocab, max_seq=seq, dim=dim, n_layers=n_layers, n_heads=heads, ffn=ffn)
    ref = _fp32_cpu_copy(model)
    ids = torch.randint(0, vocab, (2 * M, seq))
    pipe = pp.pipeline(model, M, (ids,), split_spec=equal_split_spec(n_layers, n_stages))
    assert pipe.num_stages == n_stages
    stages = [pp.PipelineStage(pipe, i, DEV, group=group, fused_accumulate=fused) for i in range(n_stages)]
    ref_stages = []
    keys = list(ref.state_dict().keys())
    # stage s of the oracle = the same children of the fp32 copy
    import torch.nn as nn
    per = n_layers // n_stages
    for s in range(n_stages):
        mods = []
        if s == 0:
            mods.append(ref.embed)
        mods += [ref.h[i] for i in range(per * s, per * (s + 1))]
        if s == n_stages - 1:
            mods.append(ref.head)
        ref_stages.append(nn.Sequential(*mods))
    return model, ref, stages, ref_stages, ids


def _ce(out, tgt):
    return torch.nn.functional.cross_entropy(out.reshape(-1, out.shape[-1]), tgt.reshape(-1))


def _check_against_oracle(model, ref, stages, ref_stages, ids, schedule_cls, M, steps=1):
    import pippy_amd as pp
    vocab = model.head.vocab
    torch.manual_seed(123)
    target = torch.randint(0, vocab, ids.shape)
    sched = schedule_cls(stages, M, loss_fn=pp.CrossEntropyLoss())
    for step in range(steps):
        losses = []
        out = sched.step(ids.to(DEV), target=target.to(DEV), losses=losses)
        torch.cuda.synchronize()
    for p in ref.parameters():
        p.grad = None
    ref_out, ref_losses = None, None
    for step in range(steps):
        ref_out, ref_losses = OP.step(ref_stages, ids, target, M, _ce)
    assert out.shape == ref_out.shape and out.is_contiguous()
    assert_close_rel(out, ref_out, BF16_TOL, "merged logits")
    assert len(losses) == M
    for m in range(M):
        assert_close_rel(losses[m].reshape(1), ref_losses[m].reshape(1), BF16_TOL, f"loss {m}")
    named = dict(model.named_parameters())
    worst = 0.0
    for name, rp in ref.named_parameters():
        g = named[name].main_grad
        err = max_rel(g, rp.grad)
        worst = max(worst, err)
        assert err <= BF16_TOL, f"grad of {name}: max relative error {err:.3e}"
    note(f"{schedule_cls.__name__}: worst grad error {worst:.3e}")
    return out, losses, {n: named[n].main_grad.clone() for n in named}


@pytest.mark.parametrize("n_stages", [1, 2, 4])
def test_decoder_gpipe_matches_oracle(n_stages):
    import pippy_amd as pp
    M = 4
    model, ref, stages, ref_stages, ids = _build_decoder(n_stages, M=M)
    _check_against_oracle(model, ref, stages, ref_stages, ids, pp.ScheduleGPipe, M)


def test_schedules_agree_bitwise_and_match_oracle():
    """Per stage, forward and backward run in ascending microbatch order in every schedule, so
    all results are identical across schedules, embedding gradients included (their row sums are
    formed in ascending token order, without atomics)."""
    import pippy_amd as pp
    M = 4
    results = {}
    for name, cls, group in (("gpipe", pp.ScheduleGPipe, None), ("1f1b", pp.Schedule1F1B, None),
                             ("bfs", pp.ScheduleLoopedBFS, 2), ("interleaved", pp.ScheduleInterleaved1F1B, 2),
                             ("interleaved_g1", pp.ScheduleInterleaved1F1B, 1),
                             ("zero_bubble", pp.ScheduleZeroBubble, None)):
        model, ref, stages, ref_stages, ids = _build_decoder(4, M=M, group=group)
        note(f"schedule {name}")
        results[name] = _check_against_oracle(model, ref, stages, ref_stages, ids, cls, M)
    base_out, base_losses, base_grads = results["gpipe"]
    for name, (out, losses, grads) in results.items():
        assert torch.equal(out, base_out), f"{name}: merged output differs from GPipe"
        for a, b in zip(losses, base_losses):
            assert torch.equal(a, b), f"{name}: loss differs from GPipe"
        for k in grads:
            assert torch.equal(grads[k], base_grads[k]), f"{name}: grad of {k} differs from GPipe"


def test_gpt2_small_full_size_schedules_and_repeats_agree_bit_for_bit():
    """The headline configuration at full size (12 layers of width 768, vocabulary 50257, 32 x 1024
    tokens in 8 microbatches, 4 virtual stages on two streams): 1F1B twice and GPipe once must give
    the same logits, losses and (sampled) gradient accumulators bit for bit, and the loss of a
    uniform guess at initialisation.  Races between the stage streams or schedule-dependent
    accumulation order would show here."""
    import pippy_amd as pp
    from pippy_amd.configs import DecoderLM, equal_split_spec
    torch.manual_seed(0)
    M = 8
    with torch.device(DEV):
        model = DecoderLM(vocab=50257, max_seq=1024, dim=768, n_layers=12, n_heads=12, ffn=3072)
    ids = torch.randint(0, 50257, (32, 1024), device=DEV)
    target = torch.randint(0, 50257, (32, 1024), device=DEV)
    pipe = pp.pipeline(model, M, (ids,), split_spec=equal_split_spec(12, 4))
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(4)]
    assert all(st.is_native for st in stages)
    named = dict(model.named_parameters())
    probe = ["h.0.attn.c_attn.weight", "h.5.mlp.c_proj.weight", "h.11.ln_2.weight", "h.7.attn.c_proj.bias",
             "h.3.mlp.c_fc.weight", "h.9.ln_1.bias"] + [n for n in named if n.startswith("head.")]
    assert all(n in named for n in probe) and len(probe) >= 7
    results = []
    for cls in (pp.Schedule1F1B, pp.ScheduleGPipe, pp.Schedule1F1B):
        sched = cls(stages, M, loss_fn=pp.CrossEntropyLoss())
        sched.zero_grad()
        losses = []
        out = sched.step(ids, target=target, losses=losses)
        results.append((out, torch.stack(losses).clone(), [named[n].main_grad.clone() for n in probe]))
    base = results[0]
    assert torch.isfinite(base[0].float()).all() and abs(float(base[1][0]) - math.log(50257)) < 0.3
    for out, losses, grads in results[1:]:
        assert torch.equal(out, base[0]) and torch.equal(losses, base[1])
        for n, a, b in zip(probe, grads, base[2]):
            assert float(a.abs().max()) > 0 and torch.equal(a, b), f"grad of {n}"


def test_two_steps_accumulate_then_zero_grad():
    """Gradients keep accumulating across steps until zero_grad, as with autograd's .grad
    (reference test_grad.py:78-82 runs two steps with zero_grad in between)."""
    import pippy_amd as pp
    M = 4
    model, ref, stages, ref_stages, ids = _build_decoder(2, M=M)
    _check_against_oracle(model, ref, stages, ref_stages, ids, pp.Schedule1F1B, M, steps=2)
    sched = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
    sched.zero_grad()
    _check_against_oracle(model, ref, stages, ref_stages, ids, pp.Schedule1F1B, M, steps=1)


def test_fused_accumulate_matches_oracle():
    import pippy_amd as pp
    M = 4
    model, ref, stages, ref_stages, ids = _build_decoder(2, M=M, fused=True)
    _check_against_oracle(model, ref, stages, ref_stages, ids, pp.Schedule1F1B, M)


def test_epilogue_accumulation_leaves_the_bits_of_the_staged_form():
    """The default adds each weight gradient, rounded to bf16, to the fp32 accumulator in the
    epilogue of its GEMM; ``fused_accumulate="staged"`` writes every gradient to the staging arena
    in bf16 and folds the arena in with the accumulate kernel (``acc += float(g)``).  Both must
    leave the same bits after two steps of four microbatches."""
    import pippy_amd as pp
    M = 4
    grads = {}
    for mode in (False, "staged"):
        model, ref, stages, ref_stages, ids = _build_decoder(2, M=M, fused=mode)
        _, _, grads[mode] = _check_against_oracle(model, ref, stages, ref_stages, ids, pp.Schedule1F1B, M, steps=2)
        n_accum = [sum(1 for k in range(st._program.mbs[0].W.n)
                       if st._program.mbs[0].W[k].kind in (pp._native.OP_ACCUM_BF16, pp._native.OP_ACCUM_F32))
                   for st in stages]
        note(f"fused_accumulate={mode!r}: accumulate launches per weight-gradient pass {n_accum}")
        assert all(n == 1 for n in n_accum)
    for k in grads[False]:
        assert torch.equal(grads[False][k], grads["staged"][k]), f"grad of {k}"


def test_inference_gpipe_forward_only():
    import pippy_amd as pp
    M = 4
    model, ref, stages, ref_stages, ids = _build_decoder(2, M=M)
    sched = pp.ScheduleGPipe(stages, M)
    out = sched.step(ids.to(DEV))
    ref_out, _ = OP.step(ref_stages, ids, None, M, None)
    assert_close_rel(out, ref_out, BF16_TOL, "inference logits")


def test_generic_loss_fn_bridge():
    """Any callable works as loss_fn: it runs under autograd on the last stage's output."""
    import pippy_amd as pp
    M = 2
    model, ref, stages, ref_stages, ids = _build_decoder(2, M=M)
    target = torch.randint(0, 1000, ids.shape)
    sched = pp.ScheduleGPipe(stages, M, loss_fn=lambda o, t: _ce(o.float(), t))
    losses = []
    sched.step(ids.to(DEV), target=target.to(DEV), losses=losses)
    for p in ref.parameters():
        p.grad = None
    _, ref_losses = OP.step(ref_stages, ids, target, M, _ce)
    named = dict(model.named_parameters())
    for name, rp in ref.named_parameters():
        assert_close_rel(named[name].main_grad, rp.grad, BF16_TOL, name)
    for a, b in zip(losses, ref_losses):
        assert_close_rel(a.reshape(1), b.reshape(1), BF16_TOL, "loss")


def test_readme_mlp_fp32_matches_oracle():
    """Configuration 1: the README MLP (examples/basic/example_train.py:9-45 of the reference),
    fp32, 2 stages split at layer1, GPipe over 4 microbatches of 64, cross entropy."""
    import torch.nn as nn
    import pippy_amd as pp

    class MyNetworkBlock(nn.Module):
        def __init__(self, i, o):
            super().__init__()
            self.lin = nn.Linear(i, o)

        def forward(self, x):
            return torch.relu(self.lin(x))

    class MyNetwork(nn.Module):
        def __init__(self):
            super().__init__()
            dims = [512, 1024, 256]
            prev = 512
            self.num_layers = len(dims)
            for i, d in enumerate(dims):
                self.add_module(f"layer{i}", MyNetworkBlock(prev, d))
                prev = d
            self.output_proj = nn.Linear(prev, 10)

        def forward(self, x):
            for i in range(self.num_layers):
                x = getattr(self, f"layer{i}")(x)
            return self.output_proj(x)

    torch.manual_seed(0)
    model = MyNetwork()
    ref = copy.deepcopy(model)
    # ReLU is discontinuous: a pre-activation within rounding distance of zero can get a different
    # mask on the GPU than in the oracle (different fp32 summation order), and one flipped mask
    # moves a whole gradient row.  Draw inputs until the oracle's smallest |pre-activation| is far
    # (2e-6, about ten times the fp32 rounding error of these dot products) from zero.
    for data_seed in range(1000):
        g = torch.Generator().manual_seed(data_seed)
        x = torch.randn(256, 512, generator=g)
        with torch.no_grad():
            h, margin = x, float("inf")
            for i in range(3):
                a = getattr(ref, f"layer{i}").lin(h)
                margin = min(margin, a.abs().min().item())
                h = torch.relu(a)
        if margin > 2e-6:
            break
    else:
        raise AssertionError("no input draw keeps ReLU pre-activations away from zero")
    note(f"mlp data seed {data_seed}, smallest |pre-activation| {margin:.2e}")
    y = torch.randint(0, 10, (256,), generator=g)
    M = 4
    pipe = pp.pipeline(model, M, (x,), split_spec={"layer1": pp.SplitPoint.BEGINNING})
    assert pipe.num_stages == 2
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
    assert all(s.is_native for s in stages)
    sched = pp.ScheduleGPipe(stages, M, loss_fn=nn.CrossEntropyLoss())
    losses = []
    out = sched.step(x.to(DEV), target=y.to(DEV), losses=losses)
    ref_stages = [nn.Sequential(ref.layer0), nn.Sequential(ref.layer1, ref.layer2, ref.output_proj)]
    ref_out, ref_losses = OP.step(ref_stages, x, y, M, nn.functional.cross_entropy)
    assert_close_rel(out, ref_out, F32_TOL, "mlp output")
    for a, b in zip(losses, ref_losses):
        assert_close_rel(a.reshape(1), b.reshape(1), F32_TOL, "mlp loss")
    named = dict(model.named_parameters())
    for name, rp in ref.named_parameters():
        assert_close_rel(named[name].grad, rp.grad, F32_TOL, f"mlp grad {name}")
        assert named[name].grad.data_ptr() == named[name].main_grad.data_ptr()


def test_fused_optimizer_trains_like_the_oracle():
    """schedule.step() + optimizer.step() twice (reference test_optim.py:83-99): parameter updates,
    the momentum-carrying second update and the losses of the second step (which run on the updated
    weights and their refreshed transposed copies) against the oracle pipeline stepped with the
    oracle's SGD."""
    import pippy_amd as pp
    from oracle import optim as OO
    M = 4
    model, ref, stages, ref_stages, ids = _build_decoder(2, M=M)
    torch.manual_seed(7)
    target = torch.randint(0, model.head.vocab, ids.shape)
    sched = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
    lr, mom = 1.0, 0.9
    opt = pp.FusedSGD(stages, lr=lr, momentum=mom, master_weights=True)
    named = dict(model.named_parameters())
    ref_named = dict(ref.named_parameters())
    arenas = [st.param_arena() for st in stages]

    def master_of(name):
        """fp32 master copy of one parameter (a slice of its stage's flat master array)."""
        k = next(i for i, a in enumerate(arenas) if id(named[name]) in a.entries)
        return arenas[k]._slice(opt.master_weights[k], named[name], padded=False).detach().cpu().clone()

    bufs = {}
    prev = {n: master_of(n) for n in named}
    for step in range(2):
        opt.zero_grad()
        losses = []
        sched.step(ids.to(DEV), target=target.to(DEV), losses=losses)
        opt.step()
        torch.cuda.synchronize()
        for p in ref.parameters():
            p.grad = None
        _, ref_losses = OP.step(ref_stages, ids, target, M, _ce)
        for m in range(M):
            assert_close_rel(losses[m].reshape(1), ref_losses[m].reshape(1), BF16_TOL, f"step {step} loss {m}")
        worst = 0.0
        for name, rp in ref_named.items():
            new, bufs[name] = OO.sgd_step(rp.detach().numpy(), rp.grad.numpy(), bufs.get(name), lr=lr,
                                          momentum=mom, first_step=step == 0)
            ref_update = torch.from_numpy(new) - rp.detach()
            with torch.no_grad():
                rp.copy_(torch.from_numpy(new))
            cur = master_of(name)
            err = max_rel(cur - prev[name], ref_update)
            worst = max(worst, err)
            assert err <= BF16_TOL, f"step {step} update of {name}: max relative error {err:.3e}"
            # the bf16 parameter is the rounding of its master copy
            assert torch.equal(named[name].detach().cpu(), cur.to(torch.bfloat16))
            prev[name] = cur
        note(f"optimizer step {step}: worst update error {worst:.3e}")


def test_stock_optimizer_zero_grad_restarts_the_accumulation_on_bf16_stages():
    """The loop of the reference's test_optim.py:85-99 with a torch optimizer on bf16 stages:
    ``materialize_grads`` hands the fp32 sums over as ``param.grad``, ``optimizer.zero_grad()`` clears
    them, and the next step must start a new accumulation.  With a zero learning rate both steps see
    the same weights, so the sums after the second step equal those after the first bit for bit
    (a stage that kept adding would hold twice the values)."""
    import pippy_amd as pp
    M = 4
    model, ref, stages, ref_stages, ids = _build_decoder(2, M=M)
    torch.manual_seed(11)
    target = torch.randint(0, model.head.vocab, ids.shape)
    sched = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
    params = [p for st in stages for p in st.submod.parameters()]
    opt = torch.optim.SGD(params, lr=0.0)
    named = dict(model.named_parameters())
    embed = {n for n in named if "wte" in n or "wpe" in n}
    first = None
    for step in range(2):
        sched.step(ids.to(DEV), target=target.to(DEV), losses=[])
        for st in stages:
            st.materialize_grads()
        torch.cuda.synchronize()
        for n, p in named.items():
            assert p.grad is not None and p.grad.dtype == p.dtype
            assert torch.equal(p.grad, p.main_grad.to(p.dtype)), n
        sums = {n: p.main_grad.clone() for n, p in named.items()}
        if first is None:
            first = sums
        opt.step()
        opt.zero_grad()
        assert all(p.grad is None for p in params)
    for n in named:
        assert torch.equal(sums[n], first[n]), f"{n}: the second step did not restart the accumulation"
    # against the oracle: one step's gradients
    for p in ref.parameters():
        p.grad = None
    OP.step(ref_stages, ids, target, M, _ce)
    for n, rp in ref.named_parameters():
        assert_close_rel(sums[n], rp.grad, BF16_TOL, f"grad of {n}")
    del embed


def test_fused_optimizer_skips_a_stage_whose_gradients_were_cleared():
    """``zero_grad`` followed by ``step`` without a backward pass in between leaves the parameters
    alone (torch.optim skips parameters without a gradient); the accumulators of the step before are
    not applied a second time."""
    import pippy_amd as pp
    M = 4
    model, ref, stages, ref_stages, ids = _build_decoder(2, M=M)
    torch.manual_seed(3)
    target = torch.randint(0, model.head.vocab, ids.shape)
    sched = pp.ScheduleGPipe(stages, M, loss_fn=pp.CrossEntropyLoss())
    opt = pp.FusedSGD(stages, lr=0.5)
    sched.step(ids.to(DEV), target=target.to(DEV), losses=[])
    opt.step()
    torch.cuda.synchronize()
    after_one = {n: p.detach().clone() for n, p in model.named_parameters()}
    opt.zero_grad()
    opt.step()
    torch.cuda.synchronize()
    for n, p in model.named_parameters():
        assert torch.equal(p.detach(), after_one[n]), n


# ---- BERT-shaped encoder (post-LayerNorm, bidirectional attention, erf-GELU) ----------------------
def _build_encoder(n_stages, n_layers=4, M=4, vocab=1000, seq=128, dim=128, heads=2, ffn=512, seed=0):
    import pippy_amd as pp
    import torch.nn as nn
    from pippy_amd.configs import EncoderModel, equal_split_spec
    torch.manual_seed(seed)
    model = EncoderModel(vocab=vocab, max_seq=seq, dim=dim, n_layers=n_layers, n_heads=heads, ffn=ffn)
    # LayerNorm weights away from their (1, 0) initial values, so that their gradients are exercised
    with torch.no_grad():
        for m in model.modules():
            if isinstance(m, nn.LayerNorm):
                m.weight.add_(0.1 * torch.randn_like(m.weight))
                m.bias.add_(0.1 * torch.randn_like(m.bias))
    ref = _fp32_cpu_copy(model)
    ids = torch.randint(0, vocab, (2 * M, seq))
    pipe = pp.pipeline(model, M, (ids,), split_spec=equal_split_spec(n_layers, n_stages))
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(n_stages)]
    per = n_layers // n_stages
    ref_stages = []
    for s in range(n_stages):
        mods = [ref.embed] if s == 0 else []
        mods += [ref.h[i] for i in range(per * s, per * (s + 1))]
        ref_stages.append(nn.Sequential(*mods))
    return model, ref, stages, ref_stages, ids


def test_encoder_inference_gpipe_matches_oracle():
    """Config 2 at a reduced size: GPipe fill-drain forward of a post-LayerNorm encoder in 4 stages."""
    import pippy_amd as pp
    M = 4
    model, ref, stages, ref_stages, ids = _build_encoder(4, M=M)
    assert all(st.is_native for st in stages)
    out = pp.ScheduleGPipe(stages, M).step(ids.to(DEV))
    ref_out, _ = OP.step(ref_stages, ids, None, M, None)
    assert out.shape == ref_out.shape == (2 * M, 128, 128)
    assert_close_rel(out, ref_out, BF16_TOL, "encoder hidden states")


def test_encoder_training_post_layernorm_matches_oracle():
    """Post-LayerNorm layers and the three-table embedding through forward, dI and dW passes."""
    import pippy_amd as pp
    M = 2
    model, ref, stages, ref_stages, ids = _build_encoder(2, n_layers=2, M=M)
    torch.manual_seed(5)
    target = torch.randn(2 * M, 128, 128)

    def loss_fn(o, t):
        return ((o.float() - t) ** 2).sum() * 1e-2

    sched = pp.Schedule1F1B(stages, M, loss_fn=loss_fn)
    losses = []
    sched.step(ids.to(DEV), target=target.to(DEV), losses=losses)
    for p in ref.parameters():
        p.grad = None
    _, ref_losses = OP.step(ref_stages, ids, target, M, loss_fn)
    for a, b in zip(losses, ref_losses):
        assert_close_rel(a.reshape(1), b.reshape(1), BF16_TOL, "loss")
    named = dict(model.named_parameters())
    worst = 0.0
    for name, rp in ref.named_parameters():
        err = max_rel(named[name].main_grad, rp.grad)
        worst = max(worst, err)
        assert err <= BF16_TOL, f"grad of {name}: max relative error {err:.3e}"
    note(f"post-LN encoder: worst grad error {worst:.3e}")


def test_encoder_bert_base_full_size_layernorm_invariant():
    """Config 2 at full size (12 layers, hidden 768, seq 512, batch 64 in 8 microbatches, 4 stages):
    the last op of a post-LayerNorm encoder is a LayerNorm with weight 1 and bias 0 at
    initialisation, so every output row has mean 0 and variance 1 whatever came before."""
    import pippy_amd as pp
    from pippy_amd.configs import bert_base, equal_split_spec
    torch.manual_seed(0)
    model = bert_base()
    M = 8
    ids = torch.randint(0, 30522, (64, 512))
    pipe = pp.pipeline(model, M, (ids,), split_spec=equal_split_spec(12, 4))
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(4)]
    out = pp.ScheduleGPipe(stages, M).step(ids.to(DEV))
    assert out.shape == (64, 512, 768) and out.is_contiguous()
    o = out.float()
    assert torch.isfinite(o).all()
    assert o.mean(-1).abs().max() < 2e-2
    assert (o.var(-1, unbiased=False) - 1).abs().max() < 3e-2


# ---- Llama-style stage (RMSNorm, rotary embedding, head dimension 128, SwiGLU), zero-bubble -------
def _upstream_loss(out, upstream):
    """A loss whose gradient w.r.t. the stage output is `upstream`: what a middle stage receives."""
    return (out.float() * upstream).sum()


def _llama_grads_match(model, ref, losses, ref_losses, ref_out, upstream):
    # the "loss" is a sum of terms of both signs: its error is measured against the sum of their
    # magnitudes, not against the (cancelled) result
    M = len(losses)
    for m, (a, b) in enumerate(zip(losses, ref_losses)):
        scale = (ref_out.chunk(M)[m].abs() * upstream.chunk(M)[m].abs()).sum()
        assert abs(float(a.detach()) - float(b.detach())) <= BF16_TOL * float(scale), f"loss {m} differs"
    named = dict(model.named_parameters())
    worst = 0.0
    for name, rp in ref.named_parameters():
        err = max_rel(named[name].main_grad, rp.grad)
        worst = max(worst, err)
        assert err <= BF16_TOL, f"grad of {name}: max relative error {err:.3e}"
    return worst


def test_llama_stage_zero_bubble_matches_oracle():
    """Config 4 at a reduced size: one hand-built stage of Llama-style layers (ManualPipelineStage),
    microbatches of one sequence, upstream gradients N(0, 1e-2), separate dI and dW passes."""
    import pippy_amd as pp
    from pippy_amd.configs import LlamaStage
    torch.manual_seed(0)
    M, S, dim = 4, 256, 256
    model = LlamaStage(n_layers=2, dim=dim, n_heads=2, ffn=640)
    with torch.no_grad():
        for m in model.modules():
            if isinstance(m, torch.nn.RMSNorm):
                m.weight.add_(0.1 * torch.randn_like(m.weight))
    ref = _fp32_cpu_copy(model)
    x = torch.randn(M, S, dim).to(torch.bfloat16)
    upstream = torch.randn(M, S, dim) * 1e-2
    stage = pp.ManualPipelineStage(model, 0, 1, DEV, M, input_args=(x[:1].to(DEV),))
    assert stage.is_native
    sched = pp.ScheduleZeroBubble([stage], M, loss_fn=_upstream_loss)
    losses = []
    out = sched.step(x.to(DEV), target=upstream.to(DEV), losses=losses)
    for p in ref.parameters():
        p.grad = None
    ref_out, ref_losses = OP.step([ref], x.float(), upstream, M, _upstream_loss)
    assert_close_rel(out, ref_out, BF16_TOL, "stage output")
    worst = _llama_grads_match(model, ref, losses, ref_losses, ref_out, upstream)
    note(f"Llama stage, zero-bubble: worst grad error {worst:.3e}")


def test_llama_fused_feed_forward_follows_parameter_updates_and_launches_fused_kernels():
    """The feed-forward of a bf16 Llama layer runs as GEMMs with SwiGLU in their epilogues (no separate
    element-wise launch), and the side-by-side transposed gate / up weights that its input-gradient GEMM
    reads are refreshed after the parameters change."""
    import pippy_amd as pp
    from pippy_amd import _native as N
    from pippy_amd.configs import LlamaStage
    torch.manual_seed(5)
    M, S, dim = 2, 128, 128
    model = LlamaStage(n_layers=1, dim=dim, n_heads=2, ffn=328)   # 328: tiles with a ragged last column block
    ref = _fp32_cpu_copy(model)
    x = torch.randn(M, S, dim).to(torch.bfloat16)
    upstream = torch.randn(M, S, dim) * 1e-2
    stage = pp.ManualPipelineStage(model, 0, 1, DEV, M, input_args=(x[:1].to(DEV),))
    sched = pp.ScheduleZeroBubble([stage], M, loss_fn=_upstream_loss)
    sched.step(x.to(DEV), target=upstream.to(DEV))
    prog = stage._program.mbs[0]
    kinds_f = [op.kind for op in prog.F.ops]
    kinds_i = [op.kind for op in prog.I.ops]
    assert N.OP_GEMM_SWIGLU in kinds_f and N.OP_SWIGLU_FWD not in kinds_f
    assert N.OP_GEMM_DSWIGLU in kinds_i and N.OP_SWIGLU_BWD not in kinds_i
    torch.manual_seed(6)
    with torch.no_grad():
        for (n, p), (_, rp) in zip(model.named_parameters(), ref.named_parameters()):
            p.add_((torch.randn(rp.shape) * 0.02).to(torch.bfloat16).to(DEV))
            rp.copy_(p.detach().float().cpu())
    sched.zero_grad()
    losses = []
    out = sched.step(x.to(DEV), target=upstream.to(DEV), losses=losses)
    ref_out, ref_losses = OP.step([ref], x.float(), upstream, M, _upstream_loss)
    assert_close_rel(out, ref_out, BF16_TOL, "stage output after the update")
    _llama_grads_match(model, ref, losses, ref_losses, ref_out, upstream)


@pytest.mark.parametrize("n_heads,n_kv_heads,dim", [(4, 2, 256), (4, 1, 256), (2, 1, 256)])
def test_llama_grouped_query_attention_two_stages_matches_oracle(n_heads, n_kv_heads, dim):
    """Llama-style layers whose query heads share key / value heads (head dimension 64 and 128), split
    into two traced stages under 1F1B: the fused projection is narrower (q | k | v = H, Hkv, Hkv heads),
    the rotary embedding covers H + Hkv heads, and a key / value head's gradient sums over its group."""
    import pippy_amd as pp
    import torch.nn as nn
    from pippy_amd.configs import LlamaStage
    torch.manual_seed(2)
    M, S = 2, 128
    model = LlamaStage(n_layers=2, dim=dim, n_heads=n_heads, ffn=256, n_kv_heads=n_kv_heads)
    assert model.layers[0].self_attn.qkv_proj.weight.shape[0] == (n_heads + 2 * n_kv_heads) * (dim // n_heads)
    ref = _fp32_cpu_copy(model)
    x = torch.randn(2 * M, S, dim).to(torch.bfloat16)
    upstream = torch.randn(2 * M, S, dim) * 1e-2
    pipe = pp.pipeline(model, M, (x,), split_spec={"layers.1": pp.SplitPoint.BEGINNING})
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
    assert all(st.is_native for st in stages)
    sched = pp.Schedule1F1B(stages, M, loss_fn=_upstream_loss)
    losses = []
    out = sched.step(x.to(DEV), target=upstream.to(DEV), losses=losses)
    ref_stages = [nn.Sequential(ref.layers[0]), nn.Sequential(ref.layers[1])]
    ref_out, ref_losses = OP.step(ref_stages, x.float(), upstream, M, _upstream_loss)
    assert_close_rel(out, ref_out, BF16_TOL, "stage output")
    worst = _llama_grads_match(model, ref, losses, ref_losses, ref_out, upstream)
    note(f"Llama layers with {n_heads} query / {n_kv_heads} key-value heads: worst grad error {worst:.3e}")


def test_llama_two_stages_1f1b_hand_off_matches_oracle():
    """The same layers split into two traced stages: the input gradient of the second stage (through
    RMSNorm, rotary embedding and attention backward) feeds the first."""
    import pippy_amd as pp
    import torch.nn as nn
    from pippy_amd.configs import LlamaStage
    torch.manual_seed(1)
    M, S, dim = 2, 128, 128
    model = LlamaStage(n_layers=2, dim=dim, n_heads=2, ffn=256)   # head dimension 64
    ref = _fp32_cpu_copy(model)
    x = torch.randn(2 * M, S, dim).to(torch.bfloat16)
    upstream = torch.randn(2 * M, S, dim) * 1e-2
    pipe = pp.pipeline(model, M, (x,), split_spec={"layers.1": pp.SplitPoint.BEGINNING})
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
    assert all(st.is_native for st in stages)
    sched = pp.Schedule1F1B(stages, M, loss_fn=_upstream_loss)
    losses = []
    out = sched.step(x.to(DEV), target=upstream.to(DEV), losses=losses)
    for p in ref.parameters():
        p.grad = None
    ref_stages = [nn.Sequential(ref.layers[0]), nn.Sequential(ref.layers[1])]
    ref_out, ref_losses = OP.step(ref_stages, x.float(), upstream, M, _upstream_loss)
    assert_close_rel(out, ref_out, BF16_TOL, "stage output")
    worst = _llama_grads_match(model, ref, losses, ref_losses, ref_out, upstream)
    note(f"Llama layers, two stages: worst grad error {worst:.3e}")


def test_split_backward_matches_the_library_split_of_autograd():
    """The separate input-gradient and weight-gradient passes against the library routines that split
    autograd the same way (torch.distributed.pipelining._backward.stage_backward_input /
    stage_backward_weight, run on an fp32 CPU copy of the same two stages): the gradient that stage 1
    hands to stage 0 for every microbatch, and the parameter gradients once the deferred weight
    passes have run."""
    import pippy_amd as pp
    import torch.nn as nn
    from torch.distributed.pipelining._backward import stage_backward_input, stage_backward_weight
    from pippy_amd.configs import LlamaStage
    torch.manual_seed(11)
    M, S, dim = 2, 128, 128
    model = LlamaStage(n_layers=2, dim=dim, n_heads=2, ffn=256)
    ref = _fp32_cpu_copy(model)
    x = torch.randn(2 * M, S, dim).to(torch.bfloat16)
    upstream = torch.randn(2 * M, S, dim) * 1e-2
    pipe = pp.pipeline(model, M, (x,), split_spec={"layers.1": pp.SplitPoint.BEGINNING})
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
    sched = pp.ScheduleZeroBubble(stages, M, loss_fn=_upstream_loss)
    sched.step(x.to(DEV), target=upstream.to(DEV))
    torch.cuda.synchronize()

    ref_stages = [nn.Sequential(ref.layers[0]), nn.Sequential(ref.layers[1])]
    for p in ref.parameters():
        p.grad = None
    handed_over, deferred = [], []
    for xm, um in zip(x.float().chunk(M), upstream.chunk(M)):
        xm = xm.clone().requires_grad_(True)
        h0 = ref_stages[0](xm)
        h1_in = h0.detach().requires_grad_(True)
        out = ref_stages[1](h1_in)
        loss = _upstream_loss(out, um)
        (d_h1,), groups1 = stage_backward_input([loss], None, [h1_in], ref_stages[1].parameters())
        assert all(p.grad is None for p in ref_stages[1].parameters()), "the input pass leaves the weights alone"
        _, groups0 = stage_backward_input([h0], [d_h1], [xm], ref_stages[0].parameters())
        handed_over.append(d_h1)
        deferred.append((groups0, groups1))
    for groups0, groups1 in deferred:   # the weight passes run later, in microbatch order
        stage_backward_weight(ref_stages[1].parameters(), groups1)
        stage_backward_weight(ref_stages[0].parameters(), groups0)

    for m in range(M):
        got = stages[1]._program.mbs[m].input_grad
        assert_close_rel(got.view(handed_over[m].shape), handed_over[m], BF16_TOL, f"input gradient of microbatch {m}")
    named = dict(model.named_parameters())
    for name, rp in ref.named_parameters():
        assert max_rel(named[name].main_grad, rp.grad) <= BF16_TOL, f"grad of {name}"


def test_llama2_7b_stage_full_size_schedule_and_scaling_invariants():
    """Config 4 at full size (8 layers, width 4096, 32 heads of 128, SwiGLU 11008, sequence 2048,
    16 microbatches of one sequence).  Two properties that hold at any size: the zero-bubble schedule
    (dI and dW as separate passes) accumulates bit-identical gradients to 1F1B, because each
    parameter receives its microbatch contributions in the same order; and the backward pass is
    linear in the upstream gradient, so doubling it (exact in binary floating point) doubles every
    accumulated gradient bit for bit."""
    import pippy_amd as pp
    from pippy_amd.configs import llama2_7b_stage
    torch.manual_seed(0)
    M = 16
    with torch.device(DEV):
        model = llama2_7b_stage()
        x = torch.randn(M, 2048, 4096).to(torch.bfloat16)
        upstream = torch.randn(M, 2048, 4096) * 1e-2
    stage = pp.ManualPipelineStage(model, 0, 1, DEV, M, input_args=(x[:1],))
    assert stage.is_native

    def grads_after(schedule_cls, up):
        sched = schedule_cls([stage], M, loss_fn=_upstream_loss)
        sched.zero_grad()
        out = sched.step(x, target=up)
        return out, [p.main_grad.clone() for p in model.layers[0].parameters()] + \
                    [p.main_grad.clone() for p in model.layers[7].parameters()]

    out_zb, g_zb = grads_after(pp.ScheduleZeroBubble, upstream)
    assert out_zb.shape == x.shape and torch.isfinite(out_zb.float()).all()
    assert all(torch.isfinite(g).all() and g.abs().max() > 0 for g in g_zb)
    out_1f1b, g_1f1b = grads_after(pp.Schedule1F1B, upstream)
    assert torch.equal(out_zb, out_1f1b)
    for a, b in zip(g_zb, g_1f1b):
        assert torch.equal(a, b)
    del g_1f1b
    _, g_2x = grads_after(pp.ScheduleZeroBubble, upstream * 2)
    for a, b in zip(g_zb, g_2x):
        assert torch.equal(a * 2, b)


def test_llama_last_stage_with_final_rmsnorm_and_head_matches_oracle():
    """The last stage of a Llama-style pipeline as a user would write it: decoder layers, the final
    ``nn.RMSNorm`` and a bias-free ``nn.Linear`` head as plain torch layers, cross-entropy loss."""
    import pippy_amd as pp
    import torch.nn as nn
    from pippy_amd.stage_modules import LlamaLayer
    torch.manual_seed(2)
    M, S, dim, vocab = 2, 128, 128, 384
    model = nn.Sequential(LlamaLayer(dim, 2, 256), nn.RMSNorm(dim, eps=1e-5, dtype=torch.bfloat16),
                          nn.Linear(dim, vocab, bias=False, dtype=torch.bfloat16))
    with torch.no_grad():
        model[1].weight.add_(0.1 * torch.randn_like(model[1].weight))
    ref = _fp32_cpu_copy(model)
    x = torch.randn(2 * M, S, dim).to(torch.bfloat16)
    target = torch.randint(0, vocab, (2 * M, S))
    stage = pp.ManualPipelineStage(model, 0, 1, DEV, M, input_args=(x[:2].to(DEV),))
    assert stage.is_native
    sched = pp.Schedule1F1B([stage], M, loss_fn=_ce)
    losses = []
    out = sched.step(x.to(DEV), target=target.to(DEV), losses=losses)
    ref_out, ref_losses = OP.step([ref], x.float(), target, M, _ce)
    assert_close_rel(out, ref_out, BF16_TOL, "logits")
    for a, b in zip(losses, ref_losses):
        assert_close_rel(a.detach().reshape(1), b.detach().reshape(1), BF16_TOL, "loss")
    named = dict(model.named_parameters())
    for name, rp in ref.named_parameters():
        err = max_rel(named[name].main_grad, rp.grad)
        assert err <= BF16_TOL, f"grad of {name}: max relative error {err:.3e}"


# ---- Mixtral-style mixture of experts under interleaved 1F1B (config 5) ---------------------------
def _moe_reference_stages(ref, n_stages, per):
    import torch.nn as nn
    out = []
    for s in range(n_stages):
        mods = [ref.embed] if s == 0 else []
        mods += [ref.h[i] for i in range(per * s, per * (s + 1))]
        if s == n_stages - 1:
            mods.append(ref.head)
        out.append(nn.Sequential(*mods))
    return out


@pytest.mark.parametrize("fused,E", [(False, 8), (True, 8), ("staged", 8), (False, 6), (False, 12), (True, 3)])
def test_moe_interleaved_1f1b_matches_oracle(fused, E):
    """Config 5 at a reduced size: two virtual stages of MoE layers on one rank under interleaved
    1F1B.  The fp32 oracle is given the expert selection of the bf16 run (a token whose second and
    third router logits nearly tie may legitimately flip under rounding); that the selection itself
    is the top-2 of the run's own logits is checked separately.  Expert counts that are not a multiple
    of 8 run with the router weight and the logits padded to one (zero rows / columns)."""
    import pippy_amd as pp
    from pippy_amd.configs import MoEDecoderLM, equal_split_spec
    torch.manual_seed(0 if E == 8 else E)
    M, S, vocab, L = 4, 128, 512, 4
    model = MoEDecoderLM(vocab=vocab, dim=128, n_layers=L, n_heads=2, ffn=256, n_experts=E)
    with torch.no_grad():
        for layer in model.h:
            layer.block_sparse_moe.gate.weight.mul_(10)     # decisive routing: few near-ties
    ref = _fp32_cpu_copy(model)
    ids = torch.randint(0, vocab, (2 * M, S))
    target = torch.randint(0, vocab, (2 * M, S))
    pipe = pp.pipeline(model, M, (ids,), split_spec=equal_split_spec(L, 2))
    stages = [pp.PipelineStage(pipe, i, DEV, group=1, fused_accumulate=fused) for i in range(2)]
    assert all(st.is_native for st in stages)
    sched = pp.ScheduleInterleaved1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
    losses = []
    out = sched.step(ids.to(DEV), target=target.to(DEV), losses=losses)
    torch.cuda.synchronize()
    # the run's own routing: top-2 of its router logits, every token placed once per slot
    routing = [[] for _ in range(L)]
    for s, st in enumerate(stages):
        for m in range(M):
            acts = st.saved_activations(m)
            idx = [v for k, v in acts.items() if k.endswith("topk_idx")]
            logits = [v for k, v in acts.items() if k.endswith("router_logits")]
            seg = [v for k, v in acts.items() if k.endswith("seg_start")]
            assert len(idx) == L // 2
            for j in range(L // 2):
                assert logits[j].shape[1] == (E + 7) // 8 * 8
                assert float(logits[j][:, E:].float().abs().sum()) == 0.0      # the padding columns
                want, _ = OO.moe_route_top2(logits[j][:, :E].float().cpu())
                assert torch.equal(idx[j].cpu().long(), want)
                assert int(seg[j][-1]) == 2 * 2 * S and int(seg[j][0]) == 0
                routing[s * (L // 2) + j].append(idx[j].cpu().long())
    for l in range(L):
        ref.h[l].forced_routing = list(routing[l])
    ref_out, ref_losses = OP.step(_moe_reference_stages(ref, 2, L // 2), ids, target, M, _ce)
    assert_close_rel(out, ref_out, BF16_TOL, "merged logits")
    for a, b in zip(losses, ref_losses):
        assert_close_rel(a.reshape(1), b.reshape(1), BF16_TOL, "loss")
    named = dict(model.named_parameters())
    worst = 0.0
    for name, rp in ref.named_parameters():
        err = max_rel(named[name].main_grad, rp.grad)
        worst = max(worst, err)
        assert err <= BF16_TOL, f"grad of {name}: max relative error {err:.3e}"
    note(f"MoE interleaved 1F1B (fused accumulate {fused}): worst grad error {worst:.3e}")


def test_moe_mixtral_style_full_size_routing_and_schedule_invariants():
    """Config 5 at full size (2 virtual stages of 4 layers, width 1024, 16 heads, 8 experts with
    SwiGLU 4096, top-2, sequence 1024, batch 16 in 8 microbatches, vocabulary 32000).  Properties
    that hold at any size: every (token, slot) pair lands in exactly one expert row, the two experts
    of a token differ, the routing weights of a token sum to one, the expert row ranges tile
    [0, 2 * tokens); and interleaved 1F1B gives bit-identical losses and gradients to GPipe."""
    import pippy_amd as pp
    from pippy_amd.configs import mixtral_style, equal_split_spec
    torch.manual_seed(0)
    M = 8
    with torch.device(DEV):
        model = mixtral_style()
    ids = torch.randint(0, 32000, (16, 1024), device=DEV)
    target = torch.randint(0, 32000, (16, 1024), device=DEV)
    pipe = pp.pipeline(model, M, (ids,), split_spec=equal_split_spec(8, 2))
    stages = [pp.PipelineStage(pipe, i, DEV, group=1) for i in range(2)]
    assert all(st.is_native for st in stages)
    probe = [model.h[0].block_sparse_moe.experts[3].w1.weight, model.h[7].block_sparse_moe.experts[0].w2.weight,
             model.h[4].block_sparse_moe.gate.weight, model.h[2].self_attn.qkv_proj.weight,
             model.h[5].post_attention_layernorm.weight]
    results = []
    for cls in (pp.ScheduleInterleaved1F1B, pp.ScheduleGPipe):
        sched = cls(stages, M, loss_fn=pp.CrossEntropyLoss())
        sched.zero_grad()
        losses = []
        out = sched.step(ids, target=target, losses=losses)
        results.append((out, [l.clone() for l in losses], [p.main_grad.clone() for p in probe]))
        if cls is pp.ScheduleInterleaved1F1B:
            T = 2 * 1024
            for st in stages:
                for m in (0, M - 1):
                    acts = st.saved_activations(m)
                    for key in [k for k in acts if k.endswith("topk_idx")]:
                        pre = key[:-len("topk_idx")]
                        idx, gate = acts[key], acts[pre + "gate"]
                        seg, row_src, pos = acts[pre + "seg_start"], acts[pre + "row_src"], acts[pre + "pos"]
                        assert bool((idx[:, 0] != idx[:, 1]).all()) and int(idx.min()) >= 0 and int(idx.max()) < 8
                        assert float((gate.sum(-1) - 1).abs().max()) <= 1e-6
                        assert int(seg[0]) == 0 and int(seg[-1]) == 2 * T and bool((seg[1:] >= seg[:-1]).all())
                        assert torch.equal(torch.sort(pos).values.long(), torch.arange(2 * T, device=DEV))
                        assert torch.equal(row_src.long()[pos.long()], torch.arange(2 * T, device=DEV))
                        # rows of expert e hold slots routed to e
                        expert_of_row = idx.reshape(-1).long()[row_src.long()]
                        bounds = torch.bucketize(torch.arange(2 * T, device=DEV), seg[1:].long(), right=True)
                        assert torch.equal(expert_of_row, bounds)
    (out_a, loss_a, g_a), (out_b, loss_b, g_b) = results
    assert torch.isfinite(out_a.float()).all() and torch.equal(out_a, out_b)
    for a, b in zip(loss_a, loss_b):
        assert torch.equal(a, b)
    # at initialisation the loss of a uniform guess over 32000 classes
    assert abs(float(loss_a[0]) - 10.37) < 0.5
    for k, (a, b) in enumerate(zip(g_a, g_b)):
        assert torch.isfinite(a).all() and float(a.abs().max()) > 0
        assert torch.equal(a, b), f"probe {k}: {int((a != b).sum())} of {a.numel()} elements differ"


def test_checkpoint_round_trip_resumes_training_bit_for_bit(tmp_path):
    """Parameters and optimizer state saved from lowered stages and loaded into freshly built ones
    (in place, into the arenas the launch lists point to) continue training with identical
    results: same losses and same parameters after the next step."""
    import pippy_amd as pp
    from pippy_amd.utilities.hf_checkpoint import load_checkpoint, save_checkpoint
    M = 4

    def build(seed):
        model, ref, stages, ref_stages, ids = _build_decoder(2, M=M, seed=seed)
        sched = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
        opt = pp.FusedAdamW(stages, lr=1e-2, weight_decay=0.1, master_weights=True)
        return model, stages, sched, opt

    torch.manual_seed(7)
    ids = torch.randint(0, 1000, (2 * M, 128), device=DEV)
    target = torch.randint(0, 1000, (2 * M, 128), device=DEV)

    def train_step(sched, opt):
        opt.zero_grad()
        losses = []
        sched.step(ids, target=target, losses=losses)
        opt.step()
        return torch.stack(losses).clone()

    model_a, stages_a, sched_a, opt_a = build(0)
    train_step(sched_a, opt_a)
    index = save_checkpoint(stages_a, str(tmp_path), optimizer=opt_a)
    loss_a = train_step(sched_a, opt_a)

    model_b, stages_b, sched_b, opt_b = build(1)              # different initial weights
    train_step(sched_b, opt_b)                               # lowers the stages, fills state
    for st in stages_b:
        load_checkpoint(st, index)
    opt_b.load_state_dict(torch.load(tmp_path / "pytorch_optim-00001-of-00001.bin", weights_only=True))
    loss_b = train_step(sched_b, opt_b)
    assert torch.equal(loss_a, loss_b)
    sd_a, sd_b = model_a.state_dict(), model_b.state_dict()
    for k in sd_a:
        assert torch.equal(sd_a[k], sd_b[k]), k


# ---- skip connections: a stage fed by several earlier stages --------------------------------------
class _SkipNet(torch.nn.Module):
    """The model of the reference's skip-connection test (``test/test_skip_conn.py:20-45``)."""

    def __init__(self, d=16):
        super().__init__()
        self.mm_param0 = torch.nn.Parameter(torch.randn(d, d) * 0.3)
        self.mm_param1 = torch.nn.Parameter(torch.randn(d, d) * 0.3)
        self.mm_param2 = torch.nn.Parameter(torch.randn(d, d) * 0.3)
        self.lin1 = torch.nn.Linear(d, d)
        self.lin2 = torch.nn.Linear(d, d)

    def forward(self, x, y):
        import pippy_amd as pp
        x = torch.mm(x, self.mm_param0)
        x = torch.relu(x + y)
        skip_conn = x
        pp.pipe_split()
        x = self.lin1(torch.mm(x, self.mm_param1))
        pp.pipe_split()
        x = torch.mm(torch.relu(x), self.mm_param2)
        pp.pipe_split()
        return torch.relu(self.lin2(x + skip_conn))


@pytest.mark.parametrize("schedule", ["ScheduleGPipe", "Schedule1F1B"])
def test_skip_connection_forward_and_backward_match_the_unsplit_model(schedule):
    import pippy_amd as pp
    torch.manual_seed(0)
    model = _SkipNet()
    x, y, target = (torch.randn(8, 16, device=DEV) for _ in range(3))
    pipe = pp.pipeline(model, 4, (x.cpu(),), {"y": y.cpu()})
    assert pipe.num_stages == 4
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(4)]
    assert not any(st.is_native for st in stages)
    loss_fn = torch.nn.MSELoss(reduction="sum")
    sched = getattr(pp, schedule)(stages, 4, loss_fn=loss_fn)
    losses = []
    out = sched.step(x, y=y, target=target, losses=losses)
    ref = copy.deepcopy(model)   # the stages moved the parameters to the GPU
    for p in ref.parameters():
        p.grad = None
    ref_out = ref(x, y)
    loss_fn(ref_out, target).backward()
    torch.testing.assert_close(out, ref_out)
    torch.testing.assert_close(sum(losses), loss_fn(ref_out, target))
    # stage 0's output has two consumers (stages 1 and 3): its gradient is their sum
    named = dict(model.named_parameters())
    for name, rp in ref.named_parameters():
        g = named[name].grad
        assert g is not None, name
        torch.testing.assert_close(g, rp.grad, rtol=1e-4, atol=1e-5)


def test_plain_torch_gpt_runs_natively_and_matches_the_oracle():
    """A GPT-2-shaped model written without any block of this package (nn.Embedding, nn.LayerNorm,
    nn.Linear, F.scaled_dot_product_attention, residual adds; the kind of model the reference is handed,
    examples/huggingface/pippy_gpt2.py:50-65): both stages must run as launch lists, and logits, losses and
    every parameter gradient must match the fp32 oracle run of the same model."""
    import sys, os
    import torch.nn as nn
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import GPT
    import pippy_amd as pp
    torch.manual_seed(0)
    M, vocab, seq = 4, 1000, 128
    model = GPT(vocab=vocab, seq=seq, d=128, h=2, L=4).to(torch.bfloat16)
    ref = copy.deepcopy(model).float()
    ids = torch.randint(0, vocab, (2 * M, seq))
    target = torch.randint(0, vocab, (2 * M, seq))
    pipe = pp.pipeline(model, M, (ids,), split_spec={"h.2": pp.SplitPoint.BEGINNING})
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
    assert all(st.is_native for st in stages), [st.eager_reason for st in stages]
    sched = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
    losses = []
    out = sched.step(ids.to(DEV), target=target.to(DEV), losses=losses)
    torch.cuda.synchronize()

    class Front(nn.Module):
        def __init__(self, g):
            super().__init__()
            self.g = g

        def forward(self, idx):
            x = self.g.wte(idx) + self.g.wpe(torch.arange(idx.shape[1]))
            for blk in self.g.h[:2]:
                x = blk(x)
            return x

    class Back(nn.Module):
        def __init__(self, g):
            super().__init__()
            self.g = g

        def forward(self, x):
            for blk in self.g.h[2:]:
                x = blk(x)
            return self.g.lm_head(self.g.ln_f(x))

    ref_out, ref_losses = OP.step([Front(ref), Back(ref)], ids, target, M, _ce)
    assert_close_rel(out, ref_out, BF16_TOL, "merged logits")
    for m in range(M):
        assert_close_rel(losses[m].reshape(1), ref_losses[m].reshape(1), BF16_TOL, f"loss {m}")
    named = dict(model.named_parameters())
    for name, rp in ref.named_parameters():
        err = max_rel(named[name].main_grad, rp.grad)
        assert err <= BF16_TOL, f"grad of {name}: max relative error {err:.3e}"


def test_small_steps_run_on_one_stream_and_give_the_same_bits(monkeypatch):
    """A schedule left to itself (``concurrent_stages = None``) runs the stages of a small model on the caller's
    stream — the host cost of two streams exceeds such kernels — and a large one on two; either way the
    results are the same bits."""
    import pippy_amd as pp
    model, ref, stages, ref_stages, ids = _build_decoder(2, n_layers=2, M=4)
    target = torch.randint(0, 1000, ids.shape)
    sched = pp.Schedule1F1B(stages, 4, loss_fn=pp.CrossEntropyLoss())
    assert sched.concurrent_stages is None
    monkeypatch.setenv("PIPPY_AMD_CONCURRENT_STAGES", "1")
    la = []
    out_a = sched.step(ids.to(DEV), target=target.to(DEV), losses=la).clone()
    assert sched._stage_streams([(ids,)]) is not None
    grads_a = [p.main_grad.clone() for p in model.parameters()]
    monkeypatch.delenv("PIPPY_AMD_CONCURRENT_STAGES")
    sched.zero_grad()
    lb = []
    out_b = sched.step(ids.to(DEV), target=target.to(DEV), losses=lb)
    assert sched._stage_streams([(ids[:2],)]) is None          # 256 rows x 1 M parameters: a small step
    assert sched._stage_streams([(ids.repeat(64, 8)[:2048],)]) is not None   # 2 M rows: not small
    assert torch.equal(out_a, out_b) and all(torch.equal(a, b) for a, b in zip(la, lb))
    assert all(torch.equal(p.main_grad, g) for p, g in zip(model.parameters(), grads_a))


def test_column_sums_come_from_the_kernels_that_produced_the_tensors(monkeypatch):
    """The weight-gradient passes of a decoder stage take the column sums of their bias and norm-parameter
    gradients from partial sums that the input-gradient pass left (LayerNorm input gradient, GELU' GEMM
    epilogue, attention backward): every reduction of a layer's own tensors is rewired, only the reduction over
    the gradient that arrives from outside the stage still reads its tensor.  The gradients equal those of
    the two-pass reductions up to fp32 summation order (and the bf16 rounding of a microbatch's gradient that it
    can move by one step)."""
    import pippy_amd as pp
    from pippy_amd import _native as N
    M = 4

    def run(two_pass):
        if two_pass:
            monkeypatch.setenv("PIPPY_AMD_TWO_PASS_COLUMN_SUMS", "1")
        else:
            monkeypatch.delenv("PIPPY_AMD_TWO_PASS_COLUMN_SUMS", raising=False)
        model, ref, stages, ref_stages, ids = _build_decoder(2, n_layers=4, M=M, dim=128, heads=2)
        target = torch.randint(0, 1000, ids.shape, generator=torch.Generator().manual_seed(5))
        sched = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
        sched.step(ids.to(DEV), target=target.to(DEV), losses=[])
        torch.cuda.synchronize()
        ready = []
        for st in stages:
            W = st._program.mbs[0].W
            ops = [W[k] for k in range(W.n) if W[k].kind in (N.OP_COLSUM, N.OP_LN_BWD_WEIGHT)]
            ready.append((sum(1 for o in ops if o.j[1] > 0), len(ops)))
        return ready, {n: p.main_grad.clone() for n, p in model.named_parameters()}

    ready, grads = run(False)
    # per layer: two norms, four biases; the first stage also has no final norm, the last stage one more norm;
    # what stays two-pass: the bias of the last linear layer of a stage's last block (its output gradient
    # comes from the next stage or from the loss path's own kernels) and the final norm's parameters, whose
    # input gradient is written by the vocabulary projection's input-gradient GEMM
    for (n_ready, n_all) in ready:
        assert n_all - n_ready <= 2 and n_ready >= 2 * 6 - 1, (n_ready, n_all)
    ready2, grads2 = run(True)
    assert all(n_ready == 0 for n_ready, _ in ready2)
    # a microbatch's gradient is rounded to bf16 before it is accumulated: a last-bit difference of an fp32
    # sum can move that rounding by one bf16 step (2^-8 of the element), no more
    for name, g in grads.items():
        err = (g - grads2[name]).abs().max().item()
        assert err <= M * 2.0 ** -8 * grads2[name].abs().max().item() + 1e-12, (name, err)


def test_a_stage_lowered_in_eval_mode_refuses_to_train_with_its_dropout_switched_on():
    """Dropout with p > 0 is identity in eval mode, so a model built that way lowers to launch lists — which
    hold no dropout.  Put into training mode afterwards the stage must raise rather than train without
    dropout; back in eval mode it runs again, with the same result as before."""
    import sys, os
    import torch.nn as nn
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import GPT
    import pippy_amd as pp
    torch.manual_seed(0)
    M, vocab, seq = 2, 1000, 64
    model = GPT(vocab=vocab, seq=seq, d=128, h=2, L=2).to(torch.bfloat16)
    for m in model.modules():
        if isinstance(m, nn.Dropout):
            m.p = 0.1
    model.eval()
    ids = torch.randint(0, vocab, (2 * M, seq))
    pipe = pp.pipeline(model, M, (ids,), split_spec={"h.1": pp.SplitPoint.BEGINNING})
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
    assert all(st.is_native for st in stages), [st.eager_reason for st in stages]
    sched = pp.ScheduleGPipe(stages, M)
    first = sched.step(ids.to(DEV)).clone()
    for st in stages:
        st.submod.train()
    with pytest.raises(RuntimeError, match="dropout"):
        sched.step(ids.to(DEV))
    for st in stages:
        st.submod.eval()
    assert torch.equal(sched.step(ids.to(DEV)), first)
    # the other direction: built in training mode with p > 0, the stages stay with torch autograd and say why
    model2 = GPT(vocab=vocab, seq=seq, d=128, h=2, L=2).to(torch.bfloat16)
    for m in model2.modules():
        if isinstance(m, nn.Dropout):
            m.p = 0.1
    model2.train()
    pipe2 = pp.pipeline(model2, M, (ids,), split_spec={"h.1": pp.SplitPoint.BEGINNING})
    st2 = pp.PipelineStage(pipe2, 0, DEV)
    assert not st2.is_native and "dropout" in st2.eager_reason


def _exported_model_against_the_oracle(model, whole, vocab, seq, split, before_oracle=None, padding=None):
    """Pipelines ``model`` (which torch.fx cannot trace: the front end exports it on one microbatch) in
    two stages, checks that both run as launch lists, and compares logits, losses and every parameter
    gradient with the fp32 oracle run of ``whole(copy of the model)``: 2e-2 per tensor, and a gradient that
    misses it must be no further from the fp32 result than torch's own bf16 autograd on the same model is
    (``_util.check_gradients``).  ``before_oracle(ref, stages, M)`` may prepare the fp32 copy from what
    the run saved (a ReLU model is given the run's own active sets).  ``padding``: a token id written over
    the end of some sequences, the start of one and a few places inside."""
    import pippy_amd as pp
    M, mb = 4, 2
    model = model.to(torch.bfloat16)
    ref = copy.deepcopy(model).float()
    ref16 = copy.deepcopy(model)
    ids = torch.randint(0, vocab, (mb * M, seq))
    if padding is not None:
        ids[0, seq - 9:] = padding
        ids[3, seq // 2:] = padding
        ids[5, :4] = padding
        ids[6, 10:13] = padding
    target = torch.randint(0, vocab, (mb * M, seq))
    pipe = pp.pipeline(model, mb_args=(ids[:mb],), split_spec={split: pp.SplitPoint.BEGINNING})
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
    assert all(st.is_native for st in stages), [st.eager_reason for st in stages]
    sched = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
    losses = []
    out = sched.step(ids.to(DEV), target=target.to(DEV), losses=losses)
    torch.cuda.synchronize()
    if isinstance(out, (tuple, list)):
        out = out[0]
    if before_oracle is not None:
        before_oracle(ref, stages, M)
    ref_out, ref_losses = OP.step([whole(ref)], ids, target, M, _ce)
    assert_close_rel(out, ref_out, BF16_TOL, "merged logits")
    for m in range(M):
        assert_close_rel(losses[m].reshape(1), ref_losses[m].reshape(1), BF16_TOL, f"loss {m}")
    def run_in_bf16():
        if before_oracle is not None:
            before_oracle(ref16, stages, M)
        OP.step([whole(ref16)], ids, target, M, _ce)
        return dict(ref16.named_parameters())

    check_gradients(dict(model.named_parameters()), dict(ref.named_parameters()), run_in_bf16, "exported model", note)


def test_exported_library_style_gpt_runs_natively_and_matches_the_oracle():
    """A GPT-2 written the way model libraries write it (affine layers with [in, out] weights, an
    activation class of its own, an explicit boolean causal mask, control flow on shapes): the front end
    has to go through torch.export, and the stages must still run as launch lists on the model's own
    parameters — the [in, out] weights feed the GEMMs as the other operand and receive X^T dY."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import LibGPT
    torch.manual_seed(0)
    _exported_model_against_the_oracle(LibGPT(vocab=1000, seq=128, d=128, h=2, L=4), lambda g: g, 1000, 128, "h.2")


def test_hugging_face_gpt2_runs_natively_and_matches_the_oracle():
    """The model of the reference's own example (examples/huggingface/pippy_gpt2.py:50-65, with untied
    embeddings: a parameter shared between stages is rejected there as here), straight from the
    ``transformers`` package with random weights."""
    transformers = pytest.importorskip("transformers")
    import torch.nn as nn
    cfg = transformers.GPT2Config(n_layer=4, n_embd=128, n_head=2, vocab_size=1000, n_positions=128,
                                  attn_pdrop=0.0, embd_pdrop=0.0, resid_pdrop=0.0, use_cache=False,
                                  tie_word_embeddings=False, bos_token_id=0, eos_token_id=0)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.GPT2LMHeadModel(cfg)

    class Logits(nn.Module):
        def __init__(self, g):
            super().__init__()
            self.g = g

        def forward(self, idx):
            return self.g(idx).logits

    _exported_model_against_the_oracle(model, Logits, 1000, 128, "transformer.h.2")


@pytest.mark.parametrize("norm_first,activation", [(True, "gelu"), (False, "relu")])
def test_torchs_own_encoder_layers_run_natively_and_match_the_oracle(norm_first, activation):
    """A model built from ``nn.TransformerEncoderLayer`` (torch.fx keeps each layer whole): both stages
    run as launch lists on the layers' own parameters, the packed q|k|v weight of ``nn.MultiheadAttention``
    included, and match the fp32 oracle run of the same model."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import TorchEncoderLM
    torch.manual_seed(0)
    vocab = 1000 if norm_first else 1003     # (a width the GEMMs and the loss kernel take only padded)
    model = TorchEncoderLM(vocab=vocab, seq=128, d=128, h=2, L=4, norm_first=norm_first, activation=activation)
    _exported_model_against_the_oracle(model, lambda g: g, vocab, 128, "layers.2",
                                       before_oracle=_relu_sets_of_torch_layers if activation == "relu" else None)


def test_a_causal_model_of_torchs_encoder_layers_runs_natively_and_matches_the_oracle():
    """A decoder-only model made of ``nn.TransformerEncoderLayer`` with a causal mask built in forward
    from the sequence length: exported (so that the mask is a constant of each stage), recognised as
    causal layers, run as launch lists."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import TorchCausalLM
    torch.manual_seed(0)
    model = TorchCausalLM(vocab=1000, seq=128, d=128, h=2, L=4)
    _exported_model_against_the_oracle(model, lambda g: g, 1000, 128, "layers.2")


@pytest.mark.parametrize("bias,flash", [(True, False), (False, True)])
def test_a_teaching_style_gpt_runs_natively_and_matches_the_oracle(bias, flash):
    """A GPT with a layer-norm class of its own (optionally without biases anywhere) and attention through
    the fused call or spelled out against a lower-triangular buffer."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import TeachingGPT
    torch.manual_seed(0)
    model = TeachingGPT(vocab=1000, seq=128, d=128, h=2, L=4, bias=bias, flash=flash)
    _exported_model_against_the_oracle(model, lambda g: g, 1000, 128, "transformer.h.2")


@pytest.mark.parametrize("need_weights,causal", [(True, False), (True, True)])
def test_blocks_around_torchs_attention_layer_run_natively_and_match_the_oracle(need_weights, causal):
    """Blocks of one's own around ``nn.MultiheadAttention`` called the default way (averaged weights
    computed and dropped), without a mask (traced: the layer is one call) and with a causal mask built
    from the sequence length (exported: the layer spells its attention out)."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import MHAModel
    torch.manual_seed(0)
    model = MHAModel(vocab=1000, seq=128, d=128, h=2, L=4, need_weights=need_weights, causal=causal)
    _exported_model_against_the_oracle(model, lambda g: g, 1000, 128, "blocks.2")


def test_torchs_encoder_stack_runs_natively_and_matches_the_oracle():
    """The layers inside ``nn.TransformerEncoder``: exported, recognised on the parameters that
    ``nn.MultiheadAttention`` applies as functions, run as launch lists."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import TorchEncoderStackLM
    torch.manual_seed(0)
    model = TorchEncoderStackLM(vocab=1000, seq=128, d=128, h=2, L=4)
    _exported_model_against_the_oracle(model, lambda g: g, 1000, 128, "encoder.layers.2")


def _relu_sets_of_torch_layers(ref, stages, M):
    """The run's ReLU active sets for a model of ``nn.TransformerEncoderLayer``s (see _relu_sets_of_the_run)."""
    import torch.nn as nn
    layers = [m for m in ref.modules() if isinstance(m, nn.TransformerEncoderLayer)]
    at = 0
    for st in stages:
        count = 0
        for m in range(M):
            hs = [v for k, v in st.saved_activations(m).items() if k.split(".")[-1] == "h"]
            count = len(hs)
            for j, h in enumerate(hs):
                layers[at + j].__dict__.setdefault("_sets", []).append((h > 0).cpu())
        at += count
    assert at == len(layers)
    for layer in layers:
        sets = layer.__dict__["_sets"]

        def forced(x, sets=sets):
            active = sets.pop(0).reshape(x.shape)
            flipped = active != (x > 0)
            assert flipped.float().mean() < 0.02 and (not flipped.any() or x[flipped].abs().max() < 2e-2 * x.abs().max())
            return x * active

        layer.activation = forced
        layer.activation_relu_or_gelu = 0


def test_an_exported_stage_runs_any_batch_size_but_only_its_sequence_length():
    """An exported stage holds constants made for the example's shape (here a causal mask cut for 64
    positions).  Its launch lists take other batch sizes, samples being independent; another sequence
    length is refused with the reason instead of being computed with whatever the blocks would assume.  A
    symbolically traced model holds no shapes and runs both."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import GPT, LibGPT
    import pippy_amd as pp
    for cls, exported in ((LibGPT, True), (GPT, False)):
        torch.manual_seed(0)
        model = cls(vocab=300, seq=128, d=128, h=2, L=4).to(torch.bfloat16)
        ids = torch.randint(0, 300, (2, 64))
        pipe = pp.pipeline(model, mb_args=(ids,), split_spec={"h.2": pp.SplitPoint.BEGINNING})
        stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
        assert all(st.is_native for st in stages)
        sched = pp.ScheduleGPipe(stages, 2)
        big = torch.randint(0, 300, (6, 64))
        out = sched.step(big.to(DEV))
        assert_close_rel(out, model.to(DEV)(big.to(DEV)), BF16_TOL, "another batch size")
        model.cpu()
        longer = torch.randint(0, 300, (4, 96))
        if exported:
            with pytest.raises(RuntimeError, match="exported on inputs of shape"):
                sched.step(longer.to(DEV))
        else:
            out = sched.step(longer.to(DEV))
            assert_close_rel(out, model.to(DEV)(longer.to(DEV)), BF16_TOL, "another sequence length")


def test_exported_stages_that_do_not_lower_run_through_autograd_on_the_gpu():
    """An exported model whose attention mask is not the causal one (a sliding window) keeps its stages
    with torch autograd.  Their graphs were exported on the host: the folded constants (mask, position
    indices) must move to the GPU with the stage, and results must equal the unsplit model's."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import LibGPT
    import pippy_amd as pp
    torch.manual_seed(0)
    model = LibGPT(vocab=300, seq=64, d=128, h=2, L=4)

    def windowed(idx):
        t = idx.shape[-1]
        if t > model.wpe.num_embeddings:
            raise ValueError("sequence too long")
        pos = torch.arange(t, device=idx.device).unsqueeze(0)
        mask = ((pos.unsqueeze(-1) >= pos.unsqueeze(-2)) & (pos.unsqueeze(-1) - pos.unsqueeze(-2) < 8))[:, None]
        mask = mask.expand(idx.shape[0], 1, t, t)
        x = model.wte(idx) + model.wpe(pos)
        for blk in model.h:
            x = blk(x, mask)
        return model.lm_head(model.ln_f(x))

    model.forward = windowed
    M, mb, seq = 4, 2, 48
    ids = torch.randint(0, 300, (mb * M, seq))
    target = torch.randint(0, 300, (mb * M, seq))
    pipe = pp.pipeline(model, mb_args=(ids[:mb],), split_spec={"h.2": pp.SplitPoint.BEGINNING})
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
    assert not any(st.is_native for st in stages) and "mask" in stages[1].eager_reason
    sched = pp.Schedule1F1B(stages, M, loss_fn=_ce)
    losses = []
    out = sched.step(ids.to(DEV), target=target.to(DEV), losses=losses)
    for p in model.parameters():          # the stages moved the model's parameters to the GPU
        assert p.is_cuda
    grads = {n: p.grad.clone() for n, p in model.named_parameters()}
    for p in model.parameters():
        p.grad = None
    ref_out = model(ids.to(DEV))
    ref_losses = [_ce(o, t) for o, t in zip(ref_out.chunk(M), target.to(DEV).chunk(M))]
    sum(ref_losses).backward()
    torch.testing.assert_close(out, ref_out, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(torch.stack(losses), torch.stack(ref_losses), rtol=1e-4, atol=1e-5)
    for name, p in model.named_parameters():
        torch.testing.assert_close(grads[name], p.grad, rtol=1e-3, atol=1e-5, msg=lambda m: f"{name}: {m}")


@pytest.mark.parametrize("heads,kv_heads", [(4, 4), (4, 2)])
def test_hugging_face_llama_runs_natively_and_matches_the_oracle(heads, kv_heads):
    """The model class of the reference's Llama example (examples/llama/pippy_llama.py:18-39) with random
    weights: separate q / k / v projections, rotary embedding from a table the model computes under
    no_grad, LlamaRMSNorm, SwiGLU, grouped-query attention when kv_heads < heads."""
    transformers = pytest.importorskip("transformers")
    import torch.nn as nn
    cfg = transformers.LlamaConfig(hidden_size=64 * heads, intermediate_size=512, num_hidden_layers=4,
                                   num_attention_heads=heads, num_key_value_heads=kv_heads, vocab_size=1000,
                                   max_position_embeddings=128, use_cache=False, tie_word_embeddings=False,
                                   attention_dropout=0.0,
                                   pad_token_id=0 if kv_heads != heads else None)   # row 0 then gets no gradient
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.LlamaForCausalLM(cfg)

    class Logits(nn.Module):
        def __init__(self, g):
            super().__init__()
            self.g = g

        def forward(self, idx):
            return self.g(idx).logits

    _exported_model_against_the_oracle(model, Logits, 1000, 128, "model.layers.2")


def test_hugging_face_bert_runs_natively_and_matches_the_oracle():
    """transformers.BertForMaskedLM (the encoder family of examples/huggingface/pippy_bert.py) with random
    weights: word + position + token-type embeddings under a LayerNorm, post-LayerNorm layers with separate
    query / key / value projections and an all-true mask, erf-GELU, and the masked-language-model head
    (dense + GELU + LayerNorm + a decoder with a bias over a vocabulary that is not a multiple of 8)."""
    transformers = pytest.importorskip("transformers")
    import torch.nn as nn
    cfg = transformers.BertConfig(hidden_size=128, intermediate_size=512, num_hidden_layers=4, num_attention_heads=2,
                                  vocab_size=1003, max_position_embeddings=128, hidden_dropout_prob=0.0,
                                  attention_probs_dropout_prob=0.0, tie_word_embeddings=False)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.BertForMaskedLM(cfg)

    class Logits(nn.Module):
        def __init__(self, g):
            super().__init__()
            self.g = g

        def forward(self, idx):
            return self.g(idx).logits

    _exported_model_against_the_oracle(model, Logits, 1003, 128, "bert.encoder.layer.2")


@pytest.mark.parametrize("family", ["qwen2", "mistral", "phi3", "distilbert", "electra", "opt", "gpt2_spelled_out",
                                    "megatron_bert", "gpt_neo", "roberta", "qwen3", "qwen3_wide_heads", "gpt_bigcode", "falcon"])
def test_more_hugging_face_families_run_natively_and_match_the_oracle(family):
    """Families that the same recognisers cover: Qwen2 (Llama layout with biases on the query / key /
    value projections), Mistral (Llama layout), Phi-3 (one fused q|k|v and one fused gate|up projection),
    DistilBERT (encoder without token types, its own layer names), ELECTRA (BERT layout with a generator
    head), OPT (the reference's examples/huggingface/pippy_opt.py: queries scaled before an attention
    call with scale 1, a position table read from row 2 on, ReLU feed-forward; exported in eval mode, as
    the example runs it, since its training-mode layer drop branches on a random number); and models whose
    attention is spelled out as softmax(q k^T c + mask) v instead of one call: GPT-2 with the library's
    "eager" attention, Megatron-BERT (pre-LayerNorm encoder, embeddings without a LayerNorm, a final
    LayerNorm in front of the head's transform; examples/huggingface/pippy_megatronBert.py) and GPT-Neo
    (scores without the 1 / sqrt(head size) factor, the causal mask applied twice, projections without
    biases, "local" layers whose window covers the sequence; examples/huggingface/pippy_gptNeo.py); and
    RoBERTa (the family of examples/huggingface/pippy_camemBert.py), whose position indices count the
    tokens that are not padding: the input holds padding at the end, the start and inside of sequences;
    Qwen3 (RMS norms over each head's values of queries and keys in front of the rotary embedding; in
    the second variant a head size of 128 that is not width / heads, so that the query projection widens
    the stream and the output projection narrows it again); GPT-BigCode (multi-query attention in a
    GPT-2-style layer: one fused projection of width d + 2 D, all query heads on one key / value head);
    Falcon (attention and feed-forward side by side on the residual stream behind one LayerNorm, rotary
    embedding, multi-query attention, no biases)."""
    T = pytest.importorskip("transformers")
    import torch.nn as nn
    common = dict(vocab_size=1000, tie_word_embeddings=False)
    llama_like = dict(hidden_size=256, intermediate_size=512, num_hidden_layers=4, num_attention_heads=4,
                      num_key_value_heads=2, max_position_embeddings=128, attention_dropout=0.0, use_cache=False)
    cls, cfg, split = {
        "qwen2": lambda: (T.Qwen2ForCausalLM, T.Qwen2Config(**llama_like, **common), "model.layers.2"),
        "mistral": lambda: (T.MistralForCausalLM, T.MistralConfig(sliding_window=None, **llama_like, **common),
                            "model.layers.2"),
        "phi3": lambda: (T.Phi3ForCausalLM,
                         T.Phi3Config(**{**llama_like, "num_key_value_heads": 4}, resid_pdrop=0.0, embd_pdrop=0.0,
                                      pad_token_id=0, **common), "model.layers.2"),
        "distilbert": lambda: (T.DistilBertForMaskedLM,
                               T.DistilBertConfig(dim=128, hidden_dim=512, n_layers=4, n_heads=2,
                                                  max_position_embeddings=128, dropout=0.0, attention_dropout=0.0,
                                                  **common), "distilbert.transformer.layer.2"),
        "electra": lambda: (T.ElectraForMaskedLM,
                            T.ElectraConfig(hidden_size=128, embedding_size=128, intermediate_size=512,
                                            num_hidden_layers=4, num_attention_heads=2, max_position_embeddings=128,
                                            hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0, **common),
                            "electra.encoder.layer.2"),
        "opt": lambda: (T.OPTForCausalLM,
                        T.OPTConfig(hidden_size=128, ffn_dim=512, num_hidden_layers=4, num_attention_heads=2,
                                    max_position_embeddings=128, dropout=0.0, layerdrop=0.0, use_cache=False,
                                    **common), "model.decoder.layers.2"),
        "gpt2_spelled_out": lambda: (T.GPT2LMHeadModel,
                                     T.GPT2Config(n_layer=4, n_embd=128, n_head=2, n_positions=128, attn_pdrop=0.0,
                                                  embd_pdrop=0.0, resid_pdrop=0.0, use_cache=False, bos_token_id=0,
                                                  eos_token_id=0, **common), "transformer.h.2"),
        "megatron_bert": lambda: (T.MegatronBertForMaskedLM,
                                  T.MegatronBertConfig(hidden_size=128, intermediate_size=512, num_hidden_layers=4,
                                                       num_attention_heads=2, max_position_embeddings=128,
                                                       hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0,
                                                       **common), "bert.encoder.layer.2"),
        "gpt_neo": lambda: (T.GPTNeoForCausalLM,
                            T.GPTNeoConfig(hidden_size=128, num_layers=4, num_heads=2, window_size=256,
                                           attention_types=[[["global", "local"], 2]], max_position_embeddings=128,
                                           embed_dropout=0.0, attention_dropout=0.0, resid_dropout=0.0,
                                           use_cache=False, bos_token_id=0, eos_token_id=0, **common),
                            "transformer.h.2"),
        "qwen3": lambda: (T.Qwen3ForCausalLM, T.Qwen3Config(head_dim=64, **llama_like, **common), "model.layers.2"),
        "qwen3_wide_heads": lambda: (T.Qwen3ForCausalLM, T.Qwen3Config(head_dim=128, **llama_like, **common),
                                     "model.layers.2"),
        "gpt_bigcode": lambda: (T.GPTBigCodeForCausalLM,
                                T.GPTBigCodeConfig(n_embd=256, n_layer=4, n_head=4, n_positions=128, attn_pdrop=0.0,
                                                   embd_pdrop=0.0, resid_pdrop=0.0, use_cache=False, multi_query=True,
                                                   bos_token_id=0, eos_token_id=0, **common), "transformer.h.2"),
        "falcon": lambda: (T.FalconForCausalLM,
                           T.FalconConfig(hidden_size=256, num_hidden_layers=4, num_attention_heads=4,
                                          hidden_dropout=0.0, attention_dropout=0.0, use_cache=False,
                                          max_position_embeddings=128, **common), "transformer.h.2"),
        "roberta": lambda: (T.RobertaForMaskedLM,
                            T.RobertaConfig(hidden_size=128, intermediate_size=512, num_hidden_layers=4,
                                            num_attention_heads=2, max_position_embeddings=132,
                                            hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0, **common),
                            "roberta.encoder.layer.2"),
    }[family]()
    cfg._attn_implementation = "eager" if family in ("gpt2_spelled_out", "megatron_bert", "gpt_neo") else "sdpa"
    torch.manual_seed(0)
    model = cls(cfg)
    if family == "opt":
        model.eval()
    if family == "qwen2":
        with torch.no_grad():      # the library initialises biases to zero: give them values
            for name, p in model.named_parameters():
                if name.endswith("_proj.bias"):
                    p.normal_(std=0.05)
    if family.startswith("qwen3"):
        with torch.no_grad():      # (and per-head norm weights to one)
            for name, p in model.named_parameters():
                if name.endswith(("q_norm.weight", "k_norm.weight")):
                    p.add_(torch.randn_like(p) * 0.3)

    class Logits(nn.Module):
        def __init__(self, g):
            super().__init__()
            self.g = g

        def forward(self, idx):
            return self.g(idx).logits

    _exported_model_against_the_oracle(model, Logits, 1000, 128, split,
                                       before_oracle=_relu_sets_of_the_run if family == "opt" else None,
                                       padding=cfg.pad_token_id if family == "roberta" else None)


def _relu_sets_of_the_run(ref, stages, M):
    """A ReLU is discontinuous: a pre-activation within rounding distance of zero is active in one
    arithmetic and not in the other, and the few such elements of a feed-forward column shift that
    column's gradients by several percent — in torch's own bf16 autograd as much as here.  The fp32 copy
    therefore multiplies by the active sets of the bf16 run (its saved feed-forward activations > 0), in
    layer order per microbatch; that those sets are the ReLU's own is checked where they differ: only at
    pre-activations that are tiny in the fp32 run."""
    import torch.nn as nn
    layers = [m for m in ref.modules() if hasattr(m, "activation_fn") and hasattr(m, "fc1")]
    per_layer = [[] for _ in layers]
    at = 0
    for st in stages:
        count = None
        for m in range(M):
            hs = [v for k, v in st.saved_activations(m).items() if k.split(".")[-1] == "h"]
            count = len(hs)
            for j, h in enumerate(hs):
                per_layer[at + j].append((h > 0).cpu())
        at += count
    assert at == len(layers)

    class RunsActiveSet(nn.Module):
        def __init__(self, sets):
            super().__init__()
            self.sets = sets

        def forward(self, x):
            active = self.sets.pop(0).reshape(x.shape)
            flipped = active != (x > 0)
            assert flipped.float().mean() < 0.02 and (not flipped.any() or
                                                       x[flipped].abs().max() < 2e-2 * x.abs().max()), \
                "the run's active set differs from the ReLU's beyond rounding"
            return x * active

    for layer, sets in zip(layers, per_layer):
        layer.activation_fn = RunsActiveSet(sets)


def test_hugging_face_mixtral_runs_natively_and_matches_the_oracle():
    """Mixtral from the ``transformers`` package: experts stacked in two parameters per layer, the
    sparse block recognised from what it reads.  The oracle is the fp32 copy of the model, pipelined and
    recognised the same way on the host (those blocks equal the library's forward: a host test), so that
    it can be given the expert selection of the bf16 run; that the selection is the top-2 of the run's own
    router logits is checked here."""
    T = pytest.importorskip("transformers")
    import torch.nn as nn
    import pippy_amd as pp
    from pippy_amd._lowering import lower_stage_module
    M, mb, S, vocab, L, E = 4, 2, 128, 1000, 4, 8
    cfg = T.MixtralConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=L, num_attention_heads=4,
                          num_key_value_heads=2, vocab_size=vocab, max_position_embeddings=S, use_cache=False,
                          tie_word_embeddings=False, num_local_experts=E, num_experts_per_tok=2,
                          attention_dropout=0.0, sliding_window=None, router_jitter_noise=0.0)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = T.MixtralForCausalLM(cfg)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("mlp.gate.weight"):
                p.mul_(10)                           # decisive routing: few near-ties
    model = model.to(torch.bfloat16)
    ref = copy.deepcopy(model).float()
    ids = torch.randint(0, vocab, (mb * M, S))
    target = torch.randint(0, vocab, (mb * M, S))
    split = {f"model.layers.{L // 2}": pp.SplitPoint.BEGINNING}
    pipe = pp.pipeline(model, mb_args=(ids[:mb],), split_spec=split)
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
    assert all(st.is_native for st in stages), [st.eager_reason for st in stages]
    sched = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
    losses = []
    out = sched.step(ids.to(DEV), target=target.to(DEV), losses=losses)
    torch.cuda.synchronize()
    out = out[0] if isinstance(out, (tuple, list)) else out
    ref_pipe = pp.pipeline(ref, mb_args=(ids[:mb],), split_spec=split)
    ref_blocks = [lower_stage_module(ref_pipe.get_stage_module(i)) for i in range(2)]
    for s, st in enumerate(stages):
        layers = [b for b in ref_blocks[s] if type(b).__name__ == "WrappedMoELayer"]
        assert len(layers) == L // 2
        for layer in layers:
            layer.forced_routing = []
        for m in range(M):
            acts = st.saved_activations(m)
            idx = [v for k, v in acts.items() if k.endswith("topk_idx")]
            logits = [v for k, v in acts.items() if k.endswith("router_logits")]
            assert len(idx) == len(layers)
            for j, layer in enumerate(layers):
                want, _ = OO.moe_route_top2(logits[j][:, :E].float().cpu())
                assert torch.equal(idx[j].cpu().long(), want)
                layer.forced_routing.append(idx[j].cpu().long())
    ref_out, ref_losses = OP.step([nn.Sequential(*bl) for bl in ref_blocks], ids, target, M, _ce)
    assert_close_rel(out, ref_out, BF16_TOL, "merged logits")
    for a, b in zip(losses, ref_losses):
        assert_close_rel(a.reshape(1), b.reshape(1), BF16_TOL, "loss")
    named = dict(model.named_parameters())
    ref_named = dict(ref.named_parameters())
    worst = 0.0
    for name, rp in ref_named.items():
        assert rp.grad is not None, name
        err = max_rel(named[name].main_grad, rp.grad)
        worst = max(worst, err)
        assert err <= BF16_TOL, f"grad of {name}: max relative error {err:.3e}"
    note(f"Hugging Face Mixtral, 1F1B: worst grad error {worst:.3e}")


def test_outputs_merged_while_the_step_runs_are_the_merge_at_the_end(monkeypatch):
    """The schedule copies each microbatch output of the last stage into the merged result as soon as
    its forward pass is issued (a side stream).  The result must be bit for bit what merging after the
    step gives, a tensor of its own (a later step must not change it), contiguous like torch.cat's, and
    uneven microbatches must fall back to the merge at the end."""
    import pippy_amd as pp
    monkeypatch.delenv("PIPPY_AMD_SERIAL_STAGES", raising=False)   # (the running merge needs the stage streams)
    monkeypatch.delenv("PIPPY_AMD_MERGE_AT_END", raising=False)
    M = 4
    model, ref, stages, ref_stages, ids = _build_decoder(2, M=M)
    target = torch.randint(0, 1000, ids.shape)
    sched = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
    ids2 = torch.randint(0, 1000, ids.shape)
    out1 = sched.step(ids.to(DEV), target=target.to(DEV))
    assert sched._merge_active is not None and out1.is_contiguous()
    kept = out1.clone()
    at_end1 = torch.cat([c.clone() for c in stages[-1].output_chunks])
    assert torch.equal(out1, at_end1)
    out2 = sched.step(ids2.to(DEV), target=target.to(DEV))
    assert torch.equal(out1, kept) and not torch.equal(out2, out1)
    monkeypatch.setenv("PIPPY_AMD_MERGE_AT_END", "1")
    out2_at_end = sched.step(ids2.to(DEV), target=target.to(DEV))
    assert sched._merge_active is None and torch.equal(out2, out2_at_end)
    monkeypatch.delenv("PIPPY_AMD_MERGE_AT_END")
    # 10 sequences in 4 microbatches: sizes 3, 3, 2, 2
    uneven = torch.randint(0, 1000, (10, ids.shape[1]))
    infer = pp.ScheduleGPipe(stages, M)
    out = infer.step(uneven.to(DEV))
    assert out.shape[0] == 10
    assert torch.equal(out, torch.cat([c.clone() for c in stages[-1].output_chunks]))
    ref_out, _ = OP.step(ref_stages, uneven, None, M, None)
    assert_close_rel(out, ref_out, BF16_TOL, "uneven microbatches")


def test_float32_transformer_stages_fall_back_to_autograd_and_say_so():
    """The attention, norm and embedding kernels are bf16: a float32 model whose structure is recognised
    still runs, through torch autograd on the GPU, and the stage says why."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from _plain_gpt import GPT
    import pippy_amd as pp
    torch.manual_seed(0)
    M, vocab, seq = 2, 300, 32
    model = GPT(vocab=vocab, seq=seq, d=128, h=2, L=2)
    ref = copy.deepcopy(model)
    ids = torch.randint(0, vocab, (2 * M, seq))
    target = torch.randint(0, vocab, (2 * M, seq))
    pipe = pp.pipeline(model, M, (ids,), split_spec={"h.1": pp.SplitPoint.BEGINNING})
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
    assert not any(st.is_native for st in stages)
    assert all("float32" in st.eager_reason and "bfloat16" in st.eager_reason for st in stages)
    sched = pp.Schedule1F1B(stages, M, loss_fn=_ce)
    losses = []
    out = sched.step(ids.to(DEV), target=target.to(DEV), losses=losses)
    ref_out = ref(ids)
    torch.testing.assert_close(out.cpu(), ref_out, rtol=1e-4, atol=1e-4)
    sum(_ce(o, t) for o, t in zip(ref_out.chunk(M), target.chunk(M))).backward()
    for (name, p), rp in zip(model.named_parameters(), ref.parameters()):
        torch.testing.assert_close(p.grad.cpu(), rp.grad, rtol=1e-3, atol=1e-5, msg=lambda m: f"{name}: {m}")


@pytest.mark.parametrize("seq", [96, 100, 40, 37])
def test_causal_layers_pad_any_sequence_length_and_match_the_oracle(seq):
    """The attention kernels take sequence lengths that are multiples of 64; causal layers run any other
    length on zero-padded copies (a key past the end is never seen, a query past the end has no output
    gradient), which must leave logits, losses and gradients those of the oracle."""
    import pippy_amd as pp
    M = 2
    model, ref, stages, ref_stages, ids = _build_decoder(2, n_layers=2, M=M, seq=seq)
    _check_against_oracle(model, ref, stages, ref_stages, ids, pp.Schedule1F1B, M)


def test_llama_layers_pad_any_sequence_length_and_match_the_oracle():
    import pippy_amd as pp
    from pippy_amd.configs import LlamaStage
    torch.manual_seed(0)
    M, seq, dim = 2, 72, 256
    model = LlamaStage(n_layers=2, dim=dim, n_heads=4, ffn=512, n_kv_heads=2)
    ref = _fp32_cpu_copy(model)
    x = (torch.randn(2 * M, seq, dim) * 0.5).to(torch.bfloat16)
    upstream = torch.randn(2 * M, seq, dim) * 1e-2
    stage = pp.ManualPipelineStage(model, 0, 1, DEV, M, input_args=(x[:2],))
    loss_fn = lambda out, up: (out.float() * up).sum()
    sched = pp.ScheduleZeroBubble([stage], M, loss_fn=loss_fn)
    losses = []
    out = sched.step(x.to(DEV), target=upstream.to(DEV), losses=losses)
    ref_out, ref_losses = OP.step([ref], x.float(), upstream, M, loss_fn)
    assert_close_rel(out, ref_out, BF16_TOL, "output")
    named = dict(model.named_parameters())
    for name, rp in ref.named_parameters():
        err = max_rel(named[name].main_grad, rp.grad)
        assert err <= BF16_TOL, f"grad of {name}: max relative error {err:.3e}"


@pytest.mark.parametrize("seq", [96, 50, 33])
def test_encoder_layers_pad_any_sequence_length_and_match_the_oracle(seq):
    """Attention without a mask over a length that is not a multiple of 64: the padded keys are left
    out of the softmax by the forward kernel (kv_len).  With 33 tokens per sequence the weight gradients
    reduce over 66 rows, not a multiple of 8."""
    import pippy_amd as pp
    from pippy_amd.configs import EncoderModel, equal_split_spec
    torch.manual_seed(0)
    M = 2
    model = EncoderModel(vocab=300, max_seq=seq, dim=128, n_layers=2, n_heads=2, ffn=256)
    ref = _fp32_cpu_copy(model)
    ids = torch.randint(0, 300, (2 * M, seq))
    upstream = torch.randn(2 * M, seq, 128) * 1e-2
    pipe = pp.pipeline(model, M, (ids,), split_spec=equal_split_spec(2, 2))
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(2)]
    assert all(st.is_native for st in stages)
    loss_fn = lambda out, up: (out.float() * up).sum()
    sched = pp.Schedule1F1B(stages, M, loss_fn=loss_fn)
    out = sched.step(ids.to(DEV), target=upstream.to(DEV), losses=[])
    import torch.nn as nn
    ref_stages = [nn.Sequential(ref.embed, ref.h[0]), nn.Sequential(ref.h[1])]
    ref_out, _ = OP.step(ref_stages, ids, upstream, M, loss_fn)
    assert_close_rel(out, ref_out, BF16_TOL, "output")
    named = dict(model.named_parameters())
    for name, rp in ref.named_parameters():
        if rp.grad is None:
            continue
        err = max_rel(named[name].main_grad, rp.grad)
        assert err <= BF16_TOL, f"grad of {name}: max relative error {err:.3e}"


def test_the_flow_of_the_reference_gpt2_example():
    """examples/huggingface/pippy_gpt2.py:20-77 with the package's names: GPT2ForSequenceClassification in
    eval mode, the microbatch given by keyword (``mb_kwargs``), ``pipe.build_stage``, ``ScheduleGPipe`` and
    ``schedule.step(**inputs)``.  The decoder stage runs as launch lists; the last stage, which picks the
    last token's scores out of the sequence, runs through torch; the result is the model's."""
    transformers = pytest.importorskip("transformers")
    from pippy_amd import ScheduleGPipe, SplitPoint, pipeline
    config = transformers.GPT2Config(n_embd=128, n_layer=4, n_head=2, n_positions=256, vocab_size=1000,
                                     attn_pdrop=0.0, embd_pdrop=0.0, resid_pdrop=0.0, use_cache=False)
    torch.manual_seed(0)
    gpt2 = transformers.GPT2ForSequenceClassification(config).to(torch.bfloat16)
    gpt2.eval()
    chunks, batch, seq, world = 4, 4, 256, 2
    mb_inputs = {"input_ids": torch.randint(0, 1000, (batch // chunks, seq))}
    split_spec = {f"transformer.h.{i * 2}": SplitPoint.BEGINNING for i in range(1, world)}
    pipe = pipeline(gpt2, mb_args=(), mb_kwargs=mb_inputs, split_spec=split_spec)
    assert pipe.num_stages == world
    stages = [pipe.build_stage(r, device=DEV) for r in range(world)]
    assert stages[0].is_native and not stages[1].is_native
    schedule = ScheduleGPipe(stages, chunks)
    inputs = {"input_ids": torch.randint(0, 1000, (batch, seq), device=DEV)}
    with torch.no_grad():
        out = schedule.step(**inputs)
        ref = torch.cat([copy.deepcopy(gpt2).float()(input_ids=inputs["input_ids"][i:i + 1]).logits
                         for i in range(batch)])
    out = out[0] if isinstance(out, (tuple, list)) else out
    assert_close_rel(out, ref, BF16_TOL, "classification scores")


def test_hugging_face_vit_runs_its_encoder_stage_natively_between_two_torch_stages():
    """transformers.ViTForImageClassification in three stages: the patch embedding (a convolution, the class
    token) and the classifier head (the class token's row) run through torch autograd, the stage of plain
    encoder layers between them as launch lists over 65 tokens (attention without a mask, padded to 128
    keys inside the layer).  Activations and gradients cross both kinds of boundary."""
    transformers = pytest.importorskip("transformers")
    import pippy_amd as pp
    cfg = transformers.ViTConfig(hidden_size=128, num_hidden_layers=6, num_attention_heads=2, intermediate_size=512,
                                 image_size=64, patch_size=8, hidden_dropout_prob=0.0,
                                 attention_probs_dropout_prob=0.0, num_labels=10)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.ViTForImageClassification(cfg).to(torch.bfloat16)
    ref = copy.deepcopy(model).float()
    ref16 = copy.deepcopy(model)
    M, mb = 4, 2
    images = torch.randn(mb * M, 3, 64, 64)
    labels = torch.randint(0, 10, (mb * M,))
    pipe = pp.pipeline(model, mb_args=(images[:mb].to(torch.bfloat16),),
                       split_spec={"vit.layers.2": pp.SplitPoint.BEGINNING, "vit.layers.4": pp.SplitPoint.BEGINNING})
    stages = [pp.PipelineStage(pipe, i, DEV) for i in range(3)]
    assert [st.is_native for st in stages] == [False, True, False], [st.eager_reason for st in stages]
    loss_fn = lambda out, tgt: torch.nn.functional.cross_entropy((out[0] if isinstance(out, tuple) else out).float(), tgt)
    sched = pp.Schedule1F1B(stages, M, loss_fn=loss_fn)
    losses = []
    out = sched.step(images.to(DEV, torch.bfloat16), target=labels.to(DEV), losses=losses)
    out = out[0] if isinstance(out, (tuple, list)) else out
    ref_losses = []
    for x, t in zip(images.chunk(M), labels.chunk(M)):
        logits = ref(x).logits
        ref_losses.append(torch.nn.functional.cross_entropy(logits, t))
        ref_losses[-1].backward()
    assert_close_rel(out, ref(images).logits.detach(), BF16_TOL, "class scores")
    for m in range(M):
        assert_close_rel(losses[m].reshape(1), ref_losses[m].detach().reshape(1), BF16_TOL, f"loss {m}")
    stages[1].materialize_grads()
    named = dict(model.named_parameters())

    class _Grad:                      # check_gradients reads .main_grad; the torch stages only hold .grad
        def __init__(self, p):
            self.main_grad = p.grad

    def run_in_bf16():
        for x, t in zip(images.to(torch.bfloat16).chunk(M), labels.chunk(M)):
            torch.nn.functional.cross_entropy(ref16(x).logits.float(), t).backward()
        return dict(ref16.named_parameters())

    for name in named:
        assert named[name].grad is not None, name
    check_gradients({n: _Grad(p) for n, p in named.items()}, dict(ref.named_parameters()), run_in_bf16,
                    "ViT between two torch stages", note)


# ---- the weight-gradient passes of a step as one batched pass ----------------------------------------
def _grads_after_steps(sched_cls, batch, steps, n_stages=2, fused=False, zero_between=True):
    import pippy_amd as pp
    M = 4
    model, ref, stages, ref_stages, ids = _build_decoder(n_stages, M=M, fused=fused)
    torch.manual_seed(123)
    target = torch.randint(0, 1000, ids.shape)
    sched = sched_cls(stages, M, loss_fn=pp.CrossEntropyLoss())
    sched.batch_weight_grads = batch
    for step in range(steps):
        if zero_between or step == 0:
            sched.zero_grad()
        losses = []
        sched.step(ids.to(DEV), target=target.to(DEV), losses=losses)
    torch.cuda.synchronize()
    n_batched = [st._program.batched_w(tuple(range(M))).n_batched if st.batch_weight_grads else 0 for st in stages]
    return {n: p.main_grad.clone() for n, p in model.named_parameters()}, [l.clone() for l in losses], n_batched


@pytest.mark.parametrize("schedule", ["1f1b", "gpipe", "zero_bubble", "interleaved"])
@pytest.mark.parametrize("fused", [False, True])
def test_weight_gradients_in_one_batched_pass_leave_the_bits_of_one_pass_per_microbatch(schedule, fused):
    """With ``schedule.batch_weight_grads`` every weight-gradient GEMM of a stage runs once per step over all
    microbatches, a tile adding the microbatches' (rounded) products to its running sum in ascending order:
    the fp32 accumulators must hold the bits that one accumulating pass per microbatch leaves, after one
    step from cleared gradients and after a second step that keeps accumulating (the sums then start from
    what the accumulators hold)."""
    import pippy_amd as pp
    cls = {"1f1b": pp.Schedule1F1B, "gpipe": pp.ScheduleGPipe, "zero_bubble": pp.ScheduleZeroBubble,
           "interleaved": pp.ScheduleInterleaved1F1B}[schedule]
    for steps, zero_between in ((1, True), (2, False)):
        got, losses_b, n_batched = _grads_after_steps(cls, True, steps, fused=fused, zero_between=zero_between)
        want, losses_p, none = _grads_after_steps(cls, False, steps, fused=fused, zero_between=zero_between)
        assert all(n >= 4 for n in n_batched) and not any(none), (n_batched, none)   # the GEMMs of a layer, at least
        for a, b in zip(losses_b, losses_p):
            assert torch.equal(a, b)
        for name in want:
            assert torch.equal(got[name], want[name]), f"{schedule}, {steps} step(s): grad of {name}"


@pytest.mark.parametrize("schedule", ["1f1b", "zero_bubble"])
def test_a_schedules_only_stage_batches_its_weight_gradients_by_default(schedule):
    """A schedule that drives one launch-list stage has no other stage's kernels to run beside that stage's
    weight-gradient launches: left to itself it forms them in one pass per step, with the bits of one pass per
    microbatch."""
    import pippy_amd as pp
    cls = {"1f1b": pp.Schedule1F1B, "zero_bubble": pp.ScheduleZeroBubble}[schedule]
    got, losses_b, n_batched = _grads_after_steps(cls, None, 1, n_stages=1)
    want, losses_p, none = _grads_after_steps(cls, False, 1, n_stages=1)
    assert n_batched[0] >= 4 and not any(none), (n_batched, none)
    for a, b in zip(losses_b, losses_p):
        assert torch.equal(a, b)
    for name in want:
        assert torch.equal(got[name], want[name]), f"grad of {name}"


def test_expert_stages_batch_their_weight_gradients_by_default():
    """Left to itself (``batch_weight_grads = None``) a schedule batches where it pays: stages with expert
    weights, under any schedule; dense stages that share the device keep one weight-gradient pass per
    microbatch."""
    import pippy_amd as pp
    from pippy_amd.configs import MoEDecoderLM, equal_split_spec
    M = 4
    model, ref, stages, ref_stages, ids = _build_decoder(2, M=M)
    target = torch.randint(0, 1000, ids.shape)
    plain = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
    plain.step(ids.to(DEV), target=target.to(DEV))
    assert not any(st.batch_weight_grads for st in stages)

    def moe_grads(batch):
        torch.manual_seed(0)
        S, vocab, L = 128, 512, 4
        moe = MoEDecoderLM(vocab=vocab, dim=128, n_layers=L, n_heads=2, ffn=256, n_experts=8)
        mids = torch.randint(0, vocab, (2 * M, S))
        mtarget = torch.randint(0, vocab, (2 * M, S))
        pipe = pp.pipeline(moe, M, (mids,), split_spec=equal_split_spec(L, 2))
        mstages = [pp.PipelineStage(pipe, i, DEV, group=1) for i in range(2)]
        sched = pp.ScheduleInterleaved1F1B(mstages, M, loss_fn=pp.CrossEntropyLoss())
        sched.batch_weight_grads = batch
        sched.step(mids.to(DEV), target=mtarget.to(DEV))
        torch.cuda.synchronize()
        return {n: p.main_grad.clone() for n, p in moe.named_parameters()}, [st.batch_weight_grads for st in mstages]

    auto, flags = moe_grads(None)
    assert all(flags)
    per_microbatch, flags = moe_grads(False)
    assert not any(flags)
    for name in auto:
        assert torch.equal(auto[name], per_microbatch[name]), f"grad of {name}"
