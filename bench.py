#!/usr/bin/env python3
"""Throughput of the pipeline-stage hot path on one MI355X.

Workload (the training configuration the headline metric is quoted on): a
GPT-2-small-shaped decoder (12 layers, d_model 768, 12 heads, FFN 3072, tanh-GELU, pre-LayerNorm,
causal attention, vocabulary 50257, sequence 1024) cut into 4 virtual stages of 3 layers on one
GPU, trained with Schedule1F1B over a batch of 32 split into 8 microbatches of 4; bf16 weights and
activations, fp32 gradient accumulation; synthetic tokens, random-initialised weights.

One "step" is one ``schedule.step()``: microbatch split, 32 stage forwards, 8 cross-entropy
losses, 32 stage backwards (input- and weight-gradient passes), fp32 gradient accumulation and
the merge of the 8 logits chunks.  Inputs are resident in HBM before the timed region.

Prints one JSON line: tokens/s, the MFMA roofline of the dominant kernel (the bf16 GEMM, timed
per launch with HIP events on its own stream in a second, instrumented pass over the same steps)
and the CPU baseline (the reference's own CPU path restated: one gloo process per stage, same schedule,
on this box's cores, run before the GPU is touched).
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
# Bytes between the L2 caches and the fabric per GEMM launch, averaged over the GEMM launches of one
# step of the default workload: rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by what the same
# counter reads for the logits merge, a copy of known size.  A counter run cannot be made from inside
# this script: the figure is read from the tracked summary of the last such run and reported, with the
# file it came from, for the default workload only.
GEMM_TRAFFIC_FILE = os.path.join("profiles", "gemm_gpt2small_1f1b_hbm_traffic.json")


def gemm_traffic():
    """(bytes per launch or None, where the figure comes from)."""
    try:
        with open(os.path.join(ROOT, GEMM_TRAFFIC_FILE)) as f:
            return float(json.load(f)["gemm_traffic_bytes_per_launch"]), GEMM_TRAFFIC_FILE
    except (OSError, KeyError, ValueError):
        return None, None


def build(args):
    """Model, schedule, stages and the step's inputs for the chosen workload."""
    import pippy_amd as pp
    from pippy_amd.configs import DecoderLM, equal_split_spec
    torch.manual_seed(0)
    if args.workload != "gpt2":
        return build_other(args)
    model = DecoderLM(vocab=args.vocab, max_seq=args.seq, dim=args.dim, n_layers=args.layers,
                      n_heads=args.heads, ffn=args.ffn)
    ids = torch.randint(0, args.vocab, (args.batch, args.seq))
    target = torch.randint(0, args.vocab, (args.batch, args.seq))
    pipe = pp.pipeline(model, args.microbatches, (ids,),
                       split_spec=equal_split_spec(args.layers, args.stages))
    stages = [pp.PipelineStage(pipe, i, "cuda", fused_accumulate=args.fused_accumulate)
              for i in range(args.stages)]
    sched_cls = {"1f1b": pp.Schedule1F1B, "gpipe": pp.ScheduleGPipe,
                 "zero_bubble": pp.ScheduleZeroBubble}[args.schedule]
    sched = sched_cls(stages, args.microbatches, loss_fn=pp.CrossEntropyLoss())
    return model, sched, stages, ids.cuda(), target.cuda()


def _upstream_loss(out, upstream):
    """A loss whose gradient w.r.t. the stage output is `upstream` (what a middle stage receives)."""
    return (out.float() * upstream).sum()


def build_other(args):
    """The other baseline configurations at full size (each sets its own shape; the --vocab ... --stages
    options only shape the default workload).  Sets args.describe / args.tokens / args.flops."""
    import pippy_amd as pp
    from pippy_amd.configs import bert_base, equal_split_spec, llama2_7b_stage, mixtral_style
    if args.workload == "bert":
        # BERT-base-shaped encoder, inference, GPipe: batch 64 x 512 in 8 microbatches, 4 stages
        model = bert_base()
        ids = torch.randint(0, 30522, (64, 512))
        pipe = pp.pipeline(model, 8, (ids,), split_spec=equal_split_spec(12, 4))
        stages = [pp.PipelineStage(pipe, i, "cuda") for i in range(4)]
        sched = pp.ScheduleGPipe(stages, 8)
        args.tokens, args.training = ids.numel(), False
        per_token = 12 * (2 * 768 * 3 * 768 + 2 * 768 * 768 + 4 * 768 * 3072 + 4 * 512 * 768)
        args.flops = float(per_token) * ids.numel()
        args.describe = ("BERT-base-shaped encoder (12 post-LayerNorm layers, hidden 768, 12 heads, FFN 3072, "
                         "vocab 30522, seq 512), inference, 4 virtual stages on one GPU, schedule gpipe, "
                         "batch 64 in 8 microbatches, bf16")
        args.batch, args.seq = 64, 512
        return model, sched, stages, ids.cuda(), None
    if args.workload == "llama":
        # one stage of a Llama-2-7B-shaped PP=4 pipeline, zero-bubble: 16 microbatches of one sequence
        M = 16
        with torch.device("cuda"):
            model = llama2_7b_stage()
            x = torch.randn(M, 2048, 4096).to(torch.bfloat16)
            upstream = torch.randn(M, 2048, 4096) * 1e-2
        stage = pp.ManualPipelineStage(model, 0, 1, "cuda", M, input_args=(x[:1],),
                                       fused_accumulate=args.fused_accumulate)
        sched = pp.ScheduleZeroBubble([stage], M, loss_fn=_upstream_loss)
        T = M * 2048
        per_layer = 4 * 4096 ** 2 + 3 * 4096 * 11008
        args.tokens, args.training = T, True
        args.flops = 3.0 * (2.0 * T * per_layer * 8 + 8 * 4.0 * T * 2048 * 4096)
        args.describe = ("one stage (8 layers) of a Llama-2-7B-shaped pipeline (d_model 4096, 32 heads of 128, "
                         "SwiGLU 11008, RMSNorm, RoPE, seq 2048), zero-bubble schedule with separate dI and dW "
                         "passes, 16 microbatches of one sequence, upstream gradients N(0, 1e-2), bf16 with fp32 "
                         f"gradient accumulation ({args.accumulate_text})")
        args.batch, args.seq = M, 2048
        return model, sched, [stage], x, upstream
    if args.workload == "moe":
        # Mixtral-style MoE, interleaved 1F1B: 2 virtual stages of 4 layers on one rank
        with torch.device("cuda"):
            model = mixtral_style()
        ids = torch.randint(0, 32000, (16, 1024))
        target = torch.randint(0, 32000, (16, 1024))
        pipe = pp.pipeline(model, 8, (ids,), split_spec=equal_split_spec(8, 2))
        stages = [pp.PipelineStage(pipe, i, "cuda", group=1, fused_accumulate=args.fused_accumulate)
                  for i in range(2)]
        sched = pp.ScheduleInterleaved1F1B(stages, 8, loss_fn=pp.CrossEntropyLoss())
        T = ids.numel()
        active = 4 * 1024 ** 2 + 2 * 3 * 1024 * 4096 + 8 * 1024   # attention, two experts, router
        args.tokens, args.training = T, True
        args.flops = 3.0 * (2.0 * T * (active * 8 + 1024 * 32000) + 8 * 4.0 * T * 1024 * 1024)
        args.describe = ("Mixtral-style decoder (8 layers in 2 virtual stages, d_model 1024, 16 heads, 8 experts "
                         "with SwiGLU 4096, top-2 router, vocab 32000, seq 1024), schedule interleaved 1f1b on one "
                         "rank, batch 16 in 8 microbatches, bf16 with fp32 gradient accumulation "
                         f"({args.accumulate_text})")
        args.batch, args.seq = 16, 1024
        return model, sched, stages, ids.cuda(), target.cuda()
    if args.workload == "hf_gpt2":
        # the headline configuration on the model class of the reference's example itself:
        # transformers.GPT2LMHeadModel (GPT-2 small, random weights, embeddings untied), cut by the front
        # end's torch.export route and run as launch lists on the model's own Conv1D parameters
        import transformers
        cfg = transformers.GPT2Config(attn_pdrop=0.0, embd_pdrop=0.0, resid_pdrop=0.0, use_cache=False,
                                      tie_word_embeddings=False)
        cfg._attn_implementation = "sdpa"
        model = transformers.GPT2LMHeadModel(cfg).to(torch.bfloat16)
        M, B, S = 8, 32, 1024
        ids = torch.randint(0, cfg.vocab_size, (B, S))
        target = torch.randint(0, cfg.vocab_size, (B, S))
        pipe = pp.pipeline(model, mb_args=(ids[:B // M],),
                           split_spec={f"transformer.h.{i}": pp.SplitPoint.BEGINNING for i in (3, 6, 9)})
        stages = [pp.PipelineStage(pipe, i, "cuda", fused_accumulate=args.fused_accumulate) for i in range(4)]
        eager = [st.eager_reason for st in stages if not st.is_native]
        if eager:
            raise RuntimeError(f"a stage of the Hugging Face model did not lower: {eager}")
        sched = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
        args.tokens, args.training = B * S, True
        args.batch, args.seq = B, S
        args.vocab, args.dim, args.layers, args.heads, args.ffn = cfg.vocab_size, 768, 12, 12, 3072
        args.flops = flops_per_step(args)
        args.describe = ("transformers.GPT2LMHeadModel (GPT-2 small: 12 layers, d_model 768, 12 heads, FFN 3072, "
                         "vocab 50257, seq 1024; random weights, embeddings untied), exported and cut by "
                         "pipeline(), 4 virtual stages on one GPU, schedule 1f1b, batch 32 in 8 microbatches, "
                         f"bf16 with fp32 gradient accumulation ({args.accumulate_text})")
        return model, sched, stages, ids.cuda(), target.cuda()
    if args.workload == "hf_bert":
        # the BERT-base inference configuration on transformers.BertModel itself
        import transformers
        cfg = transformers.BertConfig(hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0)
        cfg._attn_implementation = "sdpa"
        model = transformers.BertModel(cfg, add_pooling_layer=False).to(torch.bfloat16).eval()
        ids = torch.randint(0, cfg.vocab_size, (64, 512))
        pipe = pp.pipeline(model, mb_args=(ids[:8],),
                           split_spec={f"encoder.layer.{i}": pp.SplitPoint.BEGINNING for i in (3, 6, 9)})
        stages = [pp.PipelineStage(pipe, i, "cuda") for i in range(4)]
        eager = [st.eager_reason for st in stages if not st.is_native]
        if eager:
            raise RuntimeError(f"a stage of the Hugging Face model did not lower: {eager}")
        sched = pp.ScheduleGPipe(stages, 8)
        args.tokens, args.training = ids.numel(), False
        per_token = 12 * (2 * 768 * 3 * 768 + 2 * 768 * 768 + 4 * 768 * 3072 + 4 * 512 * 768)
        args.flops = float(per_token) * ids.numel()
        args.describe = ("transformers.BertModel (BERT-base: 12 post-LayerNorm layers, hidden 768, 12 heads, FFN "
                         "3072, vocab 30522, seq 512; random weights), exported and cut by pipeline(), inference, "
                         "4 virtual stages on one GPU, schedule gpipe, batch 64 in 8 microbatches, bf16")
        args.batch, args.seq = 64, 512
        return model, sched, stages, ids.cuda(), None
    raise ValueError(args.workload)


def flops_per_step(args):
    """Algorithmic FLOPs of one training step: matmul 2mnk, attention dense, backward 2x forward."""
    T = args.batch * args.seq
    d, f, V, L, S = args.dim, args.ffn, args.vocab, args.layers, args.seq
    per_token_fwd = L * (2 * d * 3 * d + 2 * d * d + 2 * 2 * d * f + 4 * S * d) + 2 * d * V
    return 3.0 * per_token_fwd * T


def cpu_baseline(args, budget_seconds=120.0):
    """The reference's own way of running this workload on host cores (its tests: backend gloo, one
    process per stage, ``test/test_fwd.py:117-129``), restated in ``oracle/gloo_pipeline.py``: S fresh
    CPU-only child processes over gloo on 127.0.0.1, each running its rank's program of the same 1F1B
    schedule on its stage of the same model, ``cores // S`` threads each, in the arithmetic of the
    configuration (bf16 parameters, activations and gradients).  One warm-up microbatch through the
    whole pipeline, one untimed warm-up step, then three timed steps whose median is reported; if the
    warm-up microbatch says that this would overrun the budget, one timed step (or the first half,
    quarter ... of its microbatches) without the warm-up step, and ``sample`` says so.
    Must be called before this process touches the GPU: the children are started from a parent that
    holds no GPU state."""
    import socket
    import subprocess
    cores = torch.get_num_threads()
    S = args.stages
    threads = max(1, cores // S)
    with socket.socket() as sock:
        sock.bind(("127.0.0.1", 0))
        port = sock.getsockname()[1]
    env = dict(os.environ, MASTER_ADDR="127.0.0.1", MASTER_PORT=str(port), OMP_NUM_THREADS=str(threads),
               HIP_VISIBLE_DEVICES="", CUDA_VISIBLE_DEVICES="")
    common = ["--world", str(S), "--threads", str(threads), "--dtype", "bf16", "--vocab", str(args.vocab),
              "--seq", str(args.seq), "--dim", str(args.dim), "--layers", str(args.layers), "--heads",
              str(args.heads), "--ffn", str(args.ffn), "--batch", str(args.batch), "--microbatches",
              str(args.microbatches), "--budget-seconds", str(budget_seconds)]
    procs = [subprocess.Popen([sys.executable, "-m", "oracle.gloo_pipeline", "--rank", str(r)] + common, cwd=ROOT,
                              env=env, stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True)
             for r in range(S)]
    try:
        out0, _ = procs[0].communicate(timeout=420)
        for p in procs[1:]:
            p.wait(timeout=60)
    except subprocess.TimeoutExpired:
        for p in procs:
            p.kill()
        return {"value": None, "unit": "tokens/s", "cores": cores, "kind": "port",
                "sample": "the CPU pipeline did not finish within 420 s and was stopped"}
    if any(p.returncode for p in procs):
        return {"value": None, "unit": "tokens/s", "cores": cores, "kind": "port",
                "sample": f"a CPU pipeline process failed (exit codes {[p.returncode for p in procs]})"}
    rep = json.loads([ln for ln in out0.splitlines() if ln.startswith("{")][-1])
    n, M = rep["microbatches_timed"], rep["microbatches"]
    k = len(rep["step_times_s"])
    what = (f"median of {k} full steps after {rep['warmup_steps']} warm-up step" if n == M and k > 1 else
            "one full step" if n == M else f"the first {n} of {M} microbatches of one step")
    return {"value": round(rep["tokens"] / rep["step_s"], 1), "unit": "tokens/s", "cores": S * threads,
            "kind": "port", "dtype": "bf16", "processes": S, "threads_per_process": threads,
            "sample": f"{what} ({rep['tokens']} tokens) of the same workload: {S} CPU processes over gloo, one "
                      f"per stage, 1F1B, bf16, after a warm-up of {rep['warmup_microbatches']} microbatch "
                      f"({rep['warmup_s']:.1f} s); timed steps "
                      f"{', '.join(f'{t:.1f}' for t in rep['step_times_s'])} s"}


GEMM_SHAPES = (
    # (M, N, K, a_trans, b_trans, what)
    (4096, 768, 768, 0, 0, "gpt2 attention projection"), (4096, 2304, 768, 0, 0, "gpt2 qkv"),
    (4096, 3072, 768, 0, 0, "gpt2 feed-forward up"), (4096, 768, 3072, 0, 0, "gpt2 feed-forward down"),
    (4096, 50304, 768, 0, 0, "gpt2 vocabulary projection"), (4096, 768, 50304, 0, 0, "its input gradient"),
    (3072, 768, 4096, 1, 1, "gpt2 weight gradient (dY^T X over 4096 tokens)"),
    (4096, 4096, 1024, 0, 0, "mid-sized"), (2048, 4096, 4096, 0, 0, "llama attention projection"),
    (2048, 12288, 4096, 0, 0, "llama qkv"), (2048, 11008, 4096, 0, 0, "llama gate / up"),
    (2048, 4096, 11008, 0, 0, "llama down"), (11008, 4096, 2048, 1, 1, "llama weight gradient"),
    (8192, 8192, 8192, 0, 0, "large square"),
)


ATTENTION_SHAPES = (
    # (batch, heads, seq, head_dim, causal, what)
    (4, 12, 1024, 64, True, "gpt2 layer, one microbatch"),
    (8, 12, 512, 64, False, "bert layer, one microbatch"),
    (1, 32, 2048, 128, True, "llama layer, one sequence"),
    (2, 16, 1024, 64, True, "mixtral-style layer, one microbatch"),
)


def attention_shapes():
    """One JSON line per shape: the library's attention forward / backward and torch's
    scaled_dot_product_attention (each of its fused backends that runs) on the same operands, timed with
    events over back-to-back launches."""
    import torch.nn.functional as F
    from torch.nn.attention import SDPBackend, sdpa_kernel
    from pippy_amd import _native as N
    N.lib()
    torch.manual_seed(0)

    def timed(fn, n=50):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e3

    for B, H, S, D, causal, what in ATTENTION_SHAPES:
        qkv = torch.randn(B, S, 3 * H * D, device="cuda").to(torch.bfloat16)
        o = torch.empty(B, S, H * D, device="cuda", dtype=torch.bfloat16)
        lse, delta = torch.empty(B, H, S, device="cuda"), torch.empty(B, H, S, device="cuda")
        d_o, dqkv = torch.randn_like(o), torch.empty_like(qkv)
        fwd = timed(lambda: N.attn_fwd(qkv, o, lse, H, causal))
        bwd = timed(lambda: N.attn_bwd(qkv, o, lse, d_o, dqkv, delta, H, causal))
        q, k, v = (t.reshape(B, S, H, D).transpose(1, 2).contiguous().requires_grad_(True)
                   for t in qkv.split(H * D, -1))
        flops = 4.0 * B * H * S * S * D
        row = {"shape": [B, H, S, D], "causal": causal, "what": what, "fwd_us": round(fwd, 1),
               "bwd_us": round(bwd, 1), "fwd_tflops_dense_count": round(flops / fwd / 1e6, 1),
               "bwd_tflops_dense_count": round(2.5 * flops / bwd / 1e6, 1)}
        for name, backend in (("flash", SDPBackend.FLASH_ATTENTION), ("efficient", SDPBackend.EFFICIENT_ATTENTION)):
            try:
                with sdpa_kernel(backend):
                    call = lambda: F.scaled_dot_product_attention(q, k, v, is_causal=causal)
                    g = torch.randn_like(call())
                    f_us = timed(call)
                    fb_us = timed(lambda: torch.autograd.grad(call(), (q, k, v), g))
                row[f"torch_sdpa_{name}_fwd_us"] = round(f_us, 1)
                row[f"torch_sdpa_{name}_bwd_us"] = round(fb_us - f_us, 1)
            except Exception as e:   # a backend that does not take the shape
                row[f"torch_sdpa_{name}"] = f"{type(e).__name__}: {str(e)[:80]}"
        print(json.dumps(row), flush=True)


def rowwise_shapes():
    """One JSON line per kernel: the library's LayerNorm forward / input gradient and cross entropy
    (loss + gradient) at the headline shapes, and torch's own operators on the same values."""
    import torch.nn.functional as F
    from pippy_amd import _native as N
    N.lib()
    torch.manual_seed(0)

    def timed(fn, n=50):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e3

    T, Cc, V = 4096, 768, 50257
    bf = dict(device="cuda", dtype=torch.bfloat16)
    x, dy = torch.randn(T, Cc, **bf), torch.randn(T, Cc, **bf)
    gamma, beta = torch.randn(Cc, **bf), torch.randn(Cc, **bf)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    mean, rstd = torch.empty(T, device="cuda"), torch.empty(T, device="cuda")
    ours = timed(lambda: N.layernorm_fwd(x, gamma, beta, y, mean, rstd, 1e-5))
    theirs = timed(lambda: F.layer_norm(x, (Cc,), gamma, beta, 1e-5))
    print(json.dumps({"kernel": "layernorm forward", "shape": [T, Cc], "us": round(ours, 1),
                      "GB/s": round(4.0 * T * Cc / ours / 1e3, 1), "torch_us": round(theirs, 1)}), flush=True)
    ours = timed(lambda: N.layernorm_bwd_input(dy, x, gamma, mean, rstd, None, dx))
    xr = x.clone().requires_grad_(True)
    out = F.layer_norm(xr, (Cc,), gamma, beta, 1e-5)
    theirs = timed(lambda: torch.autograd.grad(out, xr, dy, retain_graph=True))
    print(json.dumps({"kernel": "layernorm input gradient", "shape": [T, Cc], "us": round(ours, 1),
                      "GB/s": round(6.0 * T * Cc / ours / 1e3, 1), "torch_us": round(theirs, 1),
                      "note": "torch's backward also forms the weight and bias gradients here"}), flush=True)
    Vp = (V + 127) // 128 * 128
    logits = torch.randn(T, Vp, **bf)
    dlogits = torch.empty_like(logits)
    target = torch.randint(0, V, (T,), device="cuda")
    loss, ws = torch.empty(1, device="cuda"), torch.empty(T + 2, device="cuda")
    ours = timed(lambda: N.ce_loss(logits, target, loss, dlogits, ws, V), n=20)
    lr = logits[:, :V].clone().requires_grad_(True)

    def torch_ce():
        torch.autograd.grad(F.cross_entropy(lr.float(), target), lr)

    theirs = timed(torch_ce, n=20)
    print(json.dumps({"kernel": "cross entropy, loss and gradient", "shape": [T, V], "us": round(ours, 1),
                      "GB/s": round(4.0 * T * V / ours / 1e3, 1), "torch_us": round(theirs, 1),
                      "note": "torch: F.cross_entropy on the fp32 cast of the bf16 logits, and its backward"}),
          flush=True)


def gemm_shapes():
    """One JSON line per shape: the library's GEMM and torch.matmul on the same operands, each timed over
    rotating operand sets (so that operands are not L2-resident from the previous launch)."""
    from pippy_amd import _native as N
    from pippy_amd._program import splitk_copies
    N.lib()
    dev = torch.device("cuda:0")
    torch.manual_seed(0)

    def timed(fns, flops):
        for f in fns:
            f()
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = max(2, min(200, int(2e12 / flops)))   # a few milliseconds of work
        ev0.record()
        for _ in range(reps):
            for f in fns:
                f()
        ev1.record()
        torch.cuda.synchronize()
        return ev0.elapsed_time(ev1) * 1e3 / (reps * len(fns))

    for (M, Nn, K, at, bt, what) in GEMM_SHAPES:
        sets = []
        for _ in range(3):
            A = torch.randn((K, M) if at else (M, K), device=dev).to(torch.bfloat16)
            B = (torch.randn((K, Nn) if bt else (Nn, K), device=dev) * 0.05).to(torch.bfloat16)
            sets.append((A, B, torch.empty(M, Nn, device=dev, dtype=torch.bfloat16)))
        flops = 2.0 * M * Nn * K
        # as the stage lowers it: a long reduction into a small output goes through the k-split entry point
        copies = 0 if (at or bt) else splitk_copies(M, Nn, K)
        if copies:
            ws = torch.empty(copies * M * Nn, device=dev)
            ours = [(lambda s=s: N.gemm_bf16_splitk(s[0], s[1], s[2], ws)) for s in sets]
        else:
            ours = [(lambda s=s: N.gemm_bf16(s[0], s[1], s[2], a_trans=bool(at), b_trans=bool(bt))) for s in sets]
        ours_us = timed(ours, flops)
        lib_us = timed([(lambda s=s: torch.matmul(s[0].t() if at else s[0], s[1] if bt else s[1].t(),
                                                           out=s[2])) for s in sets], flops)
        # the per-layer shapes once more as 2 and 4 independent problems in one grouped launch: what the
        # same-shaped GEMMs of several pipeline stages would cost each if the stages ran in lock step
        grouped = {}
        if flops < 3e10 and not copies:
            for k in (2, 4):
                more = [[(torch.randn_like(s[0]), torch.randn_like(s[1]) * 0.05, torch.empty_like(s[2]),
                          dict(a_trans=bool(at), b_trans=bool(bt))) for _ in range(k)] for s in sets]
                us_k = timed([(lambda ps=ps: N.gemm_bf16_grouped(ps)) for ps in more], k * flops)
                grouped[f"grouped{k}_us_each"] = round(us_k / k, 1)
                del more
        print(json.dumps({"shape": [M, Nn, K], "a_trans": at, "b_trans": bt, "what": what, "k_splits": copies,
                          "us": round(ours_us, 1), "tflops": round(flops / ours_us / 1e6, 1),
                          "vendor_us": round(lib_us, 1), "vendor_tflops": round(flops / lib_us / 1e6, 1),
                          **grouped}),
              flush=True)
        del sets


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--schedule", default="1f1b", choices=["1f1b", "gpipe", "zero_bubble"])
    ap.add_argument("--fused-accumulate", action="store_true",
                    help="add the unrounded fp32 sums of the dW GEMMs to the accumulators (default: rounded "
                         "to bf16 first, the bits of a bf16 gradient folded in by the accumulate kernel)")
    ap.add_argument("--staged-accumulate", action="store_true",
                    help="write every gradient to the bf16 staging arena and fold it in with the accumulate "
                         "kernel (the same bits as the default, one more pass over the parameters)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--serial-stages", action="store_true",
                    help="run all virtual stages on one stream instead of two")
    ap.add_argument("--no-roofline", action="store_true")
    ap.add_argument("--batch-weight-grads", default="auto", choices=["auto", "on", "off"],
                    help="one batched weight-gradient pass per stage and step (auto: the schedule's own choice: "
                         "zero-bubble schedules and stages with expert weights)")
    ap.add_argument("--gemm-shapes", action="store_true",
                    help="instead of a step: time the stage GEMM alone on the shapes of the workloads (HIP "
                         "events, cold operands) and torch.matmul (the vendor library) on the same operands beside "
                         "it; one JSON line per shape")
    ap.add_argument("--attention-shapes", action="store_true",
                    help="instead of a step: time the attention kernels alone on the shapes of the workloads, "
                         "torch's scaled_dot_product_attention backends on the same operands beside them, then "
                         "LayerNorm and cross entropy at the headline shapes beside torch's operators; one JSON "
                         "line per shape")
    ap.add_argument("--workload", default="gpt2", choices=["gpt2", "bert", "llama", "moe", "hf_gpt2", "hf_bert"],
                    help="gpt2: the headline configuration (default); bert / llama / moe: the BERT-base "
                         "inference, Llama-2-7B stage (zero-bubble) and Mixtral-style (interleaved 1F1B) "
                         "configurations at full size; hf_gpt2 / hf_bert: the headline and the BERT-base configurations on "
                         "transformers.GPT2LMHeadModel / transformers.BertModel themselves")
    # workload shape (defaults: GPT-2 small, configs[2])
    ap.add_argument("--vocab", type=int, default=50257)
    ap.add_argument("--seq", type=int, default=1024)
    ap.add_argument("--dim", type=int, default=768)
    ap.add_argument("--layers", type=int, default=12)
    ap.add_argument("--heads", type=int, default=12)
    ap.add_argument("--ffn", type=int, default=3072)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--microbatches", type=int, default=8)
    ap.add_argument("--stages", type=int, default=4)
    args = ap.parse_args()
    if args.staged_accumulate:
        args.fused_accumulate = "staged"
    args.accumulate_text = {False: "added in the dW GEMM epilogue, rounded to bf16 first",
                            True: "unrounded sums added in the dW GEMM epilogue",
                            "staged": "staging arena + accumulate kernel"}[args.fused_accumulate]

    if args.gpus != 1:
        print("bench.py: this build runs every pipeline stage as a virtual stage on ONE GPU; "
              "there is no multi-GPU path to measure (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)
    if torch.cuda.device_count() < 1:   # counting devices does not initialise the GPU runtime
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    # the CPU baseline runs first, in child processes started while this process holds no GPU state
    cpu_result = None
    if not args.no_cpu_baseline and args.workload == "gpt2" and not (args.gemm_shapes or args.attention_shapes):
        cpu_result = cpu_baseline(args)

    if args.attention_shapes:
        attention_shapes()
        rowwise_shapes()
        return
    if args.gemm_shapes:
        gemm_shapes()
        return

    from pippy_amd import _native as N
    N.lib()  # fail loudly if the kernel library is missing
    model, sched, stages, ids, target = build(args)
    default_workload = args.workload == "gpt2"
    tokens = ids.numel() if default_workload else args.tokens
    training = True if default_workload else args.training
    sched.concurrent_stages = not args.serial_stages
    if args.batch_weight_grads != "auto":
        sched.batch_weight_grads = args.batch_weight_grads == "on"

    def step():
        losses = []
        if not training:
            return sched.step(ids), losses
        sched.zero_grad()
        out = sched.step(ids, target=target, losses=losses)
        return out, losses

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out, losses = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    value = tokens * args.steps / dt
    loss0 = float(losses[0]) if losses else None

    result = {
        "metric": "tokens/sec per schedule step on 1 MI355X + stage GEMM MFMA util %",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": (f"GPT-2-small-shaped decoder ({args.layers} layers, d_model {args.dim}, "
                                f"{args.heads} heads, FFN {args.ffn}, vocab {args.vocab}, seq {args.seq}), "
                                f"{args.stages} virtual stages on one GPU, schedule {args.schedule}, "
                                f"batch {args.batch} in {args.microbatches} microbatches, bf16 with fp32 "
                                f"gradient accumulation ({args.accumulate_text})")
                               if default_workload else args.describe,
                   "global_batch": args.batch, "seq_len": args.seq},
        "step_tflops": round((flops_per_step(args) if default_workload else args.flops)
                             / (ms_per_step * 1e-3) / 1e12, 1),
        "loss_microbatch0": round(loss0, 4) if loss0 is not None else None,
    }

    if not args.no_roofline:
        # Instrumented pass: the same steps with every launch-list op bracketed by HIP events on
        # its stream.  Kept apart from the timed region above so that event records do not perturb
        # `value`; the kernels, shapes and order are identical.
        # The stages run one after the other here (one stream), so that a launch's duration is its
        # own and not that of kernels of other stages sharing the device with it.
        n_prof = max(1, min(args.steps, 3))
        sched.concurrent_stages = False
        N.profile_start(1 << 17)
        for _ in range(n_prof):
            step()
        torch.cuda.synchronize()
        N.profile_stop()
        sched.concurrent_stages = not args.serial_stages
        ms, work, cnt = N.profile_read(N.OP_GEMM_BF16)
        sms_, swork, scnt = N.profile_read(N.OP_GEMM_SEG)   # expert GEMMs of a mixture-of-experts layer
        ms, work, cnt = ms + sms_, work + swork, cnt + scnt
        bcnt = 0
        for kind in (N.OP_GEMM_KSEG, N.OP_GEMM_SEG_KSEG):   # weight gradients of all microbatches in one launch
            kms, kwork, kcnt = N.profile_read(kind)
            ms, work, cnt, bcnt = ms + kms, work + kwork, cnt + kcnt, bcnt + kcnt
            scnt += kcnt if kind == N.OP_GEMM_SEG_KSEG else 0
        gcnt = sgcnt = 0
        for kind in (N.OP_GEMM_SWIGLU, N.OP_GEMM_DSWIGLU):   # feed-forward GEMMs with SwiGLU in the epilogue
            kms, kwork, kcnt = N.profile_read(kind)
            ms, work, cnt, gcnt = ms + kms, work + kwork, cnt + kcnt, gcnt + kcnt
        for kind in (N.OP_GEMM_SEG_SWIGLU, N.OP_GEMM_SEG_DSWIGLU):   # the same over expert segments
            kms, kwork, kcnt = N.profile_read(kind)
            ms, work, cnt, sgcnt = ms + kms, work + kwork, cnt + kcnt, sgcnt + kcnt
        achieved = work / (ms * 1e-3) / 1e12 if ms > 0 else 0.0
        result["roofline"] = {"bound": "mfma", "achieved": round(achieved, 1), "peak": MFMA_PEAK_TFLOPS,
                              "unit": "TFLOP/s", "frac": round(achieved / MFMA_PEAK_TFLOPS, 4),
                              "traffic": gemm_traffic()[0] if default_workload else None,
                              "traffic_source": gemm_traffic()[1] if default_workload else None,
                              "kernel": "gemm_bf16_dma_kernel + gemm_bf16_dma8_kernel + gemm_bf16_group_kernel + gemm_bf16_splitk_kernel"
                                        + (" + gemm_bf16_seg_rows_kernel + gemm_bf16_seg_k_kernel" if scnt else "")
                                        + (" + gemm_bf16_swiglu_kernel + gemm_bf16_dswiglu_kernel" if gcnt else "")
                                        + (" + gemm_bf16_seg_gated_kernel" if sgcnt else "")
                                        + (" + gemm_bf16_group_kseg_kernel / gemm_bf16_seg_k_multi_kernel" if bcnt else ""),
                              "launches_per_step": cnt // n_prof,
                              "avg_launch_us": round(ms / max(cnt, 1) * 1e3, 2),
                              "gemm_ms_per_step": round(ms / n_prof, 3)}
        hbm = {}
        # with the default accumulation the in-step accumulate launches only cover the small
        # tensors (biases, LayerNorm): the kernel's bandwidth is measured at arena size below
        accum_rows = (("grad_accumulate", N.OP_ACCUM_BF16),) if args.fused_accumulate == "staged" else ()
        for name, kind in accum_rows + (("cross_entropy", N.OP_CE_LOSS),
                           ("layernorm_fwd", N.OP_LN_FWD), ("layernorm_bwd_input", N.OP_LN_BWD_INPUT)):
            kms, kwork, kcnt = N.profile_read(kind)
            if kcnt:
                gbs = kwork / (kms * 1e-3) / 1e9
                hbm[name] = {"achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": round(gbs / HBM_PEAK_GBS, 4), "ms_per_step": round(kms / n_prof, 3)}
        for name, kind in (("attention_fwd", N.OP_ATTN_FWD), ("attention_bwd", N.OP_ATTN_BWD)):
            kms, kwork, kcnt = N.profile_read(kind)
            if kcnt:
                tf = kwork / (kms * 1e-3) / 1e12
                hbm[name] = {"achieved": round(tf, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s (dense count)",
                             "frac": round(tf / MFMA_PEAK_TFLOPS, 4), "ms_per_step": round(kms / n_prof, 3)}
        if not default_workload:
            result["other_kernels"] = hbm
            print(json.dumps(result))
            return
        # the merge of the logits chunks runs outside the launch lists: time it alone
        from pippy_amd.microbatch import merge_chunks
        chunks = stages[-1].output_chunks
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        merge_chunks(chunks, None)
        ev0.record()
        for _ in range(5):
            merged = merge_chunks(chunks, None)
        ev1.record()
        torch.cuda.synchronize()
        mms = ev0.elapsed_time(ev1) / 5
        mbytes = 2.0 * merged.numel() * merged.element_size()
        hbm["merge"] = {"achieved": round(mbytes / (mms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": round(mbytes / (mms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "ms_per_step": round(mms, 3)}
        # the split kernel at a size that shows its bandwidth: the step's own split moves 0.5 MB of
        # token ids (and a split along dim 0 of a contiguous tensor is a set of views), so the merged
        # logits are split along the sequence dimension, which copies every chunk
        from pippy_amd.microbatch import TensorChunkSpec, split_args_kwargs_into_chunks
        spec = (TensorChunkSpec(1),)
        split_args_kwargs_into_chunks((merged,), None, args.microbatches, spec)
        ev0.record()
        for _ in range(5):
            split_args_kwargs_into_chunks((merged,), None, args.microbatches, spec)
        ev1.record()
        torch.cuda.synchronize()
        sms = ev0.elapsed_time(ev1) / 5
        hbm["split_logits_sized"] = {"achieved": round(mbytes / (sms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                                     "unit": "GB/s", "frac": round(mbytes / (sms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                     "ms": round(sms, 3),
                                     "note": "8-way split of the merged logits along dim 1; not part of the "
                                             "step, whose own split is 0.5 MB of token ids"}
        del merged
        # the accumulate kernel over a whole stage arena (what a staged weight-gradient pass runs)
        arena = max((st.param_arena() for st in stages), key=lambda a: a.total)
        acc_t, g_t = torch.zeros_like(arena.acc), torch.zeros_like(arena.staging)
        N.grad_accum(acc_t, g_t, init=False)
        ev0.record()
        for _ in range(5):
            N.grad_accum(acc_t, g_t, init=False)
        ev1.record()
        torch.cuda.synchronize()
        ams = ev0.elapsed_time(ev1) / 5
        abytes = 10.0 * acc_t.numel()
        hbm["grad_accumulate_arena_sized"] = {
            "achieved": round(abytes / (ams * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(abytes / (ams * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "ms": round(ams, 3),
            "note": f"pp_grad_accum_f32_bf16 over {acc_t.numel()} elements (the largest stage's arena), 10 B per "
                    "element; in the step the weight gradients are accumulated by their GEMM's epilogue unless "
                    "--staged-accumulate"}
        del acc_t, g_t
        # the optimizer step that follows schedule.step() in training: timed alone, outside `value`
        import pippy_amd as pp
        opt = pp.FusedAdamW(stages, lr=1e-4, weight_decay=0.1)
        opt.step()
        ev0.record()
        for _ in range(5):
            opt.step()
        ev1.record()
        torch.cuda.synchronize()
        oms = ev0.elapsed_time(ev1) / 5
        obytes = sum(a.total for a in (st.param_arena() for st in stages)) * 24.0  # g 4, m 8, v 8, bf16 p 4
        hbm["adamw_step"] = {"achieved": round(obytes / (oms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": round(obytes / (oms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "ms_per_step": round(oms, 3)}
        result["other_kernels"] = hbm

    if cpu_result is not None:
        result["cpu_baseline"] = cpu_result

    print(json.dumps(result))


if __name__ == "__main__":
    main()
