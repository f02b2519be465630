"""Pins the block definitions and the oracle's rotary embedding to an implementation outside this
repository: Hugging Face ``transformers`` (importable in the build container; no download, random
weights copied over).  What is pinned is configuration fidelity: layer order, ``gelu_new``, the
q|k|v layout of the fused projection, rotate-half RoPE and its frequency table, the Mixtral routing
(softmax over all experts, top-2, renormalised).  CPU only, fp32; never runs with ``-m gpu``.
"""
import pytest
import torch

transformers = pytest.importorskip("transformers")

from oracle import ops as OO  # noqa: E402
from pippy_amd import stage_modules as SM  # noqa: E402

TOL = 2e-5


def _close(a, b, what):
    err = (a - b).abs().max().item() / max(b.abs().max().item(), 1e-30)
    assert err <= TOL, f"{what}: max relative error {err:.3e}"


@pytest.mark.parametrize("theta,D,seq", [(1e4, 128, 96), (1e6, 64, 40), (5e5, 32, 17)])
def test_rope_tables_and_rotation_match_llama_rotary_embedding(theta, D, seq):
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding, apply_rotary_pos_emb
    H = 2
    cfg = LlamaConfig(hidden_size=H * D, num_attention_heads=H, num_key_value_heads=H, intermediate_size=64,
                      num_hidden_layers=1, max_position_embeddings=4 * seq, rope_theta=theta, vocab_size=32)
    if getattr(cfg, "rope_parameters", None) is not None:  # newer configs keep theta here
        cfg.rope_parameters["rope_theta"] = theta
    rot = LlamaRotaryEmbedding(cfg)
    torch.manual_seed(0)
    q, k = torch.randn(1, H, seq, D), torch.randn(1, H, seq, D)
    pos = torch.arange(seq)[None]
    cos_hf, sin_hf = rot(q, pos)                   # [1, seq, D]: the half table repeated twice
    cos, sin = OO.rope_tables(seq, D, theta)       # [seq, D / 2]
    _close(cos, cos_hf[0, :, :D // 2], "cos table")
    _close(sin, sin_hf[0, :, :D // 2], "sin table")
    assert torch.equal(cos_hf[0, :, :D // 2], cos_hf[0, :, D // 2:])
    q_hf, k_hf = apply_rotary_pos_emb(q, k, cos_hf, sin_hf)
    _close(OO.rope(q, cos, sin), q_hf, "rotated q")
    _close(OO.rope(k, cos, sin), k_hf, "rotated k")
    # the block's own table builder and torch statement agree with the oracle's
    c2, s2 = SM.rope_tables(seq, D, theta, "cpu")
    assert torch.equal(c2, cos) and torch.equal(s2, sin)
    _close(SM._apply_rope(q, cos, sin), q_hf, "block rotation")


def test_transformer_layer_is_a_gpt2_block():
    """Pre-LayerNorm, causal, gelu_new; GPT-2 keeps its projections as Conv1D ([in, out] weights)."""
    from transformers import GPT2Config
    from transformers.models.gpt2.modeling_gpt2 import GPT2Block
    dim, heads, ffn, S = 64, 4, 256, 24
    cfg = GPT2Config(n_embd=dim, n_head=heads, n_layer=1, n_inner=ffn, n_positions=64, vocab_size=32,
                     activation_function="gelu_new", resid_pdrop=0.0, attn_pdrop=0.0, embd_pdrop=0.0,
                     layer_norm_epsilon=1e-5)
    cfg._attn_implementation = "eager"
    hf = GPT2Block(cfg, layer_idx=0).eval()
    torch.manual_seed(1)
    for p in hf.parameters():
        torch.nn.init.normal_(p, std=0.2)
    mine = SM.TransformerLayer(dim, heads, ffn, causal=True, pre_ln=True, activation="gelu_tanh", eps=1e-5,
                               dtype=torch.float32)
    sd = hf.state_dict()
    with torch.no_grad():
        for name, p in mine.named_parameters():
            src = sd[name]
            p.copy_(src.t() if (name.endswith("weight") and src.dim() == 2) else src)
    x = torch.randn(2, S, dim)
    # the causal mask is built by the enclosing model in this library version: hand it to the block
    mask = torch.full((S, S), torch.finfo(torch.float32).min).triu(1)[None, None]
    out_hf = hf(x, attention_mask=mask)
    out_hf = out_hf[0] if isinstance(out_hf, tuple) else out_hf
    _close(mine(x), out_hf, "GPT-2 block output")


def test_transformer_layer_post_ln_is_a_bert_layer():
    from transformers import BertConfig
    from transformers.models.bert.modeling_bert import BertLayer
    dim, heads, ffn, S = 64, 4, 256, 24
    cfg = BertConfig(hidden_size=dim, num_attention_heads=heads, intermediate_size=ffn, num_hidden_layers=1,
                     hidden_act="gelu", hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0,
                     layer_norm_eps=1e-12, vocab_size=32)
    cfg._attn_implementation = "eager"
    hf = BertLayer(cfg).eval()
    torch.manual_seed(2)
    for p in hf.parameters():
        torch.nn.init.normal_(p, std=0.2)
    mine = SM.TransformerLayer(dim, heads, ffn, causal=False, pre_ln=False, activation="gelu_erf", eps=1e-12,
                               dtype=torch.float32)
    sd = hf.state_dict()
    att = "attention.self."
    with torch.no_grad():
        mine.attn.c_attn.weight.copy_(torch.cat([sd[att + "query.weight"], sd[att + "key.weight"],
                                                 sd[att + "value.weight"]], 0))
        mine.attn.c_attn.bias.copy_(torch.cat([sd[att + "query.bias"], sd[att + "key.bias"], sd[att + "value.bias"]], 0))
        mine.attn.c_proj.weight.copy_(sd["attention.output.dense.weight"])
        mine.attn.c_proj.bias.copy_(sd["attention.output.dense.bias"])
        mine.ln_1.weight.copy_(sd["attention.output.LayerNorm.weight"])
        mine.ln_1.bias.copy_(sd["attention.output.LayerNorm.bias"])
        mine.mlp.c_fc.weight.copy_(sd["intermediate.dense.weight"])
        mine.mlp.c_fc.bias.copy_(sd["intermediate.dense.bias"])
        mine.mlp.c_proj.weight.copy_(sd["output.dense.weight"])
        mine.mlp.c_proj.bias.copy_(sd["output.dense.bias"])
        mine.ln_2.weight.copy_(sd["output.LayerNorm.weight"])
        mine.ln_2.bias.copy_(sd["output.LayerNorm.bias"])
    x = torch.randn(2, S, dim)
    out_hf = hf(x)
    out_hf = out_hf[0] if isinstance(out_hf, tuple) else out_hf
    _close(mine(x), out_hf, "BERT layer output")


def _llama_position_embeddings(cfg, x, S):
    from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding
    return LlamaRotaryEmbedding(cfg)(x, torch.arange(S)[None])


@pytest.mark.parametrize("heads,kv_heads", [(2, 2), (4, 2), (4, 1)])
def test_llama_layer_is_a_llama_decoder_layer(heads, kv_heads):
    """Multi-head and grouped-query attention (``num_key_value_heads`` < ``num_attention_heads``: which
    query heads share which key / value head is pinned here)."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaDecoderLayer
    dim, ffn, S, theta = 64 * heads, 192, 24, 1e4
    cfg = LlamaConfig(hidden_size=dim, num_attention_heads=heads, num_key_value_heads=kv_heads,
                      intermediate_size=ffn, num_hidden_layers=1, rms_norm_eps=1e-5, rope_theta=theta,
                      max_position_embeddings=64, vocab_size=32, attention_dropout=0.0, hidden_act="silu")
    if getattr(cfg, "rope_parameters", None) is not None:
        cfg.rope_parameters["rope_theta"] = theta
    cfg._attn_implementation = "eager"
    hf = LlamaDecoderLayer(cfg, layer_idx=0).eval()
    torch.manual_seed(3)
    for p in hf.parameters():
        torch.nn.init.normal_(p, std=0.1)
    mine = SM.LlamaLayer(dim, heads, ffn, eps=1e-5, rope_theta=theta, dtype=torch.float32, n_kv_heads=kv_heads)
    sd = hf.state_dict()
    with torch.no_grad():
        mine.self_attn.qkv_proj.weight.copy_(torch.cat([sd["self_attn.q_proj.weight"], sd["self_attn.k_proj.weight"],
                                                        sd["self_attn.v_proj.weight"]], 0))
        for name in ("self_attn.o_proj.weight", "mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight",
                     "input_layernorm.weight", "post_attention_layernorm.weight"):
            mine.get_parameter(name).copy_(sd[name])
    x = torch.randn(2, S, dim)
    mask = torch.full((S, S), float("-inf")).triu(1)[None, None]
    out_hf = hf(x, attention_mask=mask, position_ids=torch.arange(S)[None],
                position_embeddings=_llama_position_embeddings(cfg, x, S))
    out_hf = out_hf[0] if isinstance(out_hf, tuple) else out_hf
    _close(mine(x), out_hf, "Llama decoder layer output")


def test_moe_feed_forward_is_a_mixtral_sparse_moe_block():
    from transformers import MixtralConfig
    from transformers.models.mixtral.modeling_mixtral import MixtralSparseMoeBlock
    dim, heads, ffn, E, T = 64, 1, 96, 8, 50
    cfg = MixtralConfig(hidden_size=dim, intermediate_size=ffn, num_attention_heads=heads, num_key_value_heads=heads,
                        num_local_experts=E, num_experts_per_tok=2, num_hidden_layers=1, vocab_size=32,
                        router_jitter_noise=0.0, hidden_act="silu")
    hf = MixtralSparseMoeBlock(cfg).eval()
    torch.manual_seed(4)
    for p in hf.parameters():
        torch.nn.init.normal_(p, std=0.2)
    mine = SM.MoELayer(dim, heads, ffn, E, dtype=torch.float32)
    sd = hf.state_dict()
    with torch.no_grad():
        mine.block_sparse_moe.gate.weight.copy_(sd["gate.weight"])
        if "experts.gate_up_proj" in sd:   # fused expert weights: [E, 2 ffn, dim] (gate rows, then up rows)
            gu, dn = sd["experts.gate_up_proj"], sd["experts.down_proj"]
            for e, ex in enumerate(mine.block_sparse_moe.experts):
                ex.w1.weight.copy_(gu[e, :ffn])
                ex.w3.weight.copy_(gu[e, ffn:])
                ex.w2.weight.copy_(dn[e])
        else:
            for e, ex in enumerate(mine.block_sparse_moe.experts):
                for w in ("w1", "w2", "w3"):
                    getattr(ex, w).weight.copy_(sd[f"experts.{e}.{w}.weight"])
    h = torch.randn(1, T, dim)
    out_hf = hf(h)
    out_hf = out_hf[0] if isinstance(out_hf, tuple) else out_hf
    _close(mine._feed_forward(h), out_hf.reshape(1, T, dim), "Mixtral sparse MoE block output")
    # and the oracle's own statement of the block
    w1 = torch.stack([ex.w1.weight for ex in mine.block_sparse_moe.experts]).detach()
    w2 = torch.stack([ex.w2.weight for ex in mine.block_sparse_moe.experts]).detach()
    w3 = torch.stack([ex.w3.weight for ex in mine.block_sparse_moe.experts]).detach()
    y = OO.moe_top2(h[0], sd["gate.weight"], w1, w2, w3)
    _close(y, out_hf.reshape(T, dim), "oracle moe_top2")


def test_hugging_face_gpt2_stages_are_recognised_on_the_models_own_layers():
    """The model of the reference's example (examples/huggingface/pippy_gpt2.py:50-65, embeddings untied)
    goes through the torch.export route of the front end; its stages must come out as the blocks the
    launch lists are built from, wrapped around the model's own Conv1D / LayerNorm / Embedding objects,
    and those blocks must reproduce the model."""
    import pippy_amd as pp
    from pippy_amd._lowering import lower_stage_module
    from pippy_amd.stage_modules import InOutLinear
    cfg = transformers.GPT2Config(n_layer=4, n_embd=128, n_head=2, vocab_size=500, n_positions=64,
                                  attn_pdrop=0.0, embd_pdrop=0.0, resid_pdrop=0.0, use_cache=False,
                                  tie_word_embeddings=False, bos_token_id=0, eos_token_id=0)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.GPT2LMHeadModel(cfg)
    ids = torch.randint(0, 500, (2, 48))
    pipe = pp.pipeline(model, mb_args=(ids,), split_spec={"transformer.h.2": pp.SplitPoint.BEGINNING})
    why = []
    blocks = [lower_stage_module(pipe.get_stage_module(i), why) for i in range(2)]
    assert not why, why
    assert [[type(b).__name__ for b in bl] for bl in blocks] == \
        [["WrappedTokenEmbedding"] + ["WrappedTransformerLayer"] * 2, ["WrappedTransformerLayer"] * 2 + ["WrappedLMHead"]]
    first = blocks[0][1]
    assert isinstance(first.attn.c_attn, InOutLinear) and first.attn.c_attn.layer is model.transformer.h[0].attn.c_attn
    assert first.ln_1 is model.transformer.h[0].ln_1 and blocks[0][0].wte is model.transformer.wte
    assert first.causal and first.n_heads == 2 and first.activation == "gelu_tanh"
    assert blocks[1][-1].lm_head is model.lm_head
    x = ids
    with torch.no_grad():
        for b in blocks[0] + blocks[1]:
            x = b(x)
        _close(x, model(ids).logits, "blocks against GPT2LMHeadModel")


def test_hugging_face_llama_stages_are_recognised_on_the_models_own_layers():
    """The model class of the reference's Llama example (examples/llama/pippy_llama.py:18-39): the rotary
    table (computed by the model under no_grad from a buffer) and the causal mask fold into constants, the
    head size is read off that table and the table itself is kept, and the stages come out as Llama blocks around the
    model's own q / k / v / o / gate / up / down projections and LlamaRMSNorm layers."""
    import pippy_amd as pp
    from pippy_amd._lowering import lower_stage_module
    from pippy_amd.stage_modules import RMSNormLike
    cfg = transformers.LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=4,
                                   num_attention_heads=4, num_key_value_heads=2, vocab_size=500,
                                   max_position_embeddings=64, use_cache=False, tie_word_embeddings=False,
                                   attention_dropout=0.0, rope_theta=5e5)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.LlamaForCausalLM(cfg)
    ids = torch.randint(0, 500, (2, 48))
    pipe = pp.pipeline(model, mb_args=(ids,), split_spec={"model.layers.2": pp.SplitPoint.BEGINNING})
    _close(pipe(ids)[0] if isinstance(pipe(ids), (tuple, list)) else pipe(ids), model(ids).logits, "Pipe against the model")
    for i in range(2):
        assert len([n for n in pipe.get_stage_module(i).graph.nodes if n.op == "placeholder"]) == 1
    why = []
    blocks = [lower_stage_module(pipe.get_stage_module(i), why) for i in range(2)]
    assert not why, why
    assert [[type(b).__name__ for b in bl] for bl in blocks] == \
        [["WrappedTokenEmbedding"] + ["WrappedLlamaLayer"] * 2, ["WrappedLlamaLayer"] * 2 + ["WrappedLMHead"]]
    layer = blocks[1][0]
    hf = model.model.layers[2]
    assert layer.self_attn.k_proj is hf.self_attn.k_proj and layer.mlp.gate_proj is hf.mlp.gate_proj
    assert isinstance(layer.input_layernorm, RMSNormLike) and layer.input_layernorm.layer is hf.input_layernorm
    assert (layer.n_heads, layer.n_kv_heads) == (4, 2)
    cos, sin = SM.rope_tables(48, 64, 5e5, "cpu")
    _close(layer._cos, cos, "the model's cosine table")
    _close(layer._sin, sin, "the model's sine table")
    x = ids
    with torch.no_grad():
        for b in blocks[0] + blocks[1]:
            x = b(x)
        _close(x, model(ids).logits, "blocks against LlamaForCausalLM")


def test_hugging_face_mixtral_stages_are_recognised_on_the_models_own_parameters():
    """Mixtral keeps its experts as two stacked parameters (gate|up [E, 2 f, d] and down [E, d, f]) and
    exports its sparse block as a soup of index arithmetic; the stage is recognised by what the branch
    reads (an RMSNorm, a router weight, the two stacked parameters, a top-2, a SiLU) and checked
    numerically against the stage itself, with the attention half handled as Llama's."""
    import pippy_amd as pp
    from pippy_amd._lowering import lower_stage_module
    cfg = transformers.MixtralConfig(hidden_size=256, intermediate_size=256, num_hidden_layers=2,
                                     num_attention_heads=4, num_key_value_heads=2, vocab_size=500,
                                     max_position_embeddings=64, use_cache=False, tie_word_embeddings=False,
                                     num_local_experts=8, num_experts_per_tok=2, attention_dropout=0.0,
                                     sliding_window=None, router_jitter_noise=0.0)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.MixtralForCausalLM(cfg)
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() == 3:
                p.normal_(std=0.05)
    ids = torch.randint(0, 500, (2, 40))
    pipe = pp.pipeline(model, mb_args=(ids,), split_spec={"model.layers.1": pp.SplitPoint.BEGINNING})
    why = []
    blocks = [lower_stage_module(pipe.get_stage_module(i), why) for i in range(2)]
    assert not why, why
    assert [[type(b).__name__ for b in bl] for bl in blocks] == \
        [["WrappedTokenEmbedding", "WrappedMoELayer"], ["WrappedMoELayer", "WrappedLMHead"]]
    layer, hf = blocks[1][0], model.model.layers[1]
    assert layer._experts.gate_up is hf.mlp.experts.gate_up_proj and layer._experts.down is hf.mlp.experts.down_proj
    assert layer._router.weight is hf.mlp.gate.weight and layer.self_attn.q_proj is hf.self_attn.q_proj
    assert (layer.n_experts, layer.ffn, layer.n_heads, layer.n_kv_heads) == (8, 256, 4, 2)
    x = ids
    with torch.no_grad():
        for b in blocks[0] + blocks[1]:
            x = b(x)
        _close(x, model(ids).logits, "blocks against MixtralForCausalLM")
    # a block that picks another number of experts per token is left to autograd, with the reason
    cfg.num_experts_per_tok = 3
    other = transformers.MixtralForCausalLM(cfg)
    pipe = pp.pipeline(other, mb_args=(ids,), split_spec={"model.layers.1": pp.SplitPoint.BEGINNING})
    why = []
    assert lower_stage_module(pipe.get_stage_module(1), why) is None and "two experts" in why[0]


def test_hugging_face_opt_stages_are_recognised_on_the_models_own_layers():
    """The model of the reference's examples/huggingface/pippy_opt.py, in eval mode as there: queries
    scaled by the model before an attention call with scale 1, a position table that is a subclass of
    nn.Embedding reading from row 2 on, ReLU feed-forward, the residual stream re-viewed as rows inside
    each layer."""
    import pippy_amd as pp
    from pippy_amd._lowering import lower_stage_module
    cfg = transformers.OPTConfig(hidden_size=128, ffn_dim=256, num_hidden_layers=2, num_attention_heads=2,
                                 max_position_embeddings=64, dropout=0.0, layerdrop=0.0, use_cache=False,
                                 vocab_size=500, tie_word_embeddings=False)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.OPTForCausalLM(cfg).eval()
    ids = torch.randint(0, 500, (2, 40))
    pipe = pp.pipeline(model, mb_args=(ids,), split_spec={"model.decoder.layers.1": pp.SplitPoint.BEGINNING})
    got = pipe(ids)
    _close(got[0] if isinstance(got, (tuple, list)) else got, model(ids).logits, "Pipe against the model")
    why = []
    blocks = [lower_stage_module(pipe.get_stage_module(i), why) for i in range(2)]
    assert not why, why
    assert [[type(b).__name__ for b in bl] for bl in blocks] == \
        [["WrappedTokenEmbedding", "WrappedTransformerLayer"], ["WrappedTransformerLayer", "WrappedLMHead"]]
    front, layer, hf = blocks[0][0], blocks[1][0], model.model.decoder.layers[1]
    assert front.position_offset == 2 and front.wpe.weight is model.model.decoder.embed_positions.weight
    assert layer.activation == "relu" and layer.causal and layer.pre_ln and layer.mlp.c_fc is hf.fc1
    x = ids
    with torch.no_grad():
        for b in blocks[0] + blocks[1]:
            x = b(x)
        _close(x, model(ids).logits, "blocks against OPTForCausalLM")


def test_positions_counted_over_real_tokens_are_robertas():
    """The oracle's loop against the library routine the RoBERTa family calls, on rows with padding at the
    front, inside, at the end, everywhere and nowhere; and the block's own torch statement of it."""
    from transformers.models.roberta.modeling_roberta import RobertaEmbeddings
    from oracle import ops as OO2
    g = torch.Generator().manual_seed(3)
    for pad in (1, 0, 5):
        ids = torch.randint(0, 9, (7, 37), generator=g)
        ids[0, :4] = pad
        ids[1, 30:] = pad
        ids[2] = pad
        ids[3][ids[3] == pad] = pad + 1
        want = RobertaEmbeddings.create_position_ids_from_input_ids(ids, pad)
        assert torch.equal(OO2.position_ids_from_padding(ids, pad), want)
        blk = SM.EncoderEmbedding(16, 64, 8)
        blk.padding_positions = pad
        assert torch.equal(blk._positions(ids), want)


def test_hugging_face_roberta_stages_are_recognised_on_the_models_own_layers():
    """RoBERTa (the family of the reference's examples/huggingface/pippy_camemBert.py): position indices
    computed from the input ids (a count over the tokens that are not padding), token types gathered from
    a buffer of zeros at those positions."""
    import pippy_amd as pp
    from pippy_amd._lowering import lower_stage_module
    cfg = transformers.RobertaConfig(hidden_size=128, intermediate_size=256, num_hidden_layers=2,
                                     num_attention_heads=2, max_position_embeddings=66, vocab_size=500,
                                     hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0,
                                     tie_word_embeddings=False)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.RobertaForMaskedLM(cfg)
    ids = torch.randint(0, 500, (2, 40))
    pipe = pp.pipeline(model, mb_args=(ids,), split_spec={"roberta.encoder.layer.1": pp.SplitPoint.BEGINNING})
    why = []
    blocks = [lower_stage_module(pipe.get_stage_module(i), why) for i in range(2)]
    assert not why, why
    assert [[type(b).__name__ for b in bl] for bl in blocks] == \
        [["WrappedEncoderEmbedding", "WrappedTransformerLayer"], ["WrappedTransformerLayer", "LinearAct", "WrappedLMHead"]]
    front = blocks[0][0]
    assert front.padding_positions == 1
    assert front.position_embeddings is model.roberta.embeddings.position_embeddings
    assert front.token_type_embeddings is model.roberta.embeddings.token_type_embeddings
    other = torch.randint(0, 500, (2, 40))
    other[0, :3] = 1
    other[1, 20:] = 1
    x = other
    with torch.no_grad():
        for b in blocks[0] + blocks[1]:
            x = b(x)
        _close(x, model(other).logits, "blocks against RobertaForMaskedLM on ids with padding")


@pytest.mark.parametrize("head_dim", [64, 128])
def test_hugging_face_qwen3_stages_are_recognised_with_their_per_head_norms(head_dim):
    """Qwen3: RMS norms over the values of each head, on queries and keys, in front of the rotary
    embedding; and a head size that need not be width / heads (128 with four heads on a width of 256: the
    query projection maps 256 -> 512 and the output projection 512 -> 256)."""
    import pippy_amd as pp
    from pippy_amd._lowering import lower_stage_module
    cfg = transformers.Qwen3Config(hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                                   num_attention_heads=4, num_key_value_heads=2, head_dim=head_dim, vocab_size=500,
                                   max_position_embeddings=64, use_cache=False, tie_word_embeddings=False,
                                   attention_dropout=0.0)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.Qwen3ForCausalLM(cfg)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith(("q_norm.weight", "k_norm.weight")):
                p.add_(torch.randn_like(p) * 0.3)
    ids = torch.randint(0, 500, (2, 48))
    pipe = pp.pipeline(model, mb_args=(ids,), split_spec={"model.layers.1": pp.SplitPoint.BEGINNING})
    why = []
    blocks = [lower_stage_module(pipe.get_stage_module(i), why) for i in range(2)]
    assert not why, why
    assert [[type(b).__name__ for b in bl] for bl in blocks] == \
        [["WrappedTokenEmbedding", "WrappedLlamaLayer"], ["WrappedLlamaLayer", "WrappedLMHead"]]
    layer, hf = blocks[1][0], model.model.layers[1]
    assert layer.q_norm.layer is hf.self_attn.q_norm and layer.k_norm.layer is hf.self_attn.k_norm
    assert (layer.n_heads, layer.n_kv_heads, layer._head_dim()) == (4, 2, head_dim)
    x = ids
    with torch.no_grad():
        for b in blocks[0] + blocks[1]:
            x = b(x)
        _close(x, model(ids).logits, "blocks against Qwen3ForCausalLM")


@pytest.mark.parametrize("attention", ["sdpa", "eager"])
def test_hugging_face_gpt_bigcode_stages_are_recognised_with_multi_query_attention(attention):
    """GPT-BigCode: a GPT-2-style layer whose fused projection is q (d) | k (D) | v (D): every query head
    attends to the one key / value head."""
    import pippy_amd as pp
    from pippy_amd._lowering import lower_stage_module
    cfg = transformers.GPTBigCodeConfig(n_embd=256, n_layer=2, n_head=4, n_positions=64, attn_pdrop=0.0,
                                        embd_pdrop=0.0, resid_pdrop=0.0, use_cache=False, multi_query=True,
                                        vocab_size=500, tie_word_embeddings=False)
    cfg._attn_implementation = attention
    torch.manual_seed(0)
    model = transformers.GPTBigCodeForCausalLM(cfg)
    ids = torch.randint(0, 500, (2, 40))
    pipe = pp.pipeline(model, mb_args=(ids,), split_spec={"transformer.h.1": pp.SplitPoint.BEGINNING})
    why = []
    blocks = [lower_stage_module(pipe.get_stage_module(i), why) for i in range(2)]
    assert not why, why
    layer, hf = blocks[1][0], model.transformer.h[1]
    assert type(layer).__name__ == "WrappedTransformerLayer" and layer.attn.c_attn is hf.attn.c_attn
    assert (layer.n_heads, layer.n_kv_heads, layer.causal, layer.attn.c_attn.out_features) == (4, 1, True, 256 + 128)
    x = ids
    with torch.no_grad():
        for b in blocks[0] + blocks[1]:
            x = b(x)
        _close(x, model(ids).logits, "blocks against GPTBigCodeForCausalLM")


def test_hugging_face_falcon_stages_are_recognised_as_side_by_side_layers():
    """Falcon: attention and feed-forward read the same LayerNorm output and are added to the residual
    stream together; rotary embedding; multi-query attention through one fused projection; no biases.
    The newer decoder layout of the family interleaves q, k and v per key / value group in that projection:
    the numerical comparison notices, and such stages stay with torch."""
    import pippy_amd as pp
    from pippy_amd._lowering import lower_stage_module
    kw = dict(hidden_size=256, num_hidden_layers=2, num_attention_heads=4, hidden_dropout=0.0, attention_dropout=0.0,
              use_cache=False, tie_word_embeddings=False, vocab_size=500, max_position_embeddings=64)
    cfg = transformers.FalconConfig(**kw)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.FalconForCausalLM(cfg)
    ids = torch.randint(0, 500, (2, 40))
    pipe = pp.pipeline(model, mb_args=(ids,), split_spec={"transformer.h.1": pp.SplitPoint.BEGINNING})
    why = []
    blocks = [lower_stage_module(pipe.get_stage_module(i), why) for i in range(2)]
    assert not why, why
    assert [[type(b).__name__ for b in bl] for bl in blocks] == \
        [["WrappedTokenEmbedding", "WrappedParallelLayer"], ["WrappedParallelLayer", "WrappedLMHead"]]
    layer, hf = blocks[1][0], model.transformer.h[1]
    assert layer.qkv is hf.self_attention.query_key_value and layer.ln_a is hf.input_layernorm
    assert layer._ln_m() is layer.ln_a and layer.fc1 is hf.mlp.dense_h_to_4h
    assert (layer.n_heads, layer.n_kv_heads, layer.head_dim, layer.activation) == (4, 1, 64, "gelu_erf")
    x = ids
    with torch.no_grad():
        for b in blocks[0] + blocks[1]:
            x = b(x)
        _close(x, model(ids).logits, "blocks against FalconForCausalLM")
    cfg = transformers.FalconConfig(new_decoder_architecture=True, num_kv_heads=2, **kw)
    cfg._attn_implementation = "sdpa"
    other = transformers.FalconForCausalLM(cfg)
    pipe = pp.pipeline(other, mb_args=(ids,), split_spec={"transformer.h.1": pp.SplitPoint.BEGINNING})
    why = []
    assert lower_stage_module(pipe.get_stage_module(1), why) is None and "differ from the stage's own forward" in why[0]


def test_library_defaults_that_cannot_be_exported_are_set_aside_for_the_export(caplog):
    """The reference's example builds ``GPT2LMHeadModel(config)`` as the library configures it, which today
    returns a key / value cache object that torch.export cannot flatten; Mixtral's default expert product
    inspects tensor addresses in bf16.  The front end exports with the cache off (a pipeline's stages do not
    return one) and with the library's batched expert form, says so, and leaves the configuration as it was."""
    import logging
    import pippy_amd as pp
    cfg = transformers.GPT2Config(n_layer=2, n_embd=128, n_head=2, n_positions=64, attn_pdrop=0.0, embd_pdrop=0.0,
                                  resid_pdrop=0.0, tie_word_embeddings=False, vocab_size=500)
    torch.manual_seed(0)
    model = transformers.GPT2LMHeadModel(cfg)
    assert model.config.use_cache
    ids = torch.randint(0, 500, (2, 32))
    with caplog.at_level(logging.WARNING, logger="pippy_amd._IR"):
        pipe = pp.pipeline(model, mb_args=(ids,), split_spec={"transformer.h.1": pp.SplitPoint.BEGINNING})
    assert "use_cache = False" in caplog.text and model.config.use_cache
    out = pipe(ids)
    _close(out[0] if isinstance(out, (tuple, list)) else out, model(ids).logits, "Pipe against the model")
    cfg = transformers.MixtralConfig(hidden_size=128, intermediate_size=128, num_hidden_layers=2,
                                     num_attention_heads=2, num_key_value_heads=1, vocab_size=300,
                                     max_position_embeddings=32, use_cache=False, tie_word_embeddings=False,
                                     num_local_experts=4, num_experts_per_tok=2, attention_dropout=0.0,
                                     sliding_window=None)
    moe = transformers.MixtralForCausalLM(cfg).to(torch.bfloat16)
    chosen = moe.config._experts_implementation
    ids = torch.randint(0, 300, (2, 16))
    caplog.clear()
    with caplog.at_level(logging.WARNING, logger="pippy_amd._IR"):
        pipe = pp.pipeline(moe, mb_args=(ids,), split_spec={"model.layers.1": pp.SplitPoint.BEGINNING})
    assert pipe.num_stages == 2 and moe.config._experts_implementation == chosen
    if chosen != "batched_mm":
        assert "batched_mm" in caplog.text


def test_hugging_face_bert_stages_are_recognised_on_the_models_own_layers():
    """transformers.BertForMaskedLM (examples/huggingface/pippy_bert.py): the encoder front (three tables
    and a LayerNorm), post-LayerNorm layers with separate query / key / value projections, the all-true
    mask read as "no mask", and the masked-language-model head."""
    import pippy_amd as pp
    from pippy_amd._lowering import lower_stage_module
    cfg = transformers.BertConfig(hidden_size=128, intermediate_size=512, num_hidden_layers=4, num_attention_heads=2,
                                  vocab_size=500, max_position_embeddings=64, hidden_dropout_prob=0.0,
                                  attention_probs_dropout_prob=0.0, tie_word_embeddings=False)
    cfg._attn_implementation = "sdpa"
    torch.manual_seed(0)
    model = transformers.BertForMaskedLM(cfg)
    ids = torch.randint(0, 500, (2, 48))
    pipe = pp.pipeline(model, mb_args=(ids,), split_spec={"bert.encoder.layer.2": pp.SplitPoint.BEGINNING})
    why = []
    blocks = [lower_stage_module(pipe.get_stage_module(i), why) for i in range(2)]
    assert not why, why
    assert [[type(b).__name__ for b in bl] for bl in blocks] == \
        [["WrappedEncoderEmbedding"] + ["WrappedTransformerLayer"] * 2,
         ["WrappedTransformerLayer"] * 2 + ["LinearAct", "WrappedLMHead"]]
    layer, hf = blocks[1][0], model.bert.encoder.layer[2]
    assert not layer.pre_ln and not layer.causal and layer.activation == "gelu_erf" and layer.n_heads == 2
    assert layer._qkv_layers() == (hf.attention.self.query, hf.attention.self.key, hf.attention.self.value)
    assert layer.ln_1 is hf.attention.output.LayerNorm and layer.ln_2 is hf.output.LayerNorm
    assert blocks[0][0].token_type_embeddings is model.bert.embeddings.token_type_embeddings
    assert blocks[1][-1].lm_head is model.cls.predictions.decoder and blocks[1][-1].lm_head.bias is not None
    x = ids
    with torch.no_grad():
        for b in blocks[0] + blocks[1]:
            x = b(x)
        _close(x, model(ids).logits, "blocks against BertForMaskedLM")
