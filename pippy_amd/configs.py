"""Model definitions of the baseline configurations, built from lowerable stage blocks.

These are the shapes the throughput metric is quoted on: random-initialised (std 0.02), no
checkpoint needed.  Each model is a plain ``nn.Module`` whose ``forward`` applies its children
in order, so ``pipeline(model, ..., split_spec={"h.3": SplitPoint.BEGINNING, ...})`` cuts it into
stages that lower to HIP launch lists.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .stage_modules import EncoderEmbedding, LlamaLayer, LMHead, MoELayer, TokenEmbedding, TransformerLayer


class DecoderLM(nn.Module):
    """GPT-2-shaped decoder: token + position embedding, pre-LayerNorm causal transformer layers
    with tanh-GELU, final LayerNorm and an untied vocabulary projection."""

    def __init__(self, vocab=50257, max_seq=1024, dim=768, n_layers=12, n_heads=12, ffn=3072,
                 dtype=torch.bfloat16, causal=True, pre_ln=True, activation="gelu_tanh", eps=1e-5):
        super().__init__()
        self.embed = TokenEmbedding(vocab, max_seq, dim, dtype=dtype)
        self.h = nn.ModuleList([
            TransformerLayer(dim, n_heads, ffn, causal=causal, pre_ln=pre_ln, activation=activation,
                             eps=eps, dtype=dtype) for _ in range(n_layers)])
        self.head = LMHead(dim, vocab, final_ln=pre_ln, eps=eps, dtype=dtype)

    def forward(self, ids):
        x = self.embed(ids)
        for layer in self.h:
            x = layer(x)
        return self.head(x)


def gpt2_small(dtype=torch.bfloat16) -> DecoderLM:
    """12 layers, width 768, 12 heads, FFN 3072, vocabulary 50257, sequence 1024."""
    return DecoderLM(dtype=dtype)


class EncoderModel(nn.Module):
    """BERT-shaped encoder: word + position + token-type embedding with LayerNorm, post-LayerNorm
    bidirectional transformer layers with erf-GELU; returns the last hidden state."""

    def __init__(self, vocab=30522, max_seq=512, dim=768, n_layers=12, n_heads=12, ffn=3072,
                 dtype=torch.bfloat16, eps=1e-12):
        super().__init__()
        self.embed = EncoderEmbedding(vocab, max_seq, dim, eps=eps, dtype=dtype)
        self.h = nn.ModuleList([
            TransformerLayer(dim, n_heads, ffn, causal=False, pre_ln=False, activation="gelu_erf",
                             eps=eps, dtype=dtype) for _ in range(n_layers)])

    def forward(self, ids):
        x = self.embed(ids)
        for layer in self.h:
            x = layer(x)
        return x


def bert_base(dtype=torch.bfloat16) -> EncoderModel:
    """12 layers, hidden 768, 12 heads, FFN 3072, vocabulary 30522, sequence 512."""
    return EncoderModel(dtype=dtype)


class LlamaStage(nn.Module):
    """One pipeline stage's share of a Llama-style decoder: ``n_layers`` decoder layers applied to
    incoming activations ``[batch, seq, dim]`` (no embedding, no head)."""

    def __init__(self, n_layers=8, dim=4096, n_heads=32, ffn=11008, eps=1e-5, rope_theta=1e4,
                 dtype=torch.bfloat16, n_kv_heads=None):
        super().__init__()
        self.layers = nn.ModuleList([
            LlamaLayer(dim, n_heads, ffn, eps=eps, rope_theta=rope_theta, dtype=dtype, n_kv_heads=n_kv_heads)
            for _ in range(n_layers)])

    def forward(self, x):
        for layer in self.layers:
            x = layer(x)
        return x


def llama2_7b_stage(dtype=torch.bfloat16) -> LlamaStage:
    """8 of the 32 layers of a Llama-2-7B-shaped model: width 4096, 32 heads of 128, SwiGLU 11008."""
    return LlamaStage(dtype=dtype)


class MoEDecoderLM(nn.Module):
    """Mixtral-shaped decoder: token embedding (positions enter through the rotary embedding),
    decoder layers whose feed-forward is a top-2 mixture of SwiGLU experts, final RMSNorm and an
    untied vocabulary projection."""

    def __init__(self, vocab=32000, dim=1024, n_layers=8, n_heads=16, ffn=4096, n_experts=8,
                 dtype=torch.bfloat16, eps=1e-5, rope_theta=1e6):
        super().__init__()
        self.embed = TokenEmbedding(vocab, 0, dim, dtype=dtype, positions=False)
        self.h = nn.ModuleList([
            MoELayer(dim, n_heads, ffn, n_experts, eps=eps, rope_theta=rope_theta, dtype=dtype)
            for _ in range(n_layers)])
        self.head = LMHead(dim, vocab, final_ln="rms", eps=eps, dtype=dtype)

    def forward(self, ids):
        x = self.embed(ids)
        for layer in self.h:
            x = layer(x)
        return self.head(x)


def mixtral_style(dtype=torch.bfloat16) -> MoEDecoderLM:
    """8 layers (2 stages of 4), width 1024, 16 heads of 64, 8 experts with SwiGLU 4096, top-2 router,
    vocabulary 32000."""
    return MoEDecoderLM(dtype=dtype)


def equal_split_spec(n_layers: int, n_stages: int, prefix: str = "h"):
    """Split points that give every stage ``n_layers / n_stages`` consecutive layers."""
    from ._IR import SplitPoint
    per = n_layers // n_stages
    return {f"{prefix}.{per * s}": SplitPoint.BEGINNING for s in range(1, n_stages)}
