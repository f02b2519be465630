"""A GPT-2-shaped decoder written with plain torch layers only (no block of ``pippy_amd.stage_modules``):
the kind of model the reference is handed (``examples/huggingface/pippy_gpt2.py:50-65``)."""
import torch
import torch.nn as nn
import torch.nn.functional as F


class Block(nn.Module):
    def __init__(self, d, h):
        super().__init__()
        self.ln_1 = nn.LayerNorm(d); self.c_attn = nn.Linear(d, 3*d); self.c_proj = nn.Linear(d, d)
        self.ln_2 = nn.LayerNorm(d); self.c_fc = nn.Linear(d, 4*d); self.mlp_proj = nn.Linear(4*d, d)
        self.n_head = h; self.drop = nn.Dropout(0.0)
    def forward(self, x):
        B, T, C = x.size()
        q, k, v = self.c_attn(self.ln_1(x)).split(C, dim=2)
        q = q.view(B, T, self.n_head, C // self.n_head).transpose(1, 2)
        k = k.view(B, T, self.n_head, C // self.n_head).transpose(1, 2)
        v = v.view(B, T, self.n_head, C // self.n_head).transpose(1, 2)
        y = F.scaled_dot_product_attention(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=True)
        y = y.transpose(1, 2).contiguous().view(B, T, C)
        x = x + self.drop(self.c_proj(y))
        x = x + self.mlp_proj(F.gelu(self.c_fc(self.ln_2(x)), approximate="tanh"))
        return x
class GPT(nn.Module):
    def __init__(self, vocab=1000, seq=128, d=128, h=2, L=4):
        super().__init__()
        self.wte = nn.Embedding(vocab, d); self.wpe = nn.Embedding(seq, d); self.drop = nn.Dropout(0.0)
        self.h = nn.ModuleList([Block(d, h) for _ in range(L)])
        self.ln_f = nn.LayerNorm(d); self.lm_head = nn.Linear(d, vocab, bias=False)
    def forward(self, idx):
        b, t = idx.size()
        pos = torch.arange(0, t, dtype=torch.long, device=idx.device)
        x = self.drop(self.wte(idx) + self.wpe(pos))
        for blk in self.h:
            x = blk(x)
        return self.lm_head(self.ln_f(x))


# ---- the same model the way model libraries write it ---------------------------------------------------
# Affine layers that keep their weight as [in, out], an activation class of their own, an explicit
# boolean mask built from the sequence length, and Python control flow on shapes (torch.fx symbolic
# tracing cannot follow it, so the front end goes through torch.export).
class Affine(nn.Module):
    def __init__(self, nx, nf):
        super().__init__()
        self.nf = nf
        self.weight = nn.Parameter(torch.randn(nx, nf) * 0.02)
        self.bias = nn.Parameter(torch.randn(nf) * 0.02)
    def forward(self, x):
        out_shape = x.size()[:-1] + (self.nf,)
        return torch.addmm(self.bias, x.view(-1, x.size(-1)), self.weight).view(out_shape)
class TanhGelu(nn.Module):
    def forward(self, x):
        return 0.5 * x * (1.0 + torch.tanh(0.7978845608028654 * (x + 0.044715 * torch.pow(x, 3.0))))
class LibAttention(nn.Module):
    def __init__(self, d, h):
        super().__init__()
        self.c_attn = Affine(d, 3*d); self.c_proj = Affine(d, d); self.n_head = h
        self.resid_dropout = nn.Dropout(0.0)
    def forward(self, x, mask):
        B, T, C = x.size()
        q, k, v = self.c_attn(x).split(C, dim=2)
        shape = (B, T, -1, C // self.n_head)
        q, k, v = (t.view(shape).transpose(1, 2) for t in (q, k, v))
        y = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=(C // self.n_head) ** -0.5)
        return self.resid_dropout(self.c_proj(y.transpose(1, 2).reshape(B, T, C)))
class LibMLP(nn.Module):
    def __init__(self, d):
        super().__init__()
        self.c_fc = Affine(d, 4*d); self.act = TanhGelu(); self.c_proj = Affine(4*d, d)
    def forward(self, x):
        return self.c_proj(self.act(self.c_fc(x)))
class LibBlock(nn.Module):
    def __init__(self, d, h):
        super().__init__()
        self.ln_1 = nn.LayerNorm(d); self.attn = LibAttention(d, h)
        self.ln_2 = nn.LayerNorm(d); self.mlp = LibMLP(d)
    def forward(self, x, mask):
        x = self.attn(self.ln_1(x), mask) + x
        return x + self.mlp(self.ln_2(x))
class LibGPT(nn.Module):
    def __init__(self, vocab=1000, seq=128, d=128, h=2, L=4):
        super().__init__()
        self.wte = nn.Embedding(vocab, d); self.wpe = nn.Embedding(seq, d)
        self.h = nn.ModuleList([LibBlock(d, h) for _ in range(L)])
        self.ln_f = nn.LayerNorm(d); self.lm_head = nn.Linear(d, vocab, bias=False)
    def forward(self, idx):
        idx = idx.view(-1, idx.shape[-1])
        t = idx.shape[-1]
        if t > self.wpe.num_embeddings:          # control flow on a shape
            raise ValueError("sequence too long")
        pos = torch.arange(t, device=idx.device).unsqueeze(0)
        mask = (pos.unsqueeze(-1) >= pos.unsqueeze(-2))[:, None].expand(idx.shape[0], 1, t, t)
        x = self.wte(idx) + self.wpe(pos)
        for blk in self.h:
            x = blk(x, mask)
        return self.lm_head(self.ln_f(x))


# ---- an encoder built from torch's own layer class ------------------------------------------------------
class TorchEncoderLM(nn.Module):
    def __init__(self, vocab=1000, seq=128, d=128, h=2, L=4, norm_first=True, activation="gelu"):
        super().__init__()
        self.emb = nn.Embedding(vocab, d); self.pos = nn.Embedding(seq, d)
        self.layers = nn.ModuleList([nn.TransformerEncoderLayer(d, h, 4 * d, dropout=0.0, activation=activation,
                                                                batch_first=True, norm_first=norm_first)
                                     for _ in range(L)])
        self.norm = nn.LayerNorm(d); self.head = nn.Linear(d, vocab, bias=False)
    def forward(self, ids):
        x = self.emb(ids) + self.pos(torch.arange(ids.shape[1], device=ids.device))
        for layer in self.layers:
            x = layer(x)
        return self.head(self.norm(x))


class TorchEncoderStackLM(nn.Module):
    """The same with the layers inside ``nn.TransformerEncoder`` (whose forward torch.fx cannot follow: the
    front end exports it, and the layers dissolve into ATen nodes on their parameters)."""
    def __init__(self, vocab=1000, seq=128, d=128, h=2, L=4, norm_first=True, activation="gelu"):
        super().__init__()
        self.emb = nn.Embedding(vocab, d); self.pos = nn.Embedding(seq, d)
        layer = nn.TransformerEncoderLayer(d, h, 4 * d, dropout=0.0, activation=activation, batch_first=True,
                                           norm_first=norm_first)
        self.encoder = nn.TransformerEncoder(layer, L, norm=nn.LayerNorm(d) if norm_first else None,
                                             enable_nested_tensor=False)
        self.head = nn.Linear(d, vocab, bias=False)
    def forward(self, ids):
        x = self.emb(ids) + self.pos(torch.arange(ids.shape[1], device=ids.device))
        return self.head(self.encoder(x))


class TorchCausalLM(nn.Module):
    """A decoder-only language model the way tutorials build it from torch's encoder layers: a causal
    mask made in forward from the sequence length, handed to every layer."""
    def __init__(self, vocab=1000, seq=128, d=128, h=2, L=4, flag=True):
        super().__init__()
        self.flag = flag
        self.emb = nn.Embedding(vocab, d); self.pos = nn.Embedding(seq, d)
        self.layers = nn.ModuleList([nn.TransformerEncoderLayer(d, h, 4 * d, dropout=0.0, activation="gelu",
                                                                batch_first=True, norm_first=True)
                                     for _ in range(L)])
        self.norm = nn.LayerNorm(d); self.head = nn.Linear(d, vocab, bias=False)
    def forward(self, ids):
        S = ids.shape[1]
        x = self.emb(ids) + self.pos(torch.arange(S, device=ids.device))
        mask = nn.Transformer.generate_square_subsequent_mask(S, device=ids.device)
        for layer in self.layers:
            x = layer(x, src_mask=mask, is_causal=True) if self.flag else layer(x, src_mask=mask)
        return self.head(self.norm(x))


# ---- a GPT in the style of small teaching code bases ------------------------------------------------------
# (a layer norm class of its own with an optional bias, a ModuleDict of parts, attention through the fused
# call or spelled out against a registered lower-triangular buffer, linear layers with or without biases)
import math


class OwnLayerNorm(nn.Module):
    def __init__(self, d, bias):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(d) + 0.1 * torch.randn(d))
        self.bias = nn.Parameter(0.1 * torch.randn(d)) if bias else None
    def forward(self, x):
        return F.layer_norm(x, self.weight.shape, self.weight, self.bias, 1e-5)
class TeachingAttention(nn.Module):
    def __init__(self, d, h, seq, bias, flash):
        super().__init__()
        self.c_attn = nn.Linear(d, 3 * d, bias=bias); self.c_proj = nn.Linear(d, d, bias=bias)
        self.attn_dropout = nn.Dropout(0.0); self.resid_dropout = nn.Dropout(0.0)
        self.n_head, self.n_embd, self.flash = h, d, flash
        if not flash:
            self.register_buffer("bias", torch.tril(torch.ones(seq, seq)).view(1, 1, seq, seq))
    def forward(self, x):
        B, T, C = x.size()
        q, k, v = self.c_attn(x).split(self.n_embd, dim=2)
        k = k.view(B, T, self.n_head, C // self.n_head).transpose(1, 2)
        q = q.view(B, T, self.n_head, C // self.n_head).transpose(1, 2)
        v = v.view(B, T, self.n_head, C // self.n_head).transpose(1, 2)
        if self.flash:
            y = F.scaled_dot_product_attention(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=True)
        else:
            att = (q @ k.transpose(-2, -1)) * (1.0 / math.sqrt(k.size(-1)))
            att = att.masked_fill(self.bias[:, :, :T, :T] == 0, float("-inf"))
            att = self.attn_dropout(F.softmax(att, dim=-1))
            y = att @ v
        y = y.transpose(1, 2).contiguous().view(B, T, C)
        return self.resid_dropout(self.c_proj(y))
class TeachingMLP(nn.Module):
    def __init__(self, d, bias):
        super().__init__()
        self.c_fc = nn.Linear(d, 4 * d, bias=bias); self.gelu = nn.GELU()
        self.c_proj = nn.Linear(4 * d, d, bias=bias); self.dropout = nn.Dropout(0.0)
    def forward(self, x):
        return self.dropout(self.c_proj(self.gelu(self.c_fc(x))))
class TeachingBlock(nn.Module):
    def __init__(self, d, h, seq, bias, flash):
        super().__init__()
        self.ln_1 = OwnLayerNorm(d, bias); self.attn = TeachingAttention(d, h, seq, bias, flash)
        self.ln_2 = OwnLayerNorm(d, bias); self.mlp = TeachingMLP(d, bias)
    def forward(self, x):
        x = x + self.attn(self.ln_1(x))
        return x + self.mlp(self.ln_2(x))
class TeachingGPT(nn.Module):
    def __init__(self, vocab=1000, seq=128, d=128, h=2, L=4, bias=True, flash=True):
        super().__init__()
        self.block_size = seq
        self.transformer = nn.ModuleDict(dict(
            wte=nn.Embedding(vocab, d), wpe=nn.Embedding(seq, d), drop=nn.Dropout(0.0),
            h=nn.ModuleList([TeachingBlock(d, h, seq, bias, flash) for _ in range(L)]), ln_f=OwnLayerNorm(d, bias)))
        self.lm_head = nn.Linear(d, vocab, bias=False)
    def forward(self, idx):
        b, t = idx.size()
        assert t <= self.block_size, "sequence longer than the block size"
        pos = torch.arange(0, t, dtype=torch.long, device=idx.device)
        x = self.transformer.drop(self.transformer.wte(idx) + self.transformer.wpe(pos))
        for block in self.transformer.h:
            x = block(x)
        return self.lm_head(self.transformer.ln_f(x))


# ---- blocks of one's own around torch's attention layer ----------------------------------------------------
class MHABlock(nn.Module):
    def __init__(self, d, h, need_weights, causal):
        super().__init__()
        self.ln1 = nn.LayerNorm(d); self.attn = nn.MultiheadAttention(d, h, batch_first=True)
        self.ln2 = nn.LayerNorm(d); self.ff = nn.Sequential(nn.Linear(d, 4 * d), nn.GELU(), nn.Linear(4 * d, d))
        self.need_weights, self.causal = need_weights, causal
    def forward(self, x):
        h = self.ln1(x)
        mask = None
        if self.causal:
            mask = torch.triu(torch.ones(x.shape[1], x.shape[1], dtype=torch.bool, device=x.device), 1)
        x = x + self.attn(h, h, h, need_weights=self.need_weights, attn_mask=mask)[0]
        return x + self.ff(self.ln2(x))
class MHAModel(nn.Module):
    def __init__(self, vocab=1000, seq=128, d=128, h=2, L=4, need_weights=True, causal=False):
        super().__init__()
        self.emb = nn.Embedding(vocab, d); self.pos = nn.Embedding(seq, d)
        self.blocks = nn.ModuleList([MHABlock(d, h, need_weights, causal) for _ in range(L)])
        self.norm = nn.LayerNorm(d); self.head = nn.Linear(d, vocab, bias=False)
    def forward(self, ids):
        x = self.emb(ids) + self.pos(torch.arange(ids.shape[1], device=ids.device))
        for b in self.blocks:
            x = b(x)
        return self.head(self.norm(x))
