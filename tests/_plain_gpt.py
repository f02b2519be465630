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
