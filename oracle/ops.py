"""fp32 CPU statements of the arithmetic a stage module performs.

The reference runs the user's ``nn.Module.forward`` (pippy/_PipelineStage.py:420-428) and one
``torch.autograd.backward`` (pippy/_backward.py:67-69); these are the torch calls the transformer
and MLP stage modules of the baseline configurations reduce to.  All functions take and return
fp32 CPU tensors; gradients come from autograd on these functions.

Pinning: every function here is a direct torch library routine or a closed form checked against
one in tests/test_oracle.py (gelu closed forms vs F.gelu, attention vs
F.scaled_dot_product_attention, layer norm vs F.layer_norm, cross entropy vs F.cross_entropy,
rms norm vs F.rms_norm, silu vs F.silu, the rotary embedding vs a complex-number rotation and its
norm / relative-position invariants; top-2 routing vs torch.topk on tie-free logits, the expert
permutation vs a stable argsort, the sparse mixture-of-experts layer vs the dense sum over all
experts with zero weight for the experts not selected).
"""
import math

import torch
import torch.nn.functional as F


def linear(x, w, b=None):
    return F.linear(x, w, b)


def gelu_erf(x):
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def gelu_tanh(x):
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


def layer_norm(x, gamma, beta, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    y = (x - mean) / torch.sqrt(var + eps) * gamma
    return y + beta if beta is not None else y


def rms_norm(x, gamma, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gamma


def swiglu(g, u):
    return g * torch.sigmoid(g) * u


def rope_tables(seq, D, theta=10000.0):
    """cos, sin [seq, D/2] (fp32): angle of position p and frequency index i is p * theta^(-2i/D)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    ang = torch.arange(seq, dtype=torch.float32)[:, None] * inv_freq[None, :]
    return torch.cos(ang), torch.sin(ang)


def rope(x, cos, sin):
    """Rotate-half rotary embedding.  x: [..., S, D]; cos, sin: [S, D/2]."""
    half = x.shape[-1] // 2
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)


def attention(q, k, v, causal, scale=None):
    """q, k, v: [B, H, S, D] -> [B, H, S, D] (softmax(q k^T * scale + mask) v)."""
    D = q.shape[-1]
    scale = D ** -0.5 if scale is None else scale
    s = torch.matmul(q, k.transpose(-1, -2)) * scale
    if causal:
        S = q.shape[-2]
        mask = torch.ones(S, S, dtype=torch.bool).tril()
        s = s.masked_fill(~mask, float("-inf"))
    return torch.matmul(torch.softmax(s, dim=-1), v)


def attention_fused_qkv(qkv, H, causal, n_kv_heads=None):
    """qkv: [B, S, (H + 2 H_kv) * D] (q | k | v on the last dim) -> [B, S, H*D].  With
    ``n_kv_heads`` = H_kv < H (grouped-query attention) query heads g * H / H_kv .. (g + 1) * H / H_kv - 1
    attend to key / value head g."""
    B, S, width = qkv.shape
    Hkv = H if n_kv_heads is None else n_kv_heads
    D = width // (H + 2 * Hkv)
    q, k, v = qkv.split([H * D, Hkv * D, Hkv * D], dim=-1)
    q = q.reshape(B, S, H, D).transpose(1, 2)
    k, v = (t.reshape(B, S, Hkv, D).transpose(1, 2).repeat_interleave(H // Hkv, dim=1) for t in (k, v))
    o = attention(q, k, v, causal)
    return o.transpose(1, 2).reshape(B, S, H * D)


def cross_entropy_mean(logits, target, ignore_index=-100):
    """Mean negative log-likelihood over rows whose target is not ignore_index."""
    lse = torch.logsumexp(logits, dim=-1)
    valid = target != ignore_index
    safe = torch.where(valid, target, torch.zeros_like(target))
    picked = logits.gather(-1, safe.unsqueeze(-1)).squeeze(-1)
    per_row = torch.where(valid, lse - picked, torch.zeros_like(lse))
    return per_row.sum() / valid.sum().clamp(min=1)


def embedding(ids, wte, wpe=None):
    y = wte[ids]
    if wpe is not None:
        S = ids.shape[-1]
        y = y + wpe[:S]
    return y


def position_ids_from_padding(ids, pad):
    """Positions counted over the tokens that are not padding, as the embeddings of the encoder in the
    reference's examples/huggingface/pippy_camemBert.py compute them (``transformers``' RoBERTa family;
    pinned against that library's own routine in tests/test_hf_fidelity.py): a padding token gets
    ``pad``, the k-th other token of its sequence (k = 1, 2, ...) gets ``pad + k``."""
    out = torch.full_like(ids, pad)
    for b in range(ids.shape[0]):
        k = 0
        for s in range(ids.shape[1]):
            if int(ids[b, s]) != pad:
                k += 1
                out[b, s] = pad + k
    return out


def embedding_at(ids, pos_ids, wte, wpe, extra_row=None):
    """wte[ids] + wpe[pos_ids] (+ one row added to every token)."""
    y = wte[ids] + wpe[pos_ids]
    return y if extra_row is None else y + extra_row


# ---- top-2 mixture of experts (Mixtral-style block) -------------------------------------------
def moe_route_top2(logits):
    """Softmax over all experts, the two largest probabilities (the lower expert index wins a tie),
    renormalised to sum to one.  Returns (idx int64 [T, 2], gate fp32 [T, 2], first slot = largest)."""
    probs = torch.softmax(logits.float(), dim=-1)
    # a stable descending sort keeps the lower index first among equal values
    order = torch.sort(probs, dim=-1, descending=True, stable=True).indices
    idx = order[:, :2]
    top = probs.gather(-1, idx)
    return idx, top / top.sum(-1, keepdim=True)


def moe_permutation(expert_of_slot, E):
    """Rows grouped by expert, ascending flat slot inside an expert.  Returns (seg_start [E + 1],
    row_src [n], pos [n]) as int64 tensors."""
    flat = expert_of_slot.reshape(-1).long()
    row_src = torch.sort(flat, stable=True).indices
    pos = torch.empty_like(row_src)
    pos[row_src] = torch.arange(flat.numel())
    counts = torch.bincount(flat, minlength=E)
    seg_start = torch.cat([torch.zeros(1, dtype=torch.long), counts.cumsum(0)])
    return seg_start, row_src, pos


def moe_top2(x, w_router, w1, w2, w3, idx=None):
    """y[t] = sum over the two selected experts e of gate[t, e] * w2_e (silu(w1_e x[t]) * (w3_e x[t])).
    ``w1, w3`` [E, ffn, d], ``w2`` [E, d, ffn], ``w_router`` [E, d].  ``idx`` ([T, 2]) forces the
    selection (the weights are then the renormalised probabilities of the forced pair)."""
    logits = F.linear(x, w_router)
    if idx is None:
        idx, gate = moe_route_top2(logits)
    else:
        top = torch.softmax(logits.float(), dim=-1).gather(-1, idx)
        gate = top / top.sum(-1, keepdim=True)
    y = torch.zeros_like(x)
    for e in range(w1.shape[0]):
        tok, slot = torch.where(idx == e)
        if tok.numel() == 0:
            continue
        xe = x[tok]
        ye = F.linear(swiglu(F.linear(xe, w1[e]), F.linear(xe, w3[e])), w2[e])
        y = y.index_add(0, tok, gate[tok, slot, None] * ye)
    return y
