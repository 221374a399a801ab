"""Decoder stack that interleaves ordinary causal attention with sliding-window 2-simplicial
attention, and a byte-level language-model wrapper around it.

Counterparts of simplicial_attention/two_simplicial_transformer.py:24-141 (``Attention``,
``FeedForward``, ``TwoSimplicialTransformer``) and of the ``TwoSimplicialLM`` class of
train.py:64-135 in the reference, with the same constructor arguments and the same
parameter names, so that a reference ``state_dict`` loads unchanged.  The ordinary layers
are library calls (``scaled_dot_product_attention``, ``Linear``); every
``two_simplicial_attn_every``-th layer is the MI355X module of this package.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .two_simplicial_attention import SlidingWindowTwoSimplicialMHA


class Attention(nn.Module):
    """Pre-normed causal attention with grouped key/value heads
    (two_simplicial_transformer.py:24-65)."""

    def __init__(self, dim, dim_head=64, heads=8, key_value_heads=8):
        super().__init__()
        if heads % key_value_heads:
            raise AssertionError('heads must be a multiple of key_value_heads')
        self.heads, self.key_value_heads, self.dim_head = heads, key_value_heads, dim_head
        self.prenorm = nn.RMSNorm(dim)
        self.to_q = nn.Linear(dim, heads * dim_head, bias=False)
        self.to_kv = nn.Linear(dim, 2 * key_value_heads * dim_head, bias=False)
        self.to_out = nn.Linear(heads * dim_head, dim, bias=False)

    def forward(self, x):
        b, n, _ = x.shape
        x = self.prenorm(x)
        q = self.to_q(x).view(b, n, self.heads, self.dim_head).transpose(1, 2)
        # channel order of the fused projection: (key | value, head, d)
        kv = self.to_kv(x).view(b, n, 2, self.key_value_heads, self.dim_head)
        k, v = kv[:, :, 0].transpose(1, 2), kv[:, :, 1].transpose(1, 2)
        out = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=self.heads != self.key_value_heads)
        return self.to_out(out.transpose(1, 2).reshape(b, n, self.heads * self.dim_head))


def FeedForward(dim, expansion=4.):
    """RMSNorm -> Linear -> GELU -> Linear (two_simplicial_transformer.py:69-76)."""
    inner = int(dim * expansion)
    return nn.Sequential(nn.RMSNorm(dim), nn.Linear(dim, inner), nn.GELU(), nn.Linear(inner, dim))


class TwoSimplicialTransformer(nn.Module):
    def __init__(self, dim, *, depth, heads=8, key_value_heads=4, dim_head=64, ff_expansion=4.,
                 two_simplicial_attn_every=4, attn_kwargs: dict | None = None,
                 two_simplicial_attn_kwargs: dict | None = None, final_norm=True):
        super().__init__()
        attn_kwargs = {} if attn_kwargs is None else attn_kwargs
        if two_simplicial_attn_kwargs is None:
            two_simplicial_attn_kwargs = dict(w1=512, w2=32, qk_rmsnorm=True)
        blocks = []
        for index in range(1, depth + 1):
            common = dict(dim=dim, heads=heads, key_value_heads=key_value_heads, dim_head=dim_head)
            if index % two_simplicial_attn_every == 0:
                attn = SlidingWindowTwoSimplicialMHA(prenorm=True, **common, **two_simplicial_attn_kwargs)
            else:
                attn = Attention(**common, **attn_kwargs)
            blocks.append(nn.ModuleList([attn, FeedForward(dim, ff_expansion)]))
        self.layers = nn.ModuleList(blocks)
        self.norm = nn.RMSNorm(dim) if final_norm else nn.Identity()

    def forward(self, x):
        for attn, ff in self.layers:
            x = x + attn(x)
            x = x + ff(x)
        return self.norm(x)


class TwoSimplicialLM(nn.Module):
    """Token + learned position embedding, the stack above, and a linear read-out
    (train.py:64-135; sampling helpers are not part of this build)."""

    def __init__(self, *, num_tokens, dim, depth, max_seq_len=512, dim_head=64, heads=8,
                 two_simplicial_attn_every=4, transformer_kwargs: dict | None = None):
        super().__init__()
        self.token_emb = nn.Embedding(num_tokens, dim)
        self.pos_emb = nn.Embedding(max_seq_len, dim)
        self.transformer = TwoSimplicialTransformer(dim=dim, depth=depth, dim_head=dim_head, heads=heads,
                                                    two_simplicial_attn_every=two_simplicial_attn_every,
                                                    **(transformer_kwargs or {}))
        self.to_logits = nn.Linear(dim, num_tokens, bias=False)

    def forward(self, x, return_loss=False):
        target = None
        if return_loss:
            x, target = x[:, :-1], x[:, 1:]
        positions = torch.arange(x.shape[-1], device=x.device)
        hidden = self.transformer(self.token_emb(x) + self.pos_emb(positions))
        logits = self.to_logits(hidden)
        if target is None:
            return logits
        return F.cross_entropy(logits.flatten(0, 1).float(), target.flatten())
