"""Multi-head wrapper around a higher-order ``attend`` callable.

Counterpart of simplicial_attention/simplicial_mha.py:28-150 of the reference: the
same constructor arguments, the same parameter names and shapes (so a reference
``state_dict`` loads unchanged) and the same channel order of the fused projection,
``(head, set, d)`` for keys and values.
"""
from __future__ import annotations

from functools import partial
from typing import Callable

import torch
from torch import nn

from .naive import naive_two_simplicial_attend, nth_order_attend


class HigherOrderAttention(nn.Module):
    def __init__(
        self,
        dim,
        causal=False,
        dim_head=64,
        dim_head_values=None,
        heads=8,
        key_value_heads=None,
        number_key_value_sets=2,
        qk_rmsnorm=True,
        prenorm=False,
        postnorm=False,
        attend: Callable | None = None,
        head_first_dim=True,
    ):
        super().__init__()
        key_value_heads = heads if key_value_heads is None else key_value_heads
        dim_head_values = dim_head if dim_head_values is None else dim_head_values
        assert heads % key_value_heads == 0, 'heads must be a multiple of key_value_heads'

        self.causal = causal
        self.scale = dim_head ** -0.5
        self.heads = heads
        self.key_value_heads = key_value_heads
        self.query_head_groups = heads // key_value_heads
        self.kv_sets = number_key_value_sets
        self.head_first_dim = head_first_dim
        self.qk_rmsnorm = qk_rmsnorm

        self.prenorm = nn.RMSNorm(dim) if prenorm else nn.Identity()
        self.postnorm = nn.RMSNorm(dim) if postnorm else nn.Identity()
        if qk_rmsnorm:
            self.q_norm = nn.RMSNorm(dim_head)
            self.k_norms = nn.ModuleList(nn.RMSNorm(dim_head) for _ in range(self.kv_sets))
            self.v_norms = nn.ModuleList(nn.RMSNorm(dim_head_values) for _ in range(self.kv_sets))

        self.split_dims = (heads * dim_head,
                           self.kv_sets * key_value_heads * dim_head,
                           self.kv_sets * key_value_heads * dim_head_values)
        self.to_qkv = nn.Linear(dim, sum(self.split_dims), bias=False)
        self.combine_heads = nn.Linear(heads * dim_head_values, dim, bias=False)

        # more than two key/value sets go to the n-th order attend (simplicial_mha.py:94-98 of the reference, which
        # like this build refuses the causal flag there)
        assert not (causal and self.kv_sets > 2), 'the n-th order attend is used without a causal mask, as in the reference'
        if attend is None:
            attend = naive_two_simplicial_attend if self.kv_sets <= 2 else nth_order_attend
        if causal:
            attend = partial(attend, causal=causal)
        self.attend = attend

    def _split(self, t, heads):
        t = t.unflatten(-1, (heads, -1))                       # b n h d
        return t.transpose(1, 2) if self.head_first_dim else t

    # fused split + RMSNorm kernel for the layout the sliding-window module uses (GPU, bf16)
    fused_qkv_norm = True

    def _can_fuse(self, qkv):
        dh = self.split_dims[0] // self.heads
        return (self.fused_qkv_norm and self.qk_rmsnorm and self.kv_sets == 2 and not self.head_first_dim
                and qkv.is_cuda and qkv.dtype is torch.bfloat16 and dh in (32, 64, 128, 256)
                and self.split_dims[1] == self.split_dims[2]
                and all(n.eps == self.q_norm.eps for n in (*self.k_norms, *self.v_norms)))

    def forward(self, tokens):
        tokens = self.prenorm(tokens)
        qkv = self.to_qkv(tokens)
        if qkv.dim() == 3 and self._can_fuse(qkv):
            from .qkv_norm import fused_qkv_norm
            norms = (self.q_norm, *self.k_norms, *self.v_norms)
            q, k1, k2, v1, v2 = fused_qkv_norm(qkv, norms, self.heads, self.key_value_heads, self.split_dims[0] // self.heads)
            out = self.attend(q, (k1, k2), (v1, v2))
            return self.postnorm(self.combine_heads(out.flatten(-2)))
        q, k, v = qkv.split(self.split_dims, dim=-1)
        queries = self._split(q, self.heads)
        keys = self._split(k, self.key_value_heads).chunk(self.kv_sets, dim=-1)
        values = self._split(v, self.key_value_heads).chunk(self.kv_sets, dim=-1)
        if self.qk_rmsnorm:
            queries = self.q_norm(queries)
            keys = tuple(norm(t) for norm, t in zip(self.k_norms, keys))
            values = tuple(norm(t) for norm, t in zip(self.v_norms, values))
        out = self.attend(queries, keys, values)
        if self.head_first_dim:
            out = out.transpose(1, 2)
        out = self.combine_heads(out.flatten(-2))
        return self.postnorm(out)


class TwoSimplicialMHA(HigherOrderAttention):
    def __init__(self, *args, **kwargs):
        assert 'number_key_value_sets' not in kwargs
        super().__init__(*args, number_key_value_sets=2, **kwargs)
