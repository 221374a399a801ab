"""Dense (unwindowed) 2-simplicial attention in plain PyTorch.

Counterpart of ``naive_two_simplicial_attend`` of the reference
(simplicial_attention/simplicial_attention.py:78-127); it is the default ``attend``
of :class:`HigherOrderAttention` and is not part of the sliding-window hot path,
which always runs the HIP kernels.
"""
from __future__ import annotations

import torch
from torch import Tensor


def naive_two_simplicial_attend(q: Tensor, k, v, causal: bool = False) -> Tensor:
    """q: (b, h, i, d); k = (k1, k2): (b, hk, j, d); v = (v1, v2): (b, hk, j, dv) -> (b, h, i, dv)."""
    if len(k) != 2 or len(v) != 2:
        raise AssertionError('two key sets and two value sets are required')
    (k1, k2), (v1, v2) = k, v
    batch, heads, n, dim = q.shape
    kv_heads = k1.shape[1]
    assert heads % kv_heads == 0, 'query heads must be a multiple of key/value heads'
    grouped = (q * dim ** -0.5).unflatten(1, (kv_heads, heads // kv_heads))
    logits = torch.einsum('bhgid,bhjd,bhkd->bhgijk', grouped, k1, k2)
    if causal:
        assert logits.shape[-1] == logits.shape[-2] == n
        future = torch.ones(n, n, dtype=torch.bool, device=q.device).triu(1)
        logits = logits.masked_fill(future[:, :, None] | future[:, None, :], -torch.finfo(logits.dtype).max)
    weights = logits.flatten(-2).softmax(dim=-1).view_as(logits)
    mixed = torch.einsum('bhgijk,bhjd,bhkd->bhgid', weights, v1, v2)
    return mixed.flatten(1, 2)
