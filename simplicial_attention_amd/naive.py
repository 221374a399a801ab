"""Dense (unwindowed) higher-order attention in plain PyTorch.

Counterparts of ``signed_determinant``, ``naive_two_simplicial_attend`` and ``nth_order_attend`` of the
reference (simplicial_attention/simplicial_attention.py:36-76, 78-127, 131-198).  ``naive_two_simplicial_attend``
is the default ``attend`` of :class:`HigherOrderAttention` (``nth_order_attend`` for more than two key/value sets);
none of them is part of the sliding-window hot path, which always runs the HIP kernels.
"""
from __future__ import annotations

import torch
from torch import Tensor


def signed_determinant(q: Tensor, k1: Tensor, k2: Tensor) -> Tensor:
    """Similarity of simplicial_attention.py:36-76: the head dimension is read as triples and every triple contributes
    the 3 x 3 determinant det[q; k1; k2] = q . (k1 x k2); channels left over after the last full triple contribute
    their plain trilinear product.  q: (b, h, ..., i, d); k1, k2: (b, h, j, d) -> (b, h, ..., i, j, k)."""
    d3 = q.shape[-1] // 3 * 3
    qt, k1t, k2t = (t[..., :d3].unflatten(-1, (-1, 3)) for t in (q, k1, k2))
    roll = lambda t, s: torch.roll(t, shifts=s, dims=-1).flatten(-2)
    # sum_r q_r (k1_{r+1} k2_{r+2} - k1_{r+2} k2_{r+1}) over the cyclic index r of a triple
    plus = torch.einsum('bh...id,bhjd,bhkd->bh...ijk', q[..., :d3], roll(k1t, -1), roll(k2t, -2))
    minus = torch.einsum('bh...id,bhjd,bhkd->bh...ijk', q[..., :d3], roll(k1t, -2), roll(k2t, -1))
    sim = plus - minus
    if d3 < q.shape[-1]:
        sim = sim + torch.einsum('bh...id,bhjd,bhkd->bh...ijk', q[..., d3:], k1[..., d3:], k2[..., d3:])
    return sim


def naive_two_simplicial_attend(q: Tensor, k, v, causal: bool = False, use_signed_determinant: bool = False) -> Tensor:
    """q: (b, h, i, d); k = (k1, k2): (b, hk, j, d); v = (v1, v2): (b, hk, j, dv) -> (b, h, i, dv)."""
    if len(k) != 2 or len(v) != 2:
        raise AssertionError('two key sets and two value sets are required')
    (k1, k2), (v1, v2) = k, v
    batch, heads, n, dim = q.shape
    kv_heads = k1.shape[1]
    assert heads % kv_heads == 0, 'query heads must be a multiple of key/value heads'
    grouped = (q * dim ** -0.5).unflatten(1, (kv_heads, heads // kv_heads))
    if use_signed_determinant:
        logits = signed_determinant(grouped, k1, k2)
    else:
        logits = torch.einsum('bhgid,bhjd,bhkd->bhgijk', grouped, k1, k2)
    if causal:
        assert logits.shape[-1] == logits.shape[-2] == n
        future = torch.ones(n, n, dtype=torch.bool, device=q.device).triu(1)
        logits = logits.masked_fill(future[:, :, None] | future[:, None, :], -torch.finfo(logits.dtype).max)
    weights = logits.flatten(-2).softmax(dim=-1).view_as(logits)
    mixed = torch.einsum('bhgijk,bhjd,bhkd->bhgid', weights, v1, v2)
    return mixed.flatten(1, 2)


def nth_order_attend(q: Tensor, keys, values, causal: bool = False) -> Tensor:
    """Attention over n key/value sets (simplicial_attention.py:131-198): logits[i, j1..jn] = scale sum_d q_i k1_j1 ... kn_jn,
    one softmax over all (j1..jn), out_i = sum attn v1_j1 * ... * vn_jn.  q: (b, h, i, d); keys[x]: (b, hk, j, d);
    values[x]: (b, hk, j, dv) -> (b, h, i, dv).  ``causal`` masks every j_x > i."""
    n = len(keys)
    assert n == len(values) and 1 <= n <= 8
    batch, heads, seq, dim = q.shape
    kv_heads = keys[0].shape[1]
    assert heads % kv_heads == 0, 'query heads must be a multiple of key/value heads'
    grouped = (q * dim ** -0.5).unflatten(1, (kv_heads, heads // kv_heads))
    idx = 'jklmnopq'[:n]
    operands = ','.join(f'bh{c}d' for c in idx)
    logits = torch.einsum(f'bhgid,{operands}->bhgi{idx}', grouped, *keys)
    if causal:
        future = torch.ones(seq, keys[0].shape[-2], dtype=torch.bool, device=q.device).triu(1)
        mask = torch.zeros(logits.shape[3:], dtype=torch.bool, device=q.device)
        for x in range(n):
            shape = [seq] + [1] * n
            shape[1 + x] = future.shape[1]
            mask = mask | future.view(shape)
        logits = logits.masked_fill(mask, -torch.finfo(logits.dtype).max)
    weights = logits.flatten(4).softmax(dim=-1).view_as(logits)
    mixed = torch.einsum(f'bhgi{idx},{operands}->bhgid', weights, *values)
    return mixed.flatten(1, 2)
